// minGRU: a gated recurrence whose gates read the current token only,
//     z = sigmoid(zr + bz),  u = xr + bx,  c = u >= 0 ? u + 1/2 : sigmoid(u),
//     S_t = (1 - z) S_(t-1) + z c,          out_t = S_t * silu(g),
// element by element over `width` channels; zr | xr | g are the three thirds of a projected row. The
// state of each request lives in a slot of 32-bit floats: a step starts from it and leaves it advanced by
// the step's tokens. Gates, candidate, state and output are 32-bit; the output is rounded at the store.
//
// A workgroup takes 64 channels of one request. With one wave it walks the request's tokens of this step
// in order (decoded tokens, short portions). With several waves the tokens are cut into as many
// stretches: each wave first folds its stretch into the pair (A, B) with S_end = A S_start + B, the pairs
// are chained through LDS from the slot's state, and each wave then walks its stretch again from the
// state it starts at, by the same recurrence as the single wave: inside a stretch the sums are the plain
// walk's, only the state at a stretch's start is rounded differently.
//
// Long portions take two kernels instead, so that the whole chip works on them: the tokens are cut into
// chunks of GRU_CHUNK, one wave per (chunk, 64 channels, request). The first kernel folds every chunk
// into its pair (A, B) and sets the slot's state aside; the second chains the pairs of the chunks before
// its own from that state, walks its chunk by the recurrence and writes the outputs, and the request's
// last chunk leaves the new state in the slot.
#include "common.h"

#define GRU_LANES 64
#define GRU_MAX_WAVES 16

static __device__ __forceinline__ float gru_sigmoid(float v) { return 1.0f / (1.0f + expf(-v)); }
// 1 / (1 + e^-v): for 32-bit results the library's exponential and a true division; for results that are rounded
// to bfloat16 the hardware's 2^x and reciprocal, each good to a unit in the last place of 32 bits, at a third
// of the instructions (the scan is bound by them, not by memory)
template <typename TO> struct GruMath {
  static __device__ __forceinline__ float sigmoid(float v) { return 1.0f / (1.0f + expf(-v)); }
};
template <> struct GruMath<bf16_t> {
  static __device__ __forceinline__ float sigmoid(float v) {
    return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.44269504088896340736f * v));
  }
};

template <typename TI> struct GruIn;
template <> struct GruIn<float> { static __device__ __forceinline__ float ld(const float* p) { return *p; } };
template <> struct GruIn<bf16_t> { static __device__ __forceinline__ float ld(const bf16_t* p) { return bf2f(*p); } };

template <typename TI, typename TO>
__global__ void __launch_bounds__(GRU_LANES * GRU_MAX_WAVES)
mingru_scan_kernel(TO* __restrict__ out, const TI* __restrict__ zxg, const void* __restrict__ bias, int bias_code,
                   float* __restrict__ state, const int32_t* __restrict__ cu_seqlens,
                   const int32_t* __restrict__ state_slots, int width) {
  __shared__ float chain[GRU_MAX_WAVES][GRU_LANES][2];
  const int lane = threadIdx.x & (GRU_LANES - 1), wave = threadIdx.x / GRU_LANES, waves = blockDim.x / GRU_LANES;
  const int s = blockIdx.y, c = blockIdx.x * GRU_LANES + lane;
  const bool on = c < width;
  const int t0 = cu_seqlens[s], t1 = cu_seqlens[s + 1];
  const int stretch = (t1 - t0 + waves - 1) / waves;
  const int ta = min(t0 + wave * stretch, t1), tb = min(ta + stretch, t1);
  const int64_t row = 3 * (int64_t)width;
  float bz = 0.f, bx = 0.f;
  if (on && bias) {
    bz = bias_code == 0 ? ((const float*)bias)[c] : bf2f(((const bf16_t*)bias)[c]);
    bx = bias_code == 0 ? ((const float*)bias)[width + c] : bf2f(((const bf16_t*)bias)[width + c]);
  }
  float* slot = state + (int64_t)state_slots[s] * width;
  float S = on ? slot[c] : 0.f;
  if (waves > 1) {
    float A = 1.f, B = 0.f;
    if (on)
      for (int t = ta; t < tb; ++t) {
        const float z = GruMath<TO>::sigmoid(GruIn<TI>::ld(zxg + t * row + c) + bz);
        const float u = GruIn<TI>::ld(zxg + t * row + width + c) + bx;
        const float cand = u >= 0.f ? u + 0.5f : GruMath<TO>::sigmoid(u);
        const float keep = 1.0f - z;
        A *= keep;
        B = fmaf(keep, B, z * cand);
      }
    chain[wave][lane][0] = A;
    chain[wave][lane][1] = B;
    __syncthreads();
    for (int w = 0; w < wave; ++w) S = fmaf(chain[w][lane][0], S, chain[w][lane][1]);
  }
  if (on) {
    for (int t = ta; t < tb; ++t) {
      const float z = GruMath<TO>::sigmoid(GruIn<TI>::ld(zxg + t * row + c) + bz);
      const float u = GruIn<TI>::ld(zxg + t * row + width + c) + bx;
      const float g = GruIn<TI>::ld(zxg + t * row + 2 * width + c);
      const float cand = u >= 0.f ? u + 0.5f : GruMath<TO>::sigmoid(u);
      S = fmaf(1.0f - z, S, z * cand);
      Num<TO>::st(out + (int64_t)t * width + c, S * (g * GruMath<TO>::sigmoid(g)));
    }
    // the last wave ends at the step's last token (or, with an empty stretch, holds the chained state as it is)
    if (wave == waves - 1) slot[c] = S;
  }
}

#define GRU_CHUNK 32
#define GRU_THREADS 64

// VEC consecutive channels a thread (4 where the width is a multiple of 4 and rows are 16-byte aligned: a wave's
// load is then a kilobyte, and a thread walks four recurrences side by side)
template <typename TI, int VEC> struct GruRow;
template <typename TI> struct GruRow<TI, 1> {
  static __device__ __forceinline__ void ld(const TI* p, float* o) { o[0] = GruIn<TI>::ld(p); }
};
template <> struct GruRow<float, 4> {
  static __device__ __forceinline__ void ld(const float* p, float* o) {
    const float4 v = *(const float4*)p;
    o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w;
  }
};
template <> struct GruRow<bf16_t, 4> {
  static __device__ __forceinline__ void ld(const bf16_t* p, float* o) {
    const uint2 v = *(const uint2*)p;
    o[0] = __uint_as_float(v.x << 16); o[1] = __uint_as_float(v.x & 0xffff0000u);
    o[2] = __uint_as_float(v.y << 16); o[3] = __uint_as_float(v.y & 0xffff0000u);
  }
};

template <int VEC>
static __device__ __forceinline__ void gru_biases(const void* bias, int bias_code, int width, int c, float* bz, float* bx) {
#pragma unroll
  for (int i = 0; i < VEC; ++i) {
    bz[i] = bx[i] = 0.f;
    if (bias) {
      bz[i] = bias_code == 0 ? ((const float*)bias)[c + i] : bf2f(((const bf16_t*)bias)[c + i]);
      bx[i] = bias_code == 0 ? ((const float*)bias)[width + c + i] : bf2f(((const bf16_t*)bias)[width + c + i]);
    }
  }
}

// folds [requests, max_chunks, 2, width] and starts [requests, width] are the two kernels' scratch.
template <typename TI, typename TO, int VEC>
__global__ void __launch_bounds__(GRU_THREADS)
mingru_fold_kernel(float* __restrict__ folds, float* __restrict__ starts, const TI* __restrict__ zxg,
                   const void* __restrict__ bias, int bias_code, const float* __restrict__ state,
                   const int32_t* __restrict__ cu_seqlens, const int32_t* __restrict__ state_slots, int width,
                   int max_chunks) {
  const int c = (blockIdx.x * GRU_THREADS + threadIdx.x) * VEC, chunk = blockIdx.y, s = blockIdx.z;
  const int t0 = cu_seqlens[s], t1 = cu_seqlens[s + 1];
  const int ta = t0 + chunk * GRU_CHUNK, tb = min(ta + GRU_CHUNK, t1);
  if (c >= width || ta >= t1) return;
  if (chunk == 0)
#pragma unroll
    for (int i = 0; i < VEC; ++i) starts[(int64_t)s * width + c + i] = state[(int64_t)state_slots[s] * width + c + i];
  const int64_t row = 3 * (int64_t)width;
  float bz[VEC], bx[VEC], A[VEC], B[VEC];
  gru_biases<VEC>(bias, bias_code, width, c, bz, bx);
#pragma unroll
  for (int i = 0; i < VEC; ++i) { A[i] = 1.f; B[i] = 0.f; }
#pragma unroll 4
  for (int t = ta; t < tb; ++t) {
    float zr[VEC], xr[VEC];
    GruRow<TI, VEC>::ld(zxg + t * row + c, zr);
    GruRow<TI, VEC>::ld(zxg + t * row + width + c, xr);
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      const float z = GruMath<TO>::sigmoid(zr[i] + bz[i]);
      const float u = xr[i] + bx[i];
      const float cand = u >= 0.f ? u + 0.5f : GruMath<TO>::sigmoid(u);
      const float keep = 1.0f - z;
      A[i] *= keep;
      B[i] = fmaf(keep, B[i], z * cand);
    }
  }
  float* f = folds + ((int64_t)s * max_chunks + chunk) * 2 * width + c;
#pragma unroll
  for (int i = 0; i < VEC; ++i) { f[i] = A[i]; f[width + i] = B[i]; }
}

template <typename TI, typename TO, int VEC>
__global__ void __launch_bounds__(GRU_THREADS)
mingru_walk_kernel(TO* __restrict__ out, const float* __restrict__ folds, const float* __restrict__ starts,
                   const TI* __restrict__ zxg, const void* __restrict__ bias, int bias_code, float* __restrict__ state,
                   const int32_t* __restrict__ cu_seqlens, const int32_t* __restrict__ state_slots, int width,
                   int max_chunks) {
  const int c = (blockIdx.x * GRU_THREADS + threadIdx.x) * VEC, chunk = blockIdx.y, s = blockIdx.z;
  const int t0 = cu_seqlens[s], t1 = cu_seqlens[s + 1];
  const int ta = t0 + chunk * GRU_CHUNK, tb = min(ta + GRU_CHUNK, t1);
  if (c >= width || ta >= t1) return;
  const int64_t row = 3 * (int64_t)width;
  float bz[VEC], bx[VEC], S[VEC];
  gru_biases<VEC>(bias, bias_code, width, c, bz, bx);
  GruRow<float, VEC>::ld(starts + (int64_t)s * width + c, S);
  const float* f = folds + (int64_t)s * max_chunks * 2 * width + c;
#pragma unroll 8
  for (int k = 0; k < chunk; ++k) {       // (the pairs do not depend on S: their loads run ahead of the chain)
    float A[VEC], B[VEC];
    GruRow<float, VEC>::ld(f + (int64_t)k * 2 * width, A);
    GruRow<float, VEC>::ld(f + (int64_t)k * 2 * width + width, B);
#pragma unroll
    for (int i = 0; i < VEC; ++i) S[i] = fmaf(A[i], S[i], B[i]);
  }
#pragma unroll 4
  for (int t = ta; t < tb; ++t) {
    float zr[VEC], xr[VEC], gr[VEC];
    GruRow<TI, VEC>::ld(zxg + t * row + c, zr);
    GruRow<TI, VEC>::ld(zxg + t * row + width + c, xr);
    GruRow<TI, VEC>::ld(zxg + t * row + 2 * width + c, gr);
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      const float z = GruMath<TO>::sigmoid(zr[i] + bz[i]);
      const float u = xr[i] + bx[i];
      const float cand = u >= 0.f ? u + 0.5f : GruMath<TO>::sigmoid(u);
      S[i] = fmaf(1.0f - z, S[i], z * cand);
      Num<TO>::st(out + (int64_t)t * width + c + i, S[i] * (gr[i] * GruMath<TO>::sigmoid(gr[i])));
    }
  }
  if (tb == t1)                                             // the request's last chunk
#pragma unroll
    for (int i = 0; i < VEC; ++i) state[(int64_t)state_slots[s] * width + c + i] = S[i];
}

// `longest`: the most tokens a request feeds (the grid's chunks); folds: 2 * requests * chunks * width floats,
// starts: requests * width floats, chunks = ceil(longest / GRU_CHUNK).
extern "C" int ts_mingru_scan_chunks(void* out, int out_dtype, const void* zxg, int in_dtype, const void* bias, int bias_dtype,
                                     float* state, float* folds, float* starts, const int32_t* cu_seqlens,
                                     const int32_t* state_slots, int num_seqs, int width, int longest, hipStream_t stream) {
  if (num_seqs <= 0 || longest <= 0) return TS_OK;
  const int chunks = (longest + GRU_CHUNK - 1) / GRU_CHUNK;
  if (width <= 0 || num_seqs > 65535 || chunks > 65535 || !folds || !starts) return TS_BAD_SHAPE;
  if (bias_dtype != 0 && bias_dtype != 1) return TS_BAD_DTYPE;
  // four channels a thread only where that still leaves every SIMD of the chip several waves
  const bool by4 = width % 4 == 0 && (((uintptr_t)zxg | (uintptr_t)folds | (uintptr_t)starts) & 15) == 0 &&
                   (int64_t)((width / 4 + GRU_THREADS - 1) / GRU_THREADS) * chunks * num_seqs >= 4096;
  const int per = by4 ? 4 : 1;
  dim3 grid((width / per + GRU_THREADS - 1) / GRU_THREADS, chunks, num_seqs);
#define GRU_CHUNKS_V(TI, TO, VV) \
  mingru_fold_kernel<TI, TO, VV><<<grid, GRU_THREADS, 0, stream>>>(folds, starts, (const TI*)zxg, bias, bias_dtype, state, cu_seqlens, \
                                                               state_slots, width, chunks); \
  mingru_walk_kernel<TI, TO, VV><<<grid, GRU_THREADS, 0, stream>>>((TO*)out, folds, starts, (const TI*)zxg, bias, bias_dtype, state, \
                                                                   cu_seqlens, state_slots, width, chunks)
#define GRU_CHUNKS(TI, TO) if (by4) { GRU_CHUNKS_V(TI, TO, 4); } else { GRU_CHUNKS_V(TI, TO, 1); }
  if (in_dtype == 0 && out_dtype == 0) { GRU_CHUNKS(float, float) }
  else if (in_dtype == 0 && out_dtype == 1) { GRU_CHUNKS(float, bf16_t) }
  else if (in_dtype == 1 && out_dtype == 1) { GRU_CHUNKS(bf16_t, bf16_t) }
  else if (in_dtype == 1 && out_dtype == 0) { GRU_CHUNKS(bf16_t, float) }
  else return TS_BAD_DTYPE;
#undef GRU_CHUNKS
#undef GRU_CHUNKS_V
  return ts_check_launch();
}

extern "C" int ts_mingru_scan(void* out, int out_dtype, const void* zxg, int in_dtype, const void* bias, int bias_dtype,
                              float* state, const int32_t* cu_seqlens, const int32_t* state_slots, int num_seqs,
                              int width, int waves, hipStream_t stream) {
  if (num_seqs <= 0) return TS_OK;
  if (width <= 0 || waves < 1 || waves > GRU_MAX_WAVES || num_seqs > 65535) return TS_BAD_SHAPE;
  if (bias_dtype != 0 && bias_dtype != 1) return TS_BAD_DTYPE;
  dim3 grid((width + GRU_LANES - 1) / GRU_LANES, num_seqs), block(GRU_LANES * waves);
#define GRU_LAUNCH(TI, TO) \
  mingru_scan_kernel<TI, TO><<<grid, block, 0, stream>>>((TO*)out, (const TI*)zxg, bias, bias_dtype, state, cu_seqlens, \
                                                        state_slots, width)
  if (in_dtype == 0 && out_dtype == 0) GRU_LAUNCH(float, float);
  else if (in_dtype == 0 && out_dtype == 1) GRU_LAUNCH(float, bf16_t);
  else if (in_dtype == 1 && out_dtype == 1) GRU_LAUNCH(bf16_t, bf16_t);
  else if (in_dtype == 1 && out_dtype == 0) GRU_LAUNCH(bf16_t, float);
  else return TS_BAD_DTYPE;
#undef GRU_LAUNCH
  return ts_check_launch();
}
