// What lies between a q|k|v projection and the cache for mixers whose projected rows first pass a short causal
// convolution over time, channel by channel:
//   y_t[c] = sum_j w[c][j] u_(t - taps + 1 + j)[c],    j = 0 .. taps - 1,
// with zeros before a request's first token. The last taps - 1 projected rows of every request are its state
// ([slots, taps - 1, channels], oldest first, zero at admission): a step's first tokens reach back into it.
//   * `ts_conv_finish`: the convolution; then, optionally, every q and k head divided by its root mean square
//     and scaled by a weight shared by all heads; q times 1 + coef ln(floor((p + 1) / every) + 1) at position p
//     (coef 0: not); q goes to [tokens, heads, dim], k and v to their cache slots. Key and value heads may
//     differ in size; a mixer that reads another's cache has q channels only (nkv = 0).
//   * `ts_conv_state_update`: after it, the state moves on by the step's rows (its own launch, so that no row
//     of the state is overwritten while a token of the step still reads it).
// Everything is 32-bit up to the store.
#include "common.h"

#define SC_WAVES 4
#define SC_MAX_HD 256
#define SC_MAX_TAPS 16
#define SC_LONG_STEP 256      // tokens from which a step's heads and values take the kernels of 16-byte pieces and tiles

template <typename TI, typename TO>
__global__ void __launch_bounds__(SC_WAVES * TS_WAVE)
conv_finish_kernel(TO* __restrict__ q_out, TO* __restrict__ k_cache, TO* __restrict__ v_cache, const TI* __restrict__ proj,
                   int64_t row_stride, const float* __restrict__ conv_w, float* state,
                   const float* __restrict__ q_norm_w, const float* __restrict__ k_norm_w, float eps,
                   const int32_t* __restrict__ positions, const int32_t* __restrict__ seq_of_token,
                   const int32_t* __restrict__ cu_seqlens, const int32_t* __restrict__ state_slots,
                   const int32_t* __restrict__ slots, int nh, int nkv, int hd, int vd_size, int taps, float temp_coef,
                   int temp_every, int page_size, int64_t kp, int64_t ks, int64_t kh, int64_t vp, int64_t vs, int64_t vh,
                   int64_t vd, int num_tokens, int with_values, int moves_state) {
  const int wave = threadIdx.x / TS_WAVE, lane = threadIdx.x & (TS_WAVE - 1);
  const int heads = nh + (with_values ? 2 : 1) * nkv;       // (without: the values go through `conv_values_kernel`)
  const int64_t item = (int64_t)blockIdx.x * SC_WAVES + wave;  // a wave per (token, head)
  if (item >= (int64_t)num_tokens * heads) return;
  const int t = (int)(item / heads), h = (int)(item - (int64_t)t * heads);
  const int channels = (nh + nkv) * hd + nkv * vd_size;
  const int pos = positions[t];
  const int seq = seq_of_token[t];
  const int first = cu_seqlens[seq];                   // the step's first token of this request
  const int local = t - first;                         // tokens of the step before this one
  float* st = taps > 1 ? state + (int64_t)state_slots[seq] * (taps - 1) * channels : nullptr;
  const int slot = slots ? slots[t] : -1;
  const bool stores = slot >= 0 && k_cache;
  const int page = stores ? slot / page_size : 0, off = stores ? slot - page * page_size : 0;
  float temp = 1.0f;
  if (temp_coef != 0.f) temp = 1.0f + temp_coef * logf((float)((pos + 1) / temp_every) + 1.0f);
  {
    const bool is_q = h < nh, is_v = h >= nh + nkv;
    if (!is_q && !stores) return;
    const int size = is_v ? vd_size : hd;
    const int c0 = is_v ? (nh + nkv) * hd + (h - nh - nkv) * vd_size : h * hd;
    float y[SC_MAX_HD / TS_WAVE];
    float squares = 0.f;
#pragma unroll
    for (int i = 0; i < SC_MAX_HD / TS_WAVE; ++i) {
      const int d = lane + i * TS_WAVE;
      float acc = 0.f;
      if (d < size) {
        const int c = c0 + d;
        for (int j = 0; j < taps; ++j) {
          const int back = taps - 1 - j;                // rows before this token
          float u;
          if (back <= local) u = Num<TI>::ld(proj + (int64_t)(t - back) * row_stride + c);
          else u = st[(int64_t)(taps - 1 - (back - local)) * channels + c];
          acc = fmaf(conv_w[(int64_t)c * taps + j], u, acc);
          // a step of single tokens: this thread alone reads the channel's past rows, and moves them on by the
          // token's own row as it goes (row j - 1 has been read when row j is written over it)
          if (moves_state && j > 0) st[(int64_t)(j - 1) * channels + c] = u;
        }
      }
      y[i] = acc;
      squares = fmaf(acc, acc, squares);
    }
    const float* nw = is_v ? nullptr : (is_q ? q_norm_w : k_norm_w);
    float scale = 1.0f;
    if (nw) scale = 1.0f / sqrtf(wave_sum(squares) / (float)size + eps);
    if (is_q) scale *= temp;
    TO* dst = is_q ? q_out + ((int64_t)t * nh + h) * hd
              : !is_v ? k_cache + page * kp + off * ks + (int64_t)(h - nh) * kh
                      : v_cache + page * vp + off * vs + (int64_t)(h - nh - nkv) * vh;
    const int64_t step = is_v ? vd : 1;
#pragma unroll
    for (int i = 0; i < SC_MAX_HD / TS_WAVE; ++i) {
      const int d = lane + i * TS_WAVE;
      if (d < size) Num<TO>::st(dst + (int64_t)d * step, y[i] * scale * (nw ? nw[d] : 1.0f));
    }
  }
}

// The same for the q and k heads of steps of many tokens, where head sizes are multiples of eight: a thread takes
// eight consecutive channels of a head (32 or 16 bytes a load, 16 a store), the threads of a head sit side by side
// in a wave (a power of two of them, the last ones idle where the head's eighths are no power of two) and add
// their squares by exchanging registers. TAPS > 0: the taps are known when the kernel is compiled.
#define SC_PIECE 8
#define SC_VEC_THREADS 256

template <typename T> struct ScRow;
template <> struct ScRow<float> {
  static __device__ __forceinline__ void ld(const float* p, float (&u)[SC_PIECE]) {
    const float4 a = *(const float4*)p, b = *(const float4*)(p + 4);
    u[0] = a.x; u[1] = a.y; u[2] = a.z; u[3] = a.w; u[4] = b.x; u[5] = b.y; u[6] = b.z; u[7] = b.w;
  }
  static __device__ __forceinline__ void st(float* p, const float (&y)[SC_PIECE]) {
    *(float4*)p = make_float4(y[0], y[1], y[2], y[3]);
    *(float4*)(p + 4) = make_float4(y[4], y[5], y[6], y[7]);
  }
};
template <> struct ScRow<bf16_t> {
  static __device__ __forceinline__ void ld(const bf16_t* p, float (&u)[SC_PIECE]) {
    const uint4 a = *(const uint4*)p;
    const uint32_t v[4] = {a.x, a.y, a.z, a.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      u[2 * i] = __uint_as_float(v[i] << 16);
      u[2 * i + 1] = __uint_as_float(v[i] & 0xffff0000u);
    }
  }
  static __device__ __forceinline__ void st(bf16_t* p, const float (&y)[SC_PIECE]) {
    uint4 a;
    a.x = (uint32_t)f2bf(y[0]) | ((uint32_t)f2bf(y[1]) << 16);
    a.y = (uint32_t)f2bf(y[2]) | ((uint32_t)f2bf(y[3]) << 16);
    a.z = (uint32_t)f2bf(y[4]) | ((uint32_t)f2bf(y[5]) << 16);
    a.w = (uint32_t)f2bf(y[6]) | ((uint32_t)f2bf(y[7]) << 16);
    *(uint4*)p = a;
  }
};

// Eight consecutive channels from c of token t's convolution; `local`: tokens of the step before it, `st`: its
// request's state rows.
template <typename TI, int TAPS>
__device__ __forceinline__ void sc_conv_piece(float (&y)[SC_PIECE], const TI* __restrict__ proj, int64_t row_stride,
                                              const float* __restrict__ conv_w, const float* __restrict__ st, int channels,
                                              int taps, int t, int local, int c) {
  if constexpr (TAPS > 0) {
    // every row and every weight asked for before the first is used
    float u[TAPS][SC_PIECE], wv[SC_PIECE * TAPS];
#pragma unroll
    for (int j = 0; j < TAPS; ++j) {
      const int back = TAPS - 1 - j;
      if (back <= local) ScRow<TI>::ld(proj + (int64_t)(t - back) * row_stride + c, u[j]);
      else ScRow<float>::ld(st + (int64_t)(TAPS - 1 - (back - local)) * channels + c, u[j]);
    }
#pragma unroll
    for (int i = 0; i < SC_PIECE * TAPS / 4; ++i) {
      const float4 a = *(const float4*)(conv_w + (int64_t)c * TAPS + 4 * i);
      wv[4 * i] = a.x; wv[4 * i + 1] = a.y; wv[4 * i + 2] = a.z; wv[4 * i + 3] = a.w;
    }
#pragma unroll
    for (int j = 0; j < TAPS; ++j)
#pragma unroll
      for (int i = 0; i < SC_PIECE; ++i) y[i] = fmaf(wv[i * TAPS + j], u[j][i], y[i]);
  } else {
    for (int j = 0; j < taps; ++j) {
      const int back = taps - 1 - j;
      float u[SC_PIECE];
      if (back <= local) ScRow<TI>::ld(proj + (int64_t)(t - back) * row_stride + c, u);
      else ScRow<float>::ld(st + (int64_t)(taps - 1 - (back - local)) * channels + c, u);
#pragma unroll
      for (int i = 0; i < SC_PIECE; ++i) y[i] = fmaf(conv_w[(int64_t)(c + i) * taps + j], u[i], y[i]);
    }
  }
}

template <typename TI, typename TO, int TAPS>
__global__ void __launch_bounds__(SC_VEC_THREADS)
conv_finish_vec_kernel(TO* __restrict__ q_out, TO* __restrict__ k_cache, const TI* __restrict__ proj, int64_t row_stride,
                       const float* __restrict__ conv_w, const float* __restrict__ state, const float* __restrict__ q_norm_w,
                       const float* __restrict__ k_norm_w, float eps, const int32_t* __restrict__ positions,
                       const int32_t* __restrict__ seq_of_token, const int32_t* __restrict__ cu_seqlens,
                       const int32_t* __restrict__ state_slots, const int32_t* __restrict__ slots, int nh, int nkv, int hd,
                       int channels, int taps_arg, float temp_coef, int temp_every, int page_size, int64_t kp, int64_t ks,
                       int64_t kh, int num_tokens, int group, int group_shift) {
  const int taps = TAPS > 0 ? TAPS : taps_arg;
  const int heads = nh + (k_cache ? nkv : 0);
  const int64_t gid = (int64_t)blockIdx.x * SC_VEC_THREADS + threadIdx.x;
  const int64_t head_item = gid >> group_shift;              // (token, head): all its threads leave together
  const int piece = (int)(gid & (group - 1));
  if (head_item >= (int64_t)num_tokens * heads) return;
  const int t = (int)(head_item / heads), h = (int)(head_item - (int64_t)t * heads);
  const bool is_q = h < nh;
  const int slot = slots ? slots[t] : -1;
  if (!is_q && slot < 0) return;
  const bool active = piece * SC_PIECE < hd;
  const int seq = seq_of_token[t];
  const int local = t - cu_seqlens[seq];
  const int c = h * hd + (active ? piece : 0) * SC_PIECE;
  float y[SC_PIECE];
#pragma unroll
  for (int i = 0; i < SC_PIECE; ++i) y[i] = 0.f;
  if (active)
    sc_conv_piece<TI, TAPS>(y, proj, row_stride, conv_w, taps > 1 ? state + (int64_t)state_slots[seq] * (taps - 1) * channels : nullptr,
                            channels, taps, t, local, c);
  const float* nw = is_q ? q_norm_w : k_norm_w;
  float scale = 1.0f;
  if (nw) {
    float squares = 0.f;
#pragma unroll
    for (int i = 0; i < SC_PIECE; ++i) squares = fmaf(y[i], y[i], squares);
    for (int d = group >> 1; d > 0; d >>= 1) squares += __shfl_xor(squares, d, TS_WAVE);
    scale = 1.0f / sqrtf(squares / (float)hd + eps);
  }
  if (!active) return;
  if (is_q && temp_coef != 0.f) scale *= 1.0f + temp_coef * logf((float)((positions[t] + 1) / temp_every) + 1.0f);
#pragma unroll
  for (int i = 0; i < SC_PIECE; ++i) y[i] = y[i] * scale * (nw ? nw[piece * SC_PIECE + i] : 1.0f);
  TO* dst;
  if (is_q) dst = q_out + ((int64_t)t * nh + h) * hd;
  else {
    const int page = slot / page_size, off = slot - page * page_size;
    dst = k_cache + page * kp + off * ks + (int64_t)(h - nh) * kh;
  }
  ScRow<TO>::st(dst + piece * SC_PIECE, y);
}

// The values of SC_VTOK consecutive tokens of one key/value head, through LDS: the convolution is taken with the
// lanes along a row's dimensions, and the rows are written with the lanes along the tokens, so that tokens in
// consecutive slots of a page (whose values lie side by side there, pages holding values transposed) leave in
// whole segments.
#define SC_VTOK 32
template <typename TI, typename TO>
__global__ void __launch_bounds__(SC_WAVES * TS_WAVE)
conv_values_kernel(TO* __restrict__ v_cache, const TI* __restrict__ proj, int64_t row_stride, const float* __restrict__ conv_w,
                   const float* __restrict__ state, const int32_t* __restrict__ seq_of_token,
                   const int32_t* __restrict__ cu_seqlens, const int32_t* __restrict__ state_slots,
                   const int32_t* __restrict__ slots, int num_tokens, int channels, int v_first, int vd_size, int taps,
                   int page_size, int64_t vp, int64_t vs, int64_t vh, int64_t vd) {
  __shared__ float rows_s[SC_VTOK][SC_MAX_HD + 1];
  __shared__ int slot_s[SC_VTOK], local_s[SC_VTOK], state_s[SC_VTOK];
  const int t0 = blockIdx.x * SC_VTOK, g = blockIdx.y;
  const int nt = min(SC_VTOK, num_tokens - t0);
  if (threadIdx.x < nt) {
    const int t = t0 + threadIdx.x, seq = seq_of_token[t];
    slot_s[threadIdx.x] = slots[t];
    local_s[threadIdx.x] = t - cu_seqlens[seq];
    state_s[threadIdx.x] = state_slots[seq];
  }
  __syncthreads();
  const int c0 = v_first + g * vd_size;
  for (int i = threadIdx.x; i < nt * vd_size; i += SC_WAVES * TS_WAVE) {
    const int tl = i / vd_size, d = i - tl * vd_size;
    const int c = c0 + d, t = t0 + tl, local = local_s[tl];
    float acc = 0.f;
    for (int j = 0; j < taps; ++j) {
      const int back = taps - 1 - j;
      float u;
      if (back <= local) u = Num<TI>::ld(proj + (int64_t)(t - back) * row_stride + c);
      else u = state[((int64_t)state_s[tl] * (taps - 1) + (taps - 1 - (back - local))) * channels + c];
      acc = fmaf(conv_w[(int64_t)c * taps + j], u, acc);
    }
    rows_s[tl][d] = acc;
  }
  __syncthreads();
  for (int i = threadIdx.x; i < vd_size * SC_VTOK; i += SC_WAVES * TS_WAVE) {
    const int d = i / SC_VTOK, tl = i - d * SC_VTOK;
    if (tl >= nt) continue;
    const int slot = slot_s[tl];
    if (slot < 0) continue;
    const int page = slot / page_size, off = slot - page * page_size;
    Num<TO>::st(v_cache + page * vp + off * vs + (int64_t)g * vh + (int64_t)d * vd, rows_s[tl][d]);
  }
}

// The same in 16-byte pieces, where a value head is whole eighths and the cache keeps a page's slots side by side:
// a thread convolves eight channels of a token, and writes eight tokens of a channel, in one store where their
// slots are eight in a row from a multiple of eight.
template <typename TI, typename TO, int TAPS>
__global__ void __launch_bounds__(SC_VEC_THREADS)
conv_values_vec_kernel(TO* __restrict__ v_cache, const TI* __restrict__ proj, int64_t row_stride, const float* __restrict__ conv_w,
                       const float* __restrict__ state, const int32_t* __restrict__ seq_of_token,
                       const int32_t* __restrict__ cu_seqlens, const int32_t* __restrict__ state_slots,
                       const int32_t* __restrict__ slots, int num_tokens, int channels, int v_first, int vd_size, int taps_arg,
                       int page_size, int64_t vp, int64_t vh, int64_t vd) {
  __shared__ float rows_s[SC_VTOK][SC_MAX_HD + 1];
  __shared__ int slot_s[SC_VTOK], local_s[SC_VTOK], state_s[SC_VTOK];
  const int taps = TAPS > 0 ? TAPS : taps_arg;
  const int t0 = blockIdx.x * SC_VTOK, g = blockIdx.y;
  const int nt = min(SC_VTOK, num_tokens - t0);
  if (threadIdx.x < SC_VTOK) {
    const int t = t0 + threadIdx.x;
    const int seq = threadIdx.x < nt ? seq_of_token[t] : 0;
    slot_s[threadIdx.x] = threadIdx.x < nt ? slots[t] : -1;
    local_s[threadIdx.x] = threadIdx.x < nt ? t - cu_seqlens[seq] : 0;
    state_s[threadIdx.x] = threadIdx.x < nt ? state_slots[seq] : 0;
  }
  __syncthreads();
  const int c0 = v_first + g * vd_size, pieces = vd_size / SC_PIECE;
  for (int i = threadIdx.x; i < nt * pieces; i += SC_VEC_THREADS) {
    const int tl = i / pieces, piece = i - tl * pieces;
    float y[SC_PIECE];
#pragma unroll
    for (int k = 0; k < SC_PIECE; ++k) y[k] = 0.f;
    sc_conv_piece<TI, TAPS>(y, proj, row_stride, conv_w, taps > 1 ? state + (int64_t)state_s[tl] * (taps - 1) * channels : nullptr,
                            channels, taps, t0 + tl, local_s[tl], c0 + piece * SC_PIECE);
#pragma unroll
    for (int k = 0; k < SC_PIECE; ++k) rows_s[tl][piece * SC_PIECE + k] = y[k];
  }
  __syncthreads();
  constexpr int RUNS = SC_VTOK / SC_PIECE;                 // runs of eight tokens
  for (int i = threadIdx.x; i < vd_size * RUNS; i += SC_VEC_THREADS) {
    const int d = i / RUNS, run = i - d * RUNS, tl0 = run * SC_PIECE;
    if (tl0 >= nt) continue;
    const int first = slot_s[tl0];
    bool row = first >= 0 && first % SC_PIECE == 0 && first % page_size + SC_PIECE <= page_size && tl0 + SC_PIECE <= nt;
#pragma unroll
    for (int k = 1; k < SC_PIECE; ++k) row = row && slot_s[min(tl0 + k, SC_VTOK - 1)] == first + k;
    if (row) {
      float y[SC_PIECE];
#pragma unroll
      for (int k = 0; k < SC_PIECE; ++k) y[k] = rows_s[tl0 + k][d];
      const int page = first / page_size, off = first - page * page_size;
      ScRow<TO>::st(v_cache + page * vp + off + (int64_t)g * vh + (int64_t)d * vd, y);
    } else {
      for (int k = 0; k < SC_PIECE && tl0 + k < nt; ++k) {
        const int slot = slot_s[tl0 + k];
        if (slot < 0) continue;
        const int page = slot / page_size, off = slot - page * page_size;
        Num<TO>::st(v_cache + page * vp + off + (int64_t)g * vh + (int64_t)d * vd, rows_s[tl0 + k][d]);
      }
    }
  }
}

// A thread per (request of the step, channel): row i of the new state is the row that lies taps - 1 - i rows
// before the end of (old state rows, the step's rows). Ascending i reads only rows not yet overwritten.
template <typename TI>
__global__ void __launch_bounds__(SC_WAVES * TS_WAVE)
conv_state_update_kernel(float* __restrict__ state, const TI* __restrict__ proj, int64_t row_stride,
                         const int32_t* __restrict__ cu_seqlens, const int32_t* __restrict__ state_slots, int num_seqs,
                         int channels, int taps) {
  const int64_t gid = (int64_t)blockIdx.x * (SC_WAVES * TS_WAVE) + threadIdx.x;
  if (gid >= (int64_t)num_seqs * channels) return;
  const int seq = (int)(gid / channels), c = (int)(gid - (int64_t)seq * channels);
  const int first = cu_seqlens[seq], n = cu_seqlens[seq + 1] - first;
  if (n <= 0) return;
  float* st = state + (int64_t)state_slots[seq] * (taps - 1) * channels;
  for (int i = 0; i < taps - 1; ++i) {
    const int src = n - (taps - 1) + i;                 // index among the step's rows; below 0: still an old row
    const float v = src >= 0 ? Num<TI>::ld(proj + (int64_t)(first + src) * row_stride + c) : st[(int64_t)(i + n) * channels + c];
    st[(int64_t)i * channels + c] = v;
  }
}

extern "C" int ts_conv_finish(void* q_out, void* k_cache, void* v_cache, const void* proj, int64_t row_stride,
                              const float* conv_w, float* state, const float* q_norm_w, const float* k_norm_w, float eps,
                              const int32_t* positions, const int32_t* seq_of_token, const int32_t* cu_seqlens,
                              const int32_t* state_slots, const int32_t* slots, int num_tokens, int nh, int nkv, int hd,
                              int vd_size, int taps, float temp_coef, int temp_every, int page_size, int64_t kp, int64_t ks,
                              int64_t kh, int64_t vp, int64_t vs, int64_t vh, int64_t vd, int in_dtype, int out_dtype,
                              int moves_state, hipStream_t stream) {
  if (num_tokens <= 0) return TS_OK;
  // (the state moves on inside this launch only where every request of the step feeds one token and the kernel of
  // a wave per head takes all channels: the caller asks for it on those steps alone)
  if (moves_state && (num_tokens >= SC_LONG_STEP || taps < 2)) return TS_BAD_SHAPE;
  if (hd <= 0 || hd > SC_MAX_HD || vd_size <= 0 || vd_size > SC_MAX_HD || nh <= 0 || nkv < 0 || taps < 1 || taps > SC_MAX_TAPS ||
      page_size <= 0 || (taps > 1 && !state) || (temp_coef != 0.f && temp_every <= 0) ||
      row_stride < (int64_t)(nh + nkv) * hd + (int64_t)nkv * vd_size)
    return TS_BAD_SHAPE;
  // several tokens of a step: their values leave through the tile kernel (a few tokens', with their heads)
  const int v_tiles = k_cache && nkv > 0 && num_tokens >= SC_LONG_STEP && nkv <= 65535;
  const int heads = nh + (v_tiles ? 1 : 2) * nkv;
  const int64_t blocks = ((int64_t)num_tokens * heads + SC_WAVES - 1) / SC_WAVES;
  if (blocks > 0x7fffffff) return TS_BAD_SHAPE;
  const int channels = (nh + nkv) * hd + nkv * vd_size;
  dim3 v_grid((num_tokens + SC_VTOK - 1) / SC_VTOK, nkv > 0 ? nkv : 1);
  // steps of many tokens whose rows and heads are whole 16-byte pieces: q and k through the kernel of eight
  // channels a thread, the values through the tile kernel
  const int in_piece = in_dtype == 0 ? 4 : 8;
  const bool aligned = hd % SC_PIECE == 0 && row_stride % in_piece == 0 && channels % 4 == 0 && kp % 8 == 0 && ks % 8 == 0 &&
                       kh % 8 == 0 && (((uintptr_t)q_out | (uintptr_t)k_cache | (uintptr_t)proj | (uintptr_t)conv_w |
                                        (uintptr_t)state | (uintptr_t)q_norm_w | (uintptr_t)k_norm_w) & 15) == 0;
  if (aligned && num_tokens >= SC_LONG_STEP && (v_tiles || nkv == 0 || !k_cache)) {
    int group = 1, group_shift = 0;
    while (group * SC_PIECE < hd) group *= 2, ++group_shift;
    const int vec_heads = nh + (k_cache ? nkv : 0);
    const int64_t vec_blocks = ((int64_t)num_tokens * vec_heads * group + SC_VEC_THREADS - 1) / SC_VEC_THREADS;
    if (vec_blocks > 0x7fffffff) return TS_BAD_SHAPE;
#define SC_VEC(TI, TO, TAPS) \
    conv_finish_vec_kernel<TI, TO, TAPS><<<(unsigned)vec_blocks, SC_VEC_THREADS, 0, stream>>>( \
        (TO*)q_out, (TO*)k_cache, (const TI*)proj, row_stride, conv_w, state, q_norm_w, k_norm_w, eps, positions, seq_of_token, \
        cu_seqlens, state_slots, slots, nh, nkv, hd, channels, taps, temp_coef, temp_every, page_size, kp, ks, kh, num_tokens, \
        group, group_shift)
#define SC_VAL(TI, TO, TAPS) \
    conv_values_vec_kernel<TI, TO, TAPS><<<v_grid, SC_VEC_THREADS, 0, stream>>>( \
        (TO*)v_cache, (const TI*)proj, row_stride, conv_w, state, seq_of_token, cu_seqlens, state_slots, slots, num_tokens, \
        channels, (nh + nkv) * hd, vd_size, taps, page_size, vp, vh, vd)
    // (values whose heads are whole eighths, in a cache whose pages keep their slots side by side)
    const bool v_pieces = vd_size % SC_PIECE == 0 && vs == 1 && page_size % SC_PIECE == 0 && vp % 8 == 0 && vh % 8 == 0 &&
                          vd % 8 == 0 && ((uintptr_t)v_cache & 15) == 0;
#define SC_VEC_TAPS(TI, TO) \
    do { \
      if (taps == 4) SC_VEC(TI, TO, 4); else if (taps == 3) SC_VEC(TI, TO, 3); else if (taps == 2) SC_VEC(TI, TO, 2); \
      else SC_VEC(TI, TO, 0); \
      if (v_tiles && v_pieces) { \
        if (taps == 4) SC_VAL(TI, TO, 4); else if (taps == 3) SC_VAL(TI, TO, 3); else if (taps == 2) SC_VAL(TI, TO, 2); \
        else SC_VAL(TI, TO, 0); \
      } else if (v_tiles) conv_values_kernel<TI, TO><<<v_grid, SC_WAVES * TS_WAVE, 0, stream>>>( \
          (TO*)v_cache, (const TI*)proj, row_stride, conv_w, state, seq_of_token, cu_seqlens, state_slots, slots, num_tokens, \
          channels, (nh + nkv) * hd, vd_size, taps, page_size, vp, vs, vh, vd); \
    } while (0)
    if (in_dtype == 0 && out_dtype == 0) SC_VEC_TAPS(float, float);
    else if (in_dtype == 0 && out_dtype == 1) SC_VEC_TAPS(float, bf16_t);
    else if (in_dtype == 1 && out_dtype == 1) SC_VEC_TAPS(bf16_t, bf16_t);
    else return TS_BAD_DTYPE;
#undef SC_VEC_TAPS
#undef SC_VAL
#undef SC_VEC
    return ts_check_launch();
  }
#define SC_LAUNCH(TI, TO) \
  conv_finish_kernel<TI, TO><<<(unsigned)blocks, SC_WAVES * TS_WAVE, 0, stream>>>( \
      (TO*)q_out, (TO*)k_cache, (TO*)v_cache, (const TI*)proj, row_stride, conv_w, state, q_norm_w, k_norm_w, eps, positions, \
      seq_of_token, cu_seqlens, state_slots, slots, nh, nkv, hd, vd_size, taps, temp_coef, temp_every, page_size, kp, ks, kh, \
      vp, vs, vh, vd, num_tokens, !v_tiles, moves_state); \
  if (v_tiles) conv_values_kernel<TI, TO><<<v_grid, SC_WAVES * TS_WAVE, 0, stream>>>( \
      (TO*)v_cache, (const TI*)proj, row_stride, conv_w, state, seq_of_token, cu_seqlens, state_slots, slots, num_tokens, \
      channels, (nh + nkv) * hd, vd_size, taps, page_size, vp, vs, vh, vd)
  if (in_dtype == 0 && out_dtype == 0) { SC_LAUNCH(float, float); }
  else if (in_dtype == 0 && out_dtype == 1) { SC_LAUNCH(float, bf16_t); }
  else if (in_dtype == 1 && out_dtype == 1) { SC_LAUNCH(bf16_t, bf16_t); }
  else return TS_BAD_DTYPE;
#undef SC_LAUNCH
  return ts_check_launch();
}

extern "C" int ts_conv_state_update(float* state, const void* proj, int64_t row_stride, const int32_t* cu_seqlens,
                                    const int32_t* state_slots, int num_seqs, int channels, int taps, int in_dtype,
                                    hipStream_t stream) {
  if (num_seqs <= 0 || taps <= 1) return TS_OK;
  if (channels <= 0 || taps > SC_MAX_TAPS || row_stride < channels) return TS_BAD_SHAPE;
  const int64_t threads = (int64_t)num_seqs * channels;
  const unsigned blocks = (unsigned)((threads + SC_WAVES * TS_WAVE - 1) / (SC_WAVES * TS_WAVE));
  if (in_dtype == 0)
    conv_state_update_kernel<float><<<blocks, SC_WAVES * TS_WAVE, 0, stream>>>(state, (const float*)proj, row_stride, cu_seqlens,
                                                                                state_slots, num_seqs, channels, taps);
  else if (in_dtype == 1)
    conv_state_update_kernel<bf16_t><<<blocks, SC_WAVES * TS_WAVE, 0, stream>>>(state, (const bf16_t*)proj, row_stride, cu_seqlens,
                                                                                 state_slots, num_seqs, channels, taps);
  else return TS_BAD_DTYPE;
  return ts_check_launch();
}
