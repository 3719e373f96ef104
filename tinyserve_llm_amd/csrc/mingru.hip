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
#include "common.h"

#define GRU_LANES 64
#define GRU_MAX_WAVES 16

static __device__ __forceinline__ float gru_sigmoid(float v) { return 1.0f / (1.0f + expf(-v)); }

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
        const float z = gru_sigmoid(GruIn<TI>::ld(zxg + t * row + c) + bz);
        const float u = GruIn<TI>::ld(zxg + t * row + width + c) + bx;
        const float cand = u >= 0.f ? u + 0.5f : gru_sigmoid(u);
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
      const float z = gru_sigmoid(GruIn<TI>::ld(zxg + t * row + c) + bz);
      const float u = GruIn<TI>::ld(zxg + t * row + width + c) + bx;
      const float g = GruIn<TI>::ld(zxg + t * row + 2 * width + c);
      const float cand = u >= 0.f ? u + 0.5f : gru_sigmoid(u);
      S = fmaf(1.0f - z, S, z * cand);
      Num<TO>::st(out + (int64_t)t * width + c, S * (g / (1.0f + expf(-g))));
    }
    // the last wave ends at the step's last token (or, with an empty stretch, holds the chained state as it is)
    if (wave == waves - 1) slot[c] = S;
  }
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
