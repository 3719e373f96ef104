// Attention with the options that the matrix-core kernels of the plain rotate-half, softmax kind do not have,
// for every storage type and every size:
//   * `ts_qkv_finish`: what lies between the q|k|v projection and the cache. Rotary positions on the first
//     `rot` dimensions of each q and k head, pairing (2i, 2i+1) (interleaved) or (i, i + rot/2) (halves), the
//     angle p * f_i taken in 64-bit from a table of frequencies (no table over positions: a request may be of
//     any length); then, optionally, each q and k head divided by its root mean square, and each value head
//     likewise; q goes to [tokens, heads, dim], k and v to their cache slots. Key and value heads may
//     differ in size.
//   * `ts_paged_attention_general`: one wavefront per (token, query head) over the request's pages, causal,
//     optionally windowed; score = q.k * scale, optionally capped as cap * tanh(score / cap); softmax,
//     optionally with a sink: a key of score 0 that has no value, i.e. one more in the denominator.
//     Scores, weights and the weighted sum are 32-bit. Keys are visited in chunks of 64 counted from position
//     0, so the order of every sum depends on the token's position alone.
#include "common.h"

#define AG_WAVES 4
#define AG_MAX_HD 256

template <typename TI, typename TO>
__global__ void __launch_bounds__(AG_WAVES * TS_WAVE)
qkv_finish_kernel(TO* __restrict__ q_out, TO* __restrict__ k_cache, TO* __restrict__ v_cache, const TI* __restrict__ qkv,
                  const double* __restrict__ freqs, const int32_t* __restrict__ positions,
                  const int32_t* __restrict__ slots, int num_tokens, int nh, int nkv, int hd, int vd_size, int rot,
                  int interleaved, int qk_norm, float qk_eps, int v_norm, float v_eps, int page_size, int64_t kp,
                  int64_t ks, int64_t kh, int64_t vp, int64_t vs, int64_t vh, int64_t vd) {
  __shared__ float head_s[AG_WAVES][AG_MAX_HD];
  const int wave = threadIdx.x / TS_WAVE, lane = threadIdx.x & (TS_WAVE - 1);
  const int heads = nh + 2 * nkv;
  const int64_t item = (int64_t)blockIdx.x * AG_WAVES + wave;
  if (item >= (int64_t)num_tokens * heads) return;       // the whole wave leaves; no block barrier below
  const int t = (int)(item / heads), h = (int)(item - (int64_t)t * heads);
  const bool is_q = h < nh, is_v = h >= nh + nkv;
  const int size = is_v ? vd_size : hd;
  const int64_t row = (int64_t)(nh + nkv) * hd + (int64_t)nkv * vd_size;
  const TI* src = qkv + t * row + (is_v ? (int64_t)(nh + nkv) * hd + (int64_t)(h - nh - nkv) * vd_size : (int64_t)h * hd);
  const int slot = slots ? slots[t] : -1;
  if (!is_q && (slot < 0 || !k_cache)) return;           // nothing to write for this token
  for (int d = lane; d < size; d += TS_WAVE) head_s[wave][d] = Num<TI>::ld(src + d);
  wave_sync();
  const int pos = positions[t];
  const int half = rot / 2;
  float y[AG_MAX_HD / TS_WAVE];
  float squares = 0.f;
#pragma unroll
  for (int i = 0; i < AG_MAX_HD / TS_WAVE; ++i) {
    const int d = lane + i * TS_WAVE;
    float v = 0.f;
    if (d < size) {
      v = head_s[wave][d];
      if (!is_v && d < rot) {
        // the pair's index, this element's partner, and whether this element is the pair's first
        const int pair = interleaved ? d >> 1 : (d < half ? d : d - half);
        const bool first = interleaved ? !(d & 1) : d < half;
        const int partner = interleaved ? d ^ 1 : (first ? d + half : d - half);
        // the angle in 64-bit, brought to [-pi, pi] before the 32-bit sine and cosine
        const double angle = (double)pos * freqs[pair];
        const double turns = rint(angle * 0.15915494309189535);
        const float a = (float)fma(-turns, 6.283185307179586, angle);
        float sn, cs;
        sincosf(a, &sn, &cs);
        const float w = head_s[wave][partner];
        v = first ? v * cs - w * sn : v * cs + w * sn;
      }
    }
    y[i] = v;
    squares = fmaf(v, v, squares);
  }
  float scale = 1.0f;
  if (is_v ? v_norm : qk_norm) scale = 1.0f / sqrtf(wave_sum(squares) / (float)size + (is_v ? v_eps : qk_eps));
  if (is_q) {
    TO* dst = q_out + ((int64_t)t * nh + h) * hd;
#pragma unroll
    for (int i = 0; i < AG_MAX_HD / TS_WAVE; ++i) {
      const int d = lane + i * TS_WAVE;
      if (d < size) Num<TO>::st(dst + d, y[i] * scale);
    }
    return;
  }
  const int page = slot / page_size, off = slot - page * page_size;
  if (!is_v) {
    TO* dst = k_cache + page * kp + off * ks + (int64_t)(h - nh) * kh;
#pragma unroll
    for (int i = 0; i < AG_MAX_HD / TS_WAVE; ++i) {
      const int d = lane + i * TS_WAVE;
      if (d < size) Num<TO>::st(dst + d, y[i] * scale);
    }
  } else {
    TO* dst = v_cache + page * vp + off * vs + (int64_t)(h - nh - nkv) * vh;
#pragma unroll
    for (int i = 0; i < AG_MAX_HD / TS_WAVE; ++i) {
      const int d = lane + i * TS_WAVE;
      if (d < size) Num<TO>::st(dst + (int64_t)d * vd, y[i] * scale);
    }
  }
}

extern "C" int ts_qkv_finish(void* q_out, void* k_cache, void* v_cache, const void* qkv, const double* freqs,
                             const int32_t* positions, const int32_t* slots, int num_tokens, int nh, int nkv, int hd,
                             int vd_size, int rot, int interleaved, int qk_norm, float qk_eps, int v_norm, float v_eps,
                             int page_size, int64_t kp, int64_t ks, int64_t kh, int64_t vp, int64_t vs, int64_t vh,
                             int64_t vd, int in_dtype, int out_dtype, hipStream_t stream) {
  if (num_tokens <= 0) return TS_OK;
  if (hd <= 0 || hd > AG_MAX_HD || vd_size <= 0 || vd_size > AG_MAX_HD || nh <= 0 || nkv <= 0 || rot < 0 || rot > hd || rot % 2 ||
      page_size <= 0 || (rot > 0 && !freqs))
    return TS_BAD_SHAPE;
  const int64_t items = (int64_t)num_tokens * (nh + 2 * nkv);
  const int64_t blocks = (items + AG_WAVES - 1) / AG_WAVES;
  if (blocks > 0x7fffffff) return TS_BAD_SHAPE;
#define QF_LAUNCH(TI, TO) \
  qkv_finish_kernel<TI, TO><<<(unsigned)blocks, AG_WAVES * TS_WAVE, 0, stream>>>( \
      (TO*)q_out, (TO*)k_cache, (TO*)v_cache, (const TI*)qkv, freqs, positions, slots, num_tokens, nh, nkv, hd, vd_size, rot, \
      interleaved, qk_norm, qk_eps, v_norm, v_eps, page_size, kp, ks, kh, vp, vs, vh, vd)
  if (in_dtype == 0 && out_dtype == 0) QF_LAUNCH(float, float);
  else if (in_dtype == 0 && out_dtype == 1) QF_LAUNCH(float, bf16_t);
  else if (in_dtype == 1 && out_dtype == 1) QF_LAUNCH(bf16_t, bf16_t);
  else return TS_BAD_DTYPE;
#undef QF_LAUNCH
  return ts_check_launch();
}

template <typename T>
__global__ void __launch_bounds__(AG_WAVES * TS_WAVE)
paged_attention_general_kernel(T* __restrict__ out, const T* __restrict__ q, const T* __restrict__ k_cache,
                               const T* __restrict__ v_cache, const int32_t* __restrict__ block_tables,
                               const int32_t* __restrict__ seq_of_token, const int32_t* __restrict__ positions,
                               int num_tokens, int nh, int nkv, int hd, int vd_size, int page_size, int64_t kp, int64_t ks,
                               int64_t kh, int64_t vp, int64_t vs, int64_t vh, int64_t vd, int max_blocks, float scale,
                               float softcap, int sink, int window, int page_run) {
  __shared__ float q_s[AG_WAVES][AG_MAX_HD];
  __shared__ float p_s[AG_WAVES][TS_WAVE];
  __shared__ int64_t row_s[AG_WAVES][TS_WAVE];   // element offset of each key's value row
  const int wave = threadIdx.x / TS_WAVE, lane = threadIdx.x & (TS_WAVE - 1);
  const int64_t item = (int64_t)blockIdx.x * AG_WAVES + wave;
  if (item >= (int64_t)num_tokens * nh) return;
  const int t = (int)(item / nh), h = (int)(item - (int64_t)t * nh);
  const int kvh = h / (nh / nkv);
  const int pos = positions[t];
  const int32_t* table = block_tables + (int64_t)seq_of_token[t] * max_blocks;
  const T* qrow = q + ((int64_t)t * nh + h) * hd;
  for (int d = lane; d < hd; d += TS_WAVE) q_s[wave][d] = Num<T>::ld(qrow + d);
  wave_sync();

  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  // the sink is a key of score 0 without a value: it starts the running maximum and the sum
  float m = sink ? 0.f : -INFINITY, l = sink ? 1.f : 0.f;
  float acc[AG_MAX_HD / TS_WAVE] = {0.f, 0.f, 0.f, 0.f};
  const float inv_cap = softcap > 0.f ? 1.0f / softcap : 0.f;

  for (int c0 = (lo / TS_WAVE) * TS_WAVE; c0 <= pos; c0 += TS_WAVE) {
    const int key = c0 + lane;
    const bool valid = key >= lo && key <= pos;
    float s = -INFINITY;
    int64_t rowoff = 0;
    if (valid) {
      const int pg = key / page_size, slot = key % page_size;
      const int64_t page = ((int64_t)table[pg >> page_run] << page_run) + (pg & ((1 << page_run) - 1));
      rowoff = page * vp + (int64_t)slot * vs + (int64_t)kvh * vh;
      const T* kr = k_cache + page * kp + (int64_t)slot * ks + (int64_t)kvh * kh;
      float dot = 0.f;
      for (int d = 0; d < hd; ++d) dot = fmaf(q_s[wave][d], Num<T>::ld(kr + d), dot);
      s = dot * scale;
      if (softcap > 0.f) s = softcap * tanhf(s * inv_cap);
    }
    const float m_new = fmaxf(m, wave_max(s));  // finite: the chunk holds at least one visible key
    const float p = valid ? expf(s - m_new) : 0.f;
    const float alpha = expf(m - m_new);
    l = l * alpha + wave_sum(p);
    m = m_new;
    p_s[wave][lane] = p;
    row_s[wave][lane] = rowoff;
    wave_sync();
    const int first = lo > c0 ? lo - c0 : 0;
    const int last = pos - c0 < TS_WAVE - 1 ? pos - c0 : TS_WAVE - 1;
#pragma unroll
    for (int i = 0; i < AG_MAX_HD / TS_WAVE; ++i) {
      const int d = lane + i * TS_WAVE;
      if (d < vd_size) {
        float a = acc[i] * alpha;
        for (int j = first; j <= last; ++j) a = fmaf(p_s[wave][j], Num<T>::ld(v_cache + row_s[wave][j] + (int64_t)d * vd), a);
        acc[i] = a;
      }
    }
    wave_sync();
  }
  T* orow = out + ((int64_t)t * nh + h) * vd_size;
  const float inv = 1.0f / l;
#pragma unroll
  for (int i = 0; i < AG_MAX_HD / TS_WAVE; ++i) {
    const int d = lane + i * TS_WAVE;
    if (d < vd_size) Num<T>::st(orow + d, acc[i] * inv);
  }
}

extern "C" int ts_paged_attention_general(void* out, const void* q, const void* k_cache, const void* v_cache,
                                          const int32_t* block_tables, const int32_t* seq_of_token,
                                          const int32_t* positions, int num_tokens, int nh, int nkv, int hd, int vd_size,
                                          int page_size, int64_t kp, int64_t ks, int64_t kh, int64_t vp, int64_t vs,
                                          int64_t vh, int64_t vd, int max_blocks, float scale, float softcap, int sink,
                                          int window, int dtype, int page_run, hipStream_t stream) {
  if (num_tokens <= 0) return TS_OK;
  if (hd <= 0 || hd > AG_MAX_HD || vd_size <= 0 || vd_size > AG_MAX_HD || nkv <= 0 || nh % nkv || page_size <= 0 ||
      max_blocks <= 0 || page_run < 0 || page_run > 16 || softcap < 0.f)
    return TS_BAD_SHAPE;
  const int64_t items = (int64_t)num_tokens * nh;
  const int64_t blocks = (items + AG_WAVES - 1) / AG_WAVES;
  if (blocks > 0x7fffffff) return TS_BAD_SHAPE;
  dim3 grid((unsigned)blocks), block(AG_WAVES * TS_WAVE);
  if (dtype == 0)
    paged_attention_general_kernel<float><<<grid, block, 0, stream>>>(
        (float*)out, (const float*)q, (const float*)k_cache, (const float*)v_cache, block_tables, seq_of_token, positions,
        num_tokens, nh, nkv, hd, vd_size, page_size, kp, ks, kh, vp, vs, vh, vd, max_blocks, scale, softcap, sink, window,
        page_run);
  else if (dtype == 1)
    paged_attention_general_kernel<bf16_t><<<grid, block, 0, stream>>>(
        (bf16_t*)out, (const bf16_t*)q, (const bf16_t*)k_cache, (const bf16_t*)v_cache, block_tables, seq_of_token, positions,
        num_tokens, nh, nkv, hd, vd_size, page_size, kp, ks, kh, vp, vs, vh, vd, max_blocks, scale, softcap, sink, window,
        page_run);
  else
    return TS_BAD_DTYPE;
  return ts_check_launch();
}
