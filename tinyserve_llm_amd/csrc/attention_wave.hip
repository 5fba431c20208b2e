// Paged attention over block tables, one wavefront per (token, query head). It serves every
// storage type, head size (a multiple of 16 up to 256), head grouping and page size, for prompt
// portions and decoded tokens alike: a token at position p sees the keys of its request at
// positions max(0, p - window + 1) .. p, all of them read from the cache pages (the step's own keys
// are written before this runs). Key rows are dense in head_dim; value elements are addressed
// with four strides (page, slot, head, dimension), so any page layout of the values works. Keys are visited in chunks of 64 counted from position 0, so the
// order of every sum depends only on the token's position, never on the batch or on the portion.
// Scores, softmax and the weighted sum are 32-bit.
#include "common.h"

#define ATT_WAVES 4
#define ATT_MAX_HD 256

template <typename T> struct Vec;  // 16-byte vector loads of a key row
template <> struct Vec<float> {
  static constexpr int N = 4;
  static __device__ __forceinline__ void ld(const float* p, float* o) {
    const float4 v = *(const float4*)p;
    o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w;
  }
};
template <> struct Vec<bf16_t> {
  static constexpr int N = 8;
  static __device__ __forceinline__ void ld(const bf16_t* p, float* o) {
    const uint4 v = *(const uint4*)p;
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      o[2 * i] = __uint_as_float(w[i] << 16);
      o[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
  }
};

template <typename T>
__global__ void __launch_bounds__(ATT_WAVES * TS_WAVE)
paged_attention_wave_kernel(T* __restrict__ out, const T* __restrict__ q, const T* __restrict__ k_cache,
                            const T* __restrict__ v_cache, const int32_t* __restrict__ block_tables,
                            const int32_t* __restrict__ seq_of_token, const int32_t* __restrict__ positions,
                            int num_tokens, int nh, int nkv, int hd, int page_size, int64_t page_stride,
                            int64_t slot_stride, int64_t head_stride, int64_t vp, int64_t vs, int64_t vh, int64_t vd,
                            int max_blocks, float scale, int window, int page_run) {
  __shared__ float q_s[ATT_WAVES][ATT_MAX_HD];
  __shared__ float p_s[ATT_WAVES][TS_WAVE];
  __shared__ int64_t row_s[ATT_WAVES][TS_WAVE];   // element offset of each key's value row
  const int wave = threadIdx.x / TS_WAVE, lane = threadIdx.x & (TS_WAVE - 1);
  const int64_t item = (int64_t)blockIdx.x * ATT_WAVES + wave;
  if (item >= (int64_t)num_tokens * nh) return;  // whole wave leaves together; no block barrier below
  const int t = (int)(item / nh), h = (int)(item - (int64_t)t * nh);
  const int kvh = h / (nh / nkv);
  const int pos = positions[t];
  const int32_t* table = block_tables + (int64_t)seq_of_token[t] * max_blocks;
  const T* qrow = q + ((int64_t)t * nh + h) * hd;
  for (int d = lane; d < hd; d += TS_WAVE) q_s[wave][d] = Num<T>::ld(qrow + d);
  wave_sync();

  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  float m = -INFINITY, l = 0.f;
  float acc[ATT_MAX_HD / TS_WAVE] = {0.f, 0.f, 0.f, 0.f};

  for (int c0 = (lo / TS_WAVE) * TS_WAVE; c0 <= pos; c0 += TS_WAVE) {
    const int key = c0 + lane;
    const bool valid = key >= lo && key <= pos;
    float s = -INFINITY;
    int64_t rowoff = 0;
    if (valid) {
      // (an entry of the table names 2^page_run consecutive pages of the pool)
      const int pg = key / page_size, slot = key % page_size;
      const int64_t page = ((int64_t)table[pg >> page_run] << page_run) + (pg & ((1 << page_run) - 1));
      rowoff = page * vp + (int64_t)slot * vs + (int64_t)kvh * vh;
      const T* kr = k_cache + page * page_stride + (int64_t)slot * slot_stride + (int64_t)kvh * head_stride;
      float dot = 0.f;
      for (int d = 0; d < hd; d += Vec<T>::N) {
        float kv[Vec<T>::N];
        Vec<T>::ld(kr + d, kv);
#pragma unroll
        for (int i = 0; i < Vec<T>::N; ++i) dot = fmaf(q_s[wave][d + i], kv[i], dot);
      }
      s = dot * scale;
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
    for (int i = 0; i < ATT_MAX_HD / TS_WAVE; ++i) {
      const int d = lane + i * TS_WAVE;
      if (d < hd) {
        float a = acc[i] * alpha;
        for (int j = first; j <= last; ++j) a = fmaf(p_s[wave][j], Num<T>::ld(v_cache + row_s[wave][j] + (int64_t)d * vd), a);
        acc[i] = a;
      }
    }
    wave_sync();
  }
  T* orow = out + ((int64_t)t * nh + h) * hd;
  const float inv = 1.0f / l;
#pragma unroll
  for (int i = 0; i < ATT_MAX_HD / TS_WAVE; ++i) {
    const int d = lane + i * TS_WAVE;
    if (d < hd) Num<T>::st(orow + d, acc[i] * inv);
  }
}

extern "C" int ts_paged_attention_wave(void* out, const void* q, const void* k_cache, const void* v_cache,
                                       const int32_t* block_tables, const int32_t* seq_of_token,
                                       const int32_t* positions, int num_tokens, int nh, int nkv, int hd,
                                       int page_size, int64_t page_stride, int64_t slot_stride, int64_t head_stride,
                                       int64_t vp, int64_t vs, int64_t vh, int64_t vd, int max_blocks, float scale,
                                       int window, int dtype, int page_run, hipStream_t stream) {
  if (num_tokens <= 0) return TS_OK;
  if (hd % 16 || hd > ATT_MAX_HD || hd <= 0 || nkv <= 0 || nh % nkv || page_size <= 0 || max_blocks <= 0 || page_run < 0 || page_run > 16)
    return TS_BAD_SHAPE;
  // 16-byte key loads need 16-byte aligned rows
  const int64_t elem = dtype == 0 ? 4 : 2;
  if ((page_stride * elem) % 16 || (slot_stride * elem) % 16 || (head_stride * elem) % 16) return TS_BAD_SHAPE;
  const int64_t items = (int64_t)num_tokens * nh;
  const int64_t blocks = (items + ATT_WAVES - 1) / ATT_WAVES;
  if (blocks > 0x7fffffff) return TS_BAD_SHAPE;
  dim3 grid((unsigned)blocks), block(ATT_WAVES * TS_WAVE);
  if (dtype == 0)
    paged_attention_wave_kernel<float><<<grid, block, 0, stream>>>(
        (float*)out, (const float*)q, (const float*)k_cache, (const float*)v_cache, block_tables, seq_of_token,
        positions, num_tokens, nh, nkv, hd, page_size, page_stride, slot_stride, head_stride, vp, vs, vh, vd, max_blocks,
        scale, window, page_run);
  else if (dtype == 1)
    paged_attention_wave_kernel<bf16_t><<<grid, block, 0, stream>>>(
        (bf16_t*)out, (const bf16_t*)q, (const bf16_t*)k_cache, (const bf16_t*)v_cache, block_tables, seq_of_token,
        positions, num_tokens, nh, nkv, hd, page_size, page_stride, slot_stride, head_stride, vp, vs, vh, vd, max_blocks,
        scale, window, page_run);
  else
    return TS_BAD_DTYPE;
  return ts_check_launch();
}
