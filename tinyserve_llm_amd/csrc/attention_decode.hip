// Split-key paged attention for tokens that each bring one query (decoding): a workgroup takes one
// (token, key/value head, chunk of keys) and serves all query heads of that key/value head's group
// from one pass over the chunk, so the cache is read once. Partial results (unnormalised output,
// running max and sum per chunk) go to a 32-bit workspace; a second kernel combines the chunks of a
// token in ascending order. The chunk size is chosen on the host (64, 128 or 256 keys) so that few
// tokens still fill the GPU; chunk boundaries are multiples of it counted from position 0.
// Scores, softmax and sums are 32-bit whatever the storage type.
#include "common.h"

#define DEC_THREADS 256

template <typename T> struct Row;   // vector loads of cache rows
template <> struct Row<float> {
  static constexpr int K = 4;       // elements per 16-byte key load
  static __device__ __forceinline__ void ldk(const float* p, float* o) {
    const float4 v = *(const float4*)p;
    o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w;
  }
  static __device__ __forceinline__ void ldv4(const float* p, float* o) {
    const float4 v = *(const float4*)p;
    o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w;
  }
};
template <> struct Row<bf16_t> {
  static constexpr int K = 8;
  static __device__ __forceinline__ void ldk(const bf16_t* p, float* o) {
    const uint4 v = *(const uint4*)p;
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      o[2 * i] = __uint_as_float(w[i] << 16);
      o[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
  }
  static __device__ __forceinline__ void ldv4(const bf16_t* p, float* o) {
    const uint2 v = *(const uint2*)p;
    o[0] = __uint_as_float(v.x << 16); o[1] = __uint_as_float(v.x & 0xffff0000u);
    o[2] = __uint_as_float(v.y << 16); o[3] = __uint_as_float(v.y & 0xffff0000u);
  }
};

// dynamic shared memory layout (floats unless noted):
//   q_s   [G * hd]
//   sc    [G * chunk]            scores, then probabilities
//   ml    [2 * G]
//   red   [nslices * G * hd]
//   rowo  [chunk] int64          element offset of each key's row
template <typename T, int G>
__global__ void __launch_bounds__(DEC_THREADS)
attn_decode_split_kernel(float* __restrict__ part_o, float* __restrict__ part_ml, const T* __restrict__ q,
                         const T* __restrict__ k_cache, const T* __restrict__ v_cache,
                         const int32_t* __restrict__ block_tables, const int32_t* __restrict__ seq_of_token,
                         const int32_t* __restrict__ positions, int nh, int hd, int page_size, int64_t page_stride,
                         int64_t slot_stride, int64_t head_stride, int max_blocks, int num_splits, int chunk, int tpk,
                         float scale, int window) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int tid = threadIdx.x;
  const int split = blockIdx.x, kvh = blockIdx.y, t = blockIdx.z;
  const int pos = positions[t];
  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int k0 = split * chunk;
  if (k0 > pos || k0 + chunk <= lo) return;   // the whole workgroup leaves: nothing of this chunk is visible
  const int tpr = hd / 4;                      // threads per value row (4 elements each)
  const int nslices = DEC_THREADS / tpr;

  int64_t* rowo = (int64_t*)smem;
  float* q_s = (float*)(rowo + chunk);
  float* sc = q_s + G * hd;
  float* ml = sc + G * chunk;
  float* red = ml + 2 * G;

  const int32_t* table = block_tables + (int64_t)seq_of_token[t] * max_blocks;
  const T* qrow = q + ((int64_t)t * nh + (int64_t)kvh * G) * hd;
  for (int i = tid; i < G * hd; i += DEC_THREADS) q_s[i] = Num<T>::ld(qrow + i);
  __syncthreads();

  // ---- scores: `tpk` threads share a key, each takes hd / tpk dimensions
  {
    const int kidx = tid / tpk, part = tid - kidx * tpk;
    const int key = k0 + kidx;
    const bool valid = kidx < chunk && key <= pos && key >= lo;
    float dots[G];
#pragma unroll
    for (int g = 0; g < G; ++g) dots[g] = 0.f;
    int64_t off = 0;
    if (valid) {
      const int page = table[key / page_size];
      off = (int64_t)page * page_stride + (int64_t)(key % page_size) * slot_stride + (int64_t)kvh * head_stride;
      const int span = hd / tpk, d0 = part * span;
      const T* kr = k_cache + off + d0;
      for (int d = 0; d < span; d += Row<T>::K) {
        float kv[Row<T>::K];
        Row<T>::ldk(kr + d, kv);
#pragma unroll
        for (int g = 0; g < G; ++g) {
          const float* qg = q_s + g * hd + d0 + d;
#pragma unroll
          for (int i = 0; i < Row<T>::K; ++i) dots[g] = fmaf(qg[i], kv[i], dots[g]);
        }
      }
    }
    // the tpk threads of a key are neighbouring lanes of one wave
    for (int o = 1; o < tpk; o <<= 1) {
#pragma unroll
      for (int g = 0; g < G; ++g) dots[g] += __shfl_xor(dots[g], o, TS_WAVE);
    }
    if (kidx < chunk && part == 0) {
      rowo[kidx] = off;
#pragma unroll
      for (int g = 0; g < G; ++g) sc[g * chunk + kidx] = valid ? dots[g] * scale : -INFINITY;
    }
  }
  __syncthreads();

  // ---- softmax over the chunk, one wave per query head at a time
  {
    const int wave = tid / TS_WAVE, lane = tid & (TS_WAVE - 1);
    for (int g = wave; g < G; g += DEC_THREADS / TS_WAVE) {
      float m = -INFINITY;
      for (int j = lane; j < chunk; j += TS_WAVE) m = fmaxf(m, sc[g * chunk + j]);
      m = wave_max(m);
      float l = 0.f;
      for (int j = lane; j < chunk; j += TS_WAVE) {
        const float s = sc[g * chunk + j];
        const float p = s == -INFINITY ? 0.f : expf(s - m);
        sc[g * chunk + j] = p;
        l += p;
      }
      l = wave_sum(l);
      if (lane == 0) { ml[2 * g] = m; ml[2 * g + 1] = l; }
    }
  }
  __syncthreads();

  // ---- weighted sum of values: thread = (slice of keys, 4 dimensions)
  {
    const int slice = tid / tpr, c = (tid - slice * tpr) * 4;
    if (slice < nslices) {
      float acc[G][4];
#pragma unroll
      for (int g = 0; g < G; ++g)
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[g][i] = 0.f;
      const int first = lo > k0 ? lo - k0 : 0;
      const int last = pos - k0 < chunk - 1 ? pos - k0 : chunk - 1;
      for (int j = first + slice; j <= last; j += nslices) {
        float v[4];
        Row<T>::ldv4(v_cache + rowo[j] + c, v);
#pragma unroll
        for (int g = 0; g < G; ++g) {
          const float p = sc[g * chunk + j];
#pragma unroll
          for (int i = 0; i < 4; ++i) acc[g][i] = fmaf(p, v[i], acc[g][i]);
        }
      }
#pragma unroll
      for (int g = 0; g < G; ++g)
#pragma unroll
        for (int i = 0; i < 4; ++i) red[((int64_t)slice * G + g) * hd + c + i] = acc[g][i];
    }
  }
  __syncthreads();
  for (int i = tid; i < G * hd; i += DEC_THREADS) {
    float sum = 0.f;
    for (int s = 0; s < nslices; ++s) sum += red[(int64_t)s * G * hd + i];
    const int g = i / hd, d = i - g * hd;
    part_o[(((int64_t)t * nh + kvh * G + g) * num_splits + split) * hd + d] = sum;
  }
  if (tid < 2 * G) {
    const int g = tid >> 1;
    part_ml[(((int64_t)t * nh + kvh * G + g) * num_splits + split) * 2 + (tid & 1)] = ml[tid];
  }
}

// out[t, h, :] = sum_s o_s e^{m_s - M} / sum_s l_s e^{m_s - M} over the chunks s that hold visible keys
template <typename T>
__global__ void attn_decode_combine_kernel(T* __restrict__ out, const float* __restrict__ part_o,
                                           const float* __restrict__ part_ml, const int32_t* __restrict__ positions,
                                           int nh, int hd, int num_splits, int chunk, int window) {
  const int t = blockIdx.x / nh;
  const int64_t th = blockIdx.x;
  const int pos = positions[t];
  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int s0 = lo / chunk, s1 = pos / chunk;
  const float* ml = part_ml + th * num_splits * 2;
  float M = -INFINITY;
  for (int s = s0; s <= s1; ++s) M = fmaxf(M, ml[2 * s]);
  float L = 0.f;
  for (int s = s0; s <= s1; ++s) L += ml[2 * s + 1] * expf(ml[2 * s] - M);
  const float inv = 1.0f / L;
  for (int d = threadIdx.x; d < hd; d += blockDim.x) {
    float acc = 0.f;
    for (int s = s0; s <= s1; ++s) acc += part_o[(th * num_splits + s) * hd + d] * expf(ml[2 * s] - M);
    Num<T>::st(out + th * hd + d, acc * inv);
  }
}

static size_t dec_smem_bytes(int G, int hd, int chunk) {
  const int tpr = hd / 4, nslices = DEC_THREADS / tpr;
  return (size_t)chunk * 8 + sizeof(float) * ((size_t)G * hd + (size_t)G * chunk + 2 * G + (size_t)nslices * G * hd);
}

template <typename T, int G>
static int launch_split(float* part_o, float* part_ml, const void* q, const void* kc, const void* vc,
                        const int32_t* tables, const int32_t* seq_of, const int32_t* positions, int num_tokens, int nh,
                        int nkv, int hd, int page_size, int64_t page_stride, int64_t slot_stride, int64_t head_stride,
                        int max_blocks, int num_splits, int chunk, int tpk, float scale, int window,
                        hipStream_t stream) {
  const size_t smem = dec_smem_bytes(G, hd, chunk);
  if (smem > 64 * 1024) return TS_BAD_SHAPE;
  dim3 grid(num_splits, nkv, num_tokens);
  attn_decode_split_kernel<T, G><<<grid, DEC_THREADS, smem, stream>>>(
      part_o, part_ml, (const T*)q, (const T*)kc, (const T*)vc, tables, seq_of, positions, nh, hd, page_size,
      page_stride, slot_stride, head_stride, max_blocks, num_splits, chunk, tpk, scale, window);
  return ts_check_launch();
}

// part_o [tokens, nh, num_splits, hd] and part_ml [tokens, nh, num_splits, 2] are float workspaces.
// num_splits * chunk must cover every position that `positions` holds.
extern "C" int ts_paged_attention_decode(void* out, float* part_o, float* part_ml, const void* q, const void* k_cache,
                                         const void* v_cache, const int32_t* block_tables,
                                         const int32_t* seq_of_token, const int32_t* positions, int num_tokens, int nh,
                                         int nkv, int hd, int page_size, int64_t page_stride, int64_t slot_stride,
                                         int64_t head_stride, int max_blocks, int num_splits, int chunk, float scale,
                                         int window, int dtype, hipStream_t stream) {
  if (num_tokens <= 0) return TS_OK;
  if (hd % 16 || hd > 256 || hd <= 0 || nkv <= 0 || nh % nkv || page_size <= 0 || max_blocks <= 0 || num_splits <= 0)
    return TS_BAD_SHAPE;
  if (chunk != 64 && chunk != 128 && chunk != 256) return TS_BAD_SHAPE;
  if (num_tokens > 65535 || nkv > 65535) return TS_BAD_SHAPE;
  const int G = nh / nkv;
  if (G > 8) return TS_BAD_SHAPE;
  const int64_t elem = dtype == 0 ? 4 : 2;
  if ((page_stride * elem) % 16 || (slot_stride * elem) % 16 || (head_stride * elem) % 16) return TS_BAD_SHAPE;
  // threads per key: as many as divide the row into whole 16-byte loads
  const int per_load = dtype == 0 ? 4 : 8;
  int tpk = DEC_THREADS / chunk;
  while (tpk > 1 && (hd % tpk || (hd / tpk) % per_load)) tpk >>= 1;
  int rc;
#define TS_DEC_CASE(GG)                                                                                              \
  case GG:                                                                                                           \
    rc = dtype == 0 ? launch_split<float, GG>(part_o, part_ml, q, k_cache, v_cache, block_tables, seq_of_token,      \
                                              positions, num_tokens, nh, nkv, hd, page_size, page_stride,            \
                                              slot_stride, head_stride, max_blocks, num_splits, chunk, tpk, scale,   \
                                              window, stream)                                                        \
                    : launch_split<bf16_t, GG>(part_o, part_ml, q, k_cache, v_cache, block_tables, seq_of_token,     \
                                               positions, num_tokens, nh, nkv, hd, page_size, page_stride,           \
                                               slot_stride, head_stride, max_blocks, num_splits, chunk, tpk, scale,  \
                                               window, stream);                                                      \
    break;
  if (dtype != 0 && dtype != 1) return TS_BAD_DTYPE;
  switch (G) {
    TS_DEC_CASE(1) TS_DEC_CASE(2) TS_DEC_CASE(3) TS_DEC_CASE(4) TS_DEC_CASE(5) TS_DEC_CASE(6) TS_DEC_CASE(7)
    TS_DEC_CASE(8)
    default: return TS_BAD_SHAPE;
  }
#undef TS_DEC_CASE
  if (rc) return rc;
  const int threads = hd < 64 ? 64 : (hd > 256 ? 256 : hd);
  if (dtype == 0)
    attn_decode_combine_kernel<float><<<num_tokens * nh, threads, 0, stream>>>((float*)out, part_o, part_ml, positions,
                                                                              nh, hd, num_splits, chunk, window);
  else
    attn_decode_combine_kernel<bf16_t><<<num_tokens * nh, threads, 0, stream>>>((bf16_t*)out, part_o, part_ml,
                                                                               positions, nh, hd, num_splits, chunk,
                                                                               window);
  return ts_check_launch();
}
