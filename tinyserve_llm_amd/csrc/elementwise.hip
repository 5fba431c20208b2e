// Row-wise kernels of the decoder step: embedding gather, (residual+)RMSNorm, rotate-half RoPE
// fused with the write of K and V into their cache pages, SiLU-gate multiply, page-prefix copy.
// Every kernel exists for float and for bfloat16 storage; sums, rsqrt, rotation and the
// residual sum are always computed in 32-bit.
#include "common.h"

// ------------------------------------------------------------------------------------------
// Embedding: out[t, :] = table[ids[t], :]
// ------------------------------------------------------------------------------------------
template <typename T>
__global__ void embedding_kernel(T* __restrict__ out, const T* __restrict__ table,
                                 const int32_t* __restrict__ ids, int hidden) {
  const int t = blockIdx.x;
  const T* src = table + (int64_t)ids[t] * hidden;
  T* dst = out + (int64_t)t * hidden;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) dst[i] = src[i];
}

extern "C" int ts_embedding(void* out, const void* table, const int32_t* ids, int num_tokens,
                            int hidden, int dtype, hipStream_t stream) {
  if (num_tokens <= 0) return TS_OK;
  if (dtype == 0)
    embedding_kernel<float><<<num_tokens, 256, 0, stream>>>((float*)out, (const float*)table, ids, hidden);
  else if (dtype == 1)
    embedding_kernel<bf16_t><<<num_tokens, 256, 0, stream>>>((bf16_t*)out, (const bf16_t*)table, ids, hidden);
  else
    return TS_BAD_DTYPE;
  return ts_check_launch();
}

// ------------------------------------------------------------------------------------------
// RMSNorm with optional residual add and optional row selection.
//   s = float(x[row]) + float(res[row])            (res may be null)
//   res_out[r] = T(s)                              (res_out may be null)
//   out[r] = T(s * rsqrt(mean(s^2) + eps)) * w     (second rounding as the storage type has it)
// One 256-thread block per output row; the reduction tree has a fixed shape, so a row's result
// does not depend on what else is in the batch.
// ------------------------------------------------------------------------------------------
#define NORM_THREADS 256

template <typename T, typename WT>
__global__ void rmsnorm_kernel(T* __restrict__ out, T* __restrict__ res_out, const T* __restrict__ x,
                               const T* __restrict__ res, const WT* __restrict__ w,
                               const int32_t* __restrict__ rows, int hidden, float eps) {
  __shared__ float partial[NORM_THREADS / TS_WAVE];
  const int r = blockIdx.x;
  const int64_t src = rows ? (int64_t)rows[r] : (int64_t)r;
  const T* xr = x + src * hidden;
  const T* rr = res ? res + src * hidden : nullptr;
  float acc = 0.f;
  for (int i = threadIdx.x; i < hidden; i += NORM_THREADS) {
    float s = Num<T>::ld(xr + i);
    if (rr) s += Num<T>::ld(rr + i);
    acc += s * s;
  }
  acc = wave_sum(acc);
  if ((threadIdx.x & (TS_WAVE - 1)) == 0) partial[threadIdx.x / TS_WAVE] = acc;
  __syncthreads();
  float total = 0.f;
#pragma unroll
  for (int i = 0; i < NORM_THREADS / TS_WAVE; ++i) total += partial[i];
  const float inv = 1.0f / sqrtf(total / (float)hidden + eps);
  T* orow = out + (int64_t)r * hidden;
  T* rorow = res_out ? res_out + (int64_t)r * hidden : nullptr;
  for (int i = threadIdx.x; i < hidden; i += NORM_THREADS) {
    float s = Num<T>::ld(xr + i);
    if (rr) s += Num<T>::ld(rr + i);
    if (rorow) Num<T>::st(rorow + i, s);
    const float y = Num<T>::round(s * inv);
    Num<T>::st(orow + i, y * Num<WT>::ld(w + i));
  }
}

// wdtype: storage of the weight vector (0 float, 1 bfloat16); dtype: storage of activations.
extern "C" int ts_rmsnorm(void* out, void* res_out, const void* x, const void* res, const void* w,
                          const int32_t* rows, int num_rows, int hidden, float eps, int dtype,
                          int wdtype, hipStream_t stream) {
  if (num_rows <= 0) return TS_OK;
  dim3 grid(num_rows), block(NORM_THREADS);
  if (dtype == 0 && wdtype == 0)
    rmsnorm_kernel<float, float><<<grid, block, 0, stream>>>((float*)out, (float*)res_out, (const float*)x,
                                                             (const float*)res, (const float*)w, rows, hidden, eps);
  else if (dtype == 1 && wdtype == 1)
    rmsnorm_kernel<bf16_t, bf16_t><<<grid, block, 0, stream>>>((bf16_t*)out, (bf16_t*)res_out, (const bf16_t*)x,
                                                               (const bf16_t*)res, (const bf16_t*)w, rows, hidden, eps);
  else if (dtype == 1 && wdtype == 0)
    rmsnorm_kernel<bf16_t, float><<<grid, block, 0, stream>>>((bf16_t*)out, (bf16_t*)res_out, (const bf16_t*)x,
                                                              (const bf16_t*)res, (const float*)w, rows, hidden, eps);
  else
    return TS_BAD_DTYPE;
  return ts_check_launch();
}

// ------------------------------------------------------------------------------------------
// Rotate-half RoPE on q and k from a 32-bit [max_pos, head_dim] table ([cos | sin] halves),
// fused with the scatter of rotated k and of v into their cache slots.
//   qkv   [T, (nh + 2*nkv) * hd]   one token's q heads, then k heads, then v heads
//   q_out [T, nh * hd]
//   cache element address: page * page_stride + offset * slot_stride + head * head_stride + d,
//   page = slot / page_size, offset = slot % page_size; slot -1 writes nothing.
// k_cache == null: this layer does not own a cache; only q is rotated.
// ------------------------------------------------------------------------------------------
template <typename T>
__global__ void rope_store_kernel(T* __restrict__ q_out, T* __restrict__ k_cache, T* __restrict__ v_cache,
                                  const T* __restrict__ qkv, const float* __restrict__ cos_sin,
                                  const int32_t* __restrict__ positions, const int64_t* __restrict__ slots,
                                  int nh, int nkv, int hd, int rotate, int page_size, int64_t page_stride,
                                  int64_t slot_stride, int64_t head_stride) {
  const int t = blockIdx.x;
  const int half = hd / 2;
  const int row = (nh + 2 * nkv) * hd;
  const T* src = qkv + (int64_t)t * row;
  const float* cs = cos_sin + (int64_t)positions[t] * hd;
  // q heads
  T* qo = q_out + (int64_t)t * nh * hd;
  for (int i = threadIdx.x; i < nh * half; i += blockDim.x) {
    const int h = i / half, j = i - h * half;
    const float x1 = Num<T>::ld(src + h * hd + j), x2 = Num<T>::ld(src + h * hd + j + half);
    float y1 = x1, y2 = x2;
    if (rotate) {
      const float c = cs[j], s = cs[half + j];
      y1 = x1 * c - x2 * s;
      y2 = x2 * c + x1 * s;
    }
    Num<T>::st(qo + h * hd + j, y1);
    Num<T>::st(qo + h * hd + j + half, y2);
  }
  if (!k_cache) return;
  const int64_t slot = slots[t];
  if (slot < 0) return;
  const int64_t base = (slot / page_size) * page_stride + (slot % page_size) * slot_stride;
  const T* ks = src + nh * hd;
  const T* vs = ks + nkv * hd;
  for (int i = threadIdx.x; i < nkv * half; i += blockDim.x) {
    const int h = i / half, j = i - h * half;
    const float x1 = Num<T>::ld(ks + h * hd + j), x2 = Num<T>::ld(ks + h * hd + j + half);
    float y1 = x1, y2 = x2;
    if (rotate) {
      const float c = cs[j], s = cs[half + j];
      y1 = x1 * c - x2 * s;
      y2 = x2 * c + x1 * s;
    }
    Num<T>::st(k_cache + base + h * head_stride + j, y1);
    Num<T>::st(k_cache + base + h * head_stride + j + half, y2);
  }
  for (int i = threadIdx.x; i < nkv * hd; i += blockDim.x) {
    const int h = i / hd;
    v_cache[base + h * head_stride + (i - h * hd)] = vs[i];
  }
}

extern "C" int ts_rope_store(void* q_out, void* k_cache, void* v_cache, const void* qkv, const float* cos_sin,
                             const int32_t* positions, const int64_t* slots, int num_tokens, int nh, int nkv,
                             int hd, int rotate, int page_size, int64_t page_stride, int64_t slot_stride,
                             int64_t head_stride, int dtype, hipStream_t stream) {
  if (num_tokens <= 0) return TS_OK;
  if (hd % 2 || nh <= 0 || nkv < 0 || page_size <= 0) return TS_BAD_SHAPE;
  if (dtype == 0)
    rope_store_kernel<float><<<num_tokens, 256, 0, stream>>>((float*)q_out, (float*)k_cache, (float*)v_cache,
                                                             (const float*)qkv, cos_sin, positions, slots, nh, nkv,
                                                             hd, rotate, page_size, page_stride, slot_stride, head_stride);
  else if (dtype == 1)
    rope_store_kernel<bf16_t><<<num_tokens, 256, 0, stream>>>((bf16_t*)q_out, (bf16_t*)k_cache, (bf16_t*)v_cache,
                                                              (const bf16_t*)qkv, cos_sin, positions, slots, nh, nkv,
                                                              hd, rotate, page_size, page_stride, slot_stride, head_stride);
  else
    return TS_BAD_DTYPE;
  return ts_check_launch();
}

// ------------------------------------------------------------------------------------------
// SiLU gate: out[t, i] = silu(gu[t, i]) * gu[t, inter + i]  (gate in the first half of a row)
// ------------------------------------------------------------------------------------------
template <typename T>
__global__ void silu_mul_kernel(T* __restrict__ out, const T* __restrict__ gu, int64_t total, int inter) {
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (int64_t)gridDim.x * blockDim.x) {
    const int64_t t = idx / inter;
    const int i = (int)(idx - t * inter);
    const float g = Num<T>::ld(gu + t * 2 * inter + i);
    const float u = Num<T>::ld(gu + t * 2 * inter + inter + i);
    const float a = g / (1.0f + expf(-g));
    Num<T>::st(out + idx, a * u);
  }
}

extern "C" int ts_silu_mul(void* out, const void* gu, int num_tokens, int inter, int dtype, hipStream_t stream) {
  const int64_t total = (int64_t)num_tokens * inter;
  if (total <= 0) return TS_OK;
  int64_t blocks = (total + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  if (dtype == 0)
    silu_mul_kernel<float><<<(int)blocks, 256, 0, stream>>>((float*)out, (const float*)gu, total, inter);
  else if (dtype == 1)
    silu_mul_kernel<bf16_t><<<(int)blocks, 256, 0, stream>>>((bf16_t*)out, (const bf16_t*)gu, total, inter);
  else
    return TS_BAD_DTYPE;
  return ts_check_launch();
}

// ------------------------------------------------------------------------------------------
// Copy the first `num_slots` slots of page `src` to page `dst` in a pool laid out
// [pages, runs, page_size, row]: `runs` = layers x kv heads of the group, row = one head's
// head_dim elements in bytes.
// ------------------------------------------------------------------------------------------
__global__ void copy_slots_kernel(uint8_t* __restrict__ pool, int64_t page_bytes, int64_t layer_bytes,
                                  int64_t copy_bytes, int src, int dst) {
  const int layer = blockIdx.y;
  const uint8_t* s = pool + src * page_bytes + layer * layer_bytes;
  uint8_t* d = pool + dst * page_bytes + layer * layer_bytes;
  // rows are multiples of 4 bytes (an even head_dim of 2-byte elements at least)
  const int64_t words = copy_bytes / 4;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < words; i += (int64_t)gridDim.x * blockDim.x)
    ((uint32_t*)d)[i] = ((const uint32_t*)s)[i];
}

extern "C" int ts_copy_slots(void* pool, int num_layers, int page_size, int64_t row_bytes, int src, int dst,
                             int num_slots, hipStream_t stream) {
  if (num_slots <= 0 || num_layers <= 0) return TS_OK;
  if (num_slots > page_size || row_bytes % 4 || src == dst) return TS_BAD_SHAPE;
  const int64_t layer_bytes = (int64_t)page_size * row_bytes;
  const int64_t page_bytes = layer_bytes * num_layers;
  const int64_t copy_bytes = (int64_t)num_slots * row_bytes;
  int64_t bx = (copy_bytes / 4 + 255) / 256;
  if (bx > 64) bx = 64;
  if (bx < 1) bx = 1;
  copy_slots_kernel<<<dim3((int)bx, num_layers), 256, 0, stream>>>((uint8_t*)pool, page_bytes, layer_bytes,
                                                                    copy_bytes, src, dst);
  return ts_check_launch();
}
