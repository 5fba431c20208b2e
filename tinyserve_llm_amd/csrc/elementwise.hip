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
  constexpr int V = 16 / sizeof(T);
  if (hidden % V == 0 && (((uintptr_t)table | (uintptr_t)out) & 15) == 0) {
    for (int i = threadIdx.x; i < hidden / V; i += blockDim.x) ((uint4*)dst)[i] = ((const uint4*)src)[i];
  } else {
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) dst[i] = src[i];
  }
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
#define NORM_MAX_CHUNKS 4     // 16-byte pieces of a row that a thread of the single-pass kernel keeps

template <typename T> struct Pack16;   // a 16-byte piece of a row as floats
template <> struct Pack16<float> {
  static constexpr int N = 4;
  static __device__ __forceinline__ void unpack(const uint4 v, float* f) {
    f[0] = __uint_as_float(v.x); f[1] = __uint_as_float(v.y); f[2] = __uint_as_float(v.z); f[3] = __uint_as_float(v.w);
  }
  static __device__ __forceinline__ void ld(const float* p, float* f) { unpack(*(const uint4*)p, f); }
  static __device__ __forceinline__ void st(float* p, const float* f) { *(float4*)p = make_float4(f[0], f[1], f[2], f[3]); }
};
template <> struct Pack16<bf16_t> {
  static constexpr int N = 8;
  static __device__ __forceinline__ void unpack(const uint4 v, float* f) {
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f[2 * i] = __uint_as_float(w[i] << 16);
      f[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
  }
  static __device__ __forceinline__ void ld(const bf16_t* p, float* f) { unpack(*(const uint4*)p, f); }
  static __device__ __forceinline__ void st(bf16_t* p, const float* f) {
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) w[i] = (uint32_t)f2bf(f[2 * i]) | ((uint32_t)f2bf(f[2 * i + 1]) << 16);
    *(uint4*)p = make_uint4(w[0], w[1], w[2], w[3]);
  }
};

// The general form: two passes over the row, any width, any weight storage.
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

// One pass: a thread keeps its 16-byte pieces of the row in registers between the sum of squares
// and the scaling. For rows of up to 256 * NORM_MAX_CHUNKS pieces whose width is a whole number of
// pieces. The order of the sums differs from the general form's but is as fixed per row; which of
// the two runs depends on the width and the storage types only, never on the batch.
template <typename T>
__global__ void __launch_bounds__(NORM_THREADS)
rmsnorm_row_kernel(T* __restrict__ out, T* __restrict__ res_out, const T* __restrict__ x, const T* __restrict__ res,
                   const T* __restrict__ w, const int32_t* __restrict__ rows, int hidden, float eps) {
  constexpr int N = Pack16<T>::N;
  __shared__ float partial[NORM_THREADS / TS_WAVE];
  const int r = blockIdx.x;
  const int64_t src = rows ? (int64_t)rows[r] : (int64_t)r;
  const T* xr = x + src * hidden;
  const T* rr = res ? res + src * hidden : nullptr;
  const int pieces = hidden / N;
  float v[NORM_MAX_CHUNKS][N];
  // everything the thread reads is asked for at once, the weights' pieces too, which are used only after the
  // barrier (without a residual the row is asked for twice, the second time from the cache: no test stands
  // between the loads that would make one wait for the other)
  uint4 xraw[NORM_MAX_CHUNKS], rraw[NORM_MAX_CHUNKS], wraw[NORM_MAX_CHUNKS];
  const T* rsrc = rr ? rr : xr;
#pragma unroll
  for (int c = 0; c < NORM_MAX_CHUNKS; ++c) {
    const int i = threadIdx.x + c * NORM_THREADS;
    if (i < pieces) {
      xraw[c] = *(const uint4*)(xr + (int64_t)i * N);
      rraw[c] = *(const uint4*)(rsrc + (int64_t)i * N);
      wraw[c] = *(const uint4*)(w + (int64_t)i * N);
    }
  }
  float acc = 0.f;
#pragma unroll
  for (int c = 0; c < NORM_MAX_CHUNKS; ++c) {
    const int i = threadIdx.x + c * NORM_THREADS;
    if (i < pieces) {
      Pack16<T>::unpack(xraw[c], v[c]);
      if (rr) {
        float t[N];
        Pack16<T>::unpack(rraw[c], t);
#pragma unroll
        for (int k = 0; k < N; ++k) v[c][k] += t[k];
      }
#pragma unroll
      for (int k = 0; k < N; ++k) acc = fmaf(v[c][k], v[c][k], acc);
    }
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
#pragma unroll
  for (int c = 0; c < NORM_MAX_CHUNKS; ++c) {
    const int i = threadIdx.x + c * NORM_THREADS;
    if (i < pieces) {
      if (rorow) Pack16<T>::st(rorow + (int64_t)i * N, v[c]);
      float wv[N];
      Pack16<T>::unpack(wraw[c], wv);
#pragma unroll
      for (int k = 0; k < N; ++k) v[c][k] = Num<T>::round(v[c][k] * inv) * wv[k];
      Pack16<T>::st(orow + (int64_t)i * N, v[c]);
    }
  }
}

// wdtype: storage of the weight vector (0 float, 1 bfloat16); dtype: storage of activations.
extern "C" int ts_rmsnorm(void* out, void* res_out, const void* x, const void* res, const void* w,
                          const int32_t* rows, int num_rows, int hidden, float eps, int dtype,
                          int wdtype, hipStream_t stream) {
  if (num_rows <= 0) return TS_OK;
  dim3 grid(num_rows), block(NORM_THREADS);
  const int per16 = dtype == 0 ? 4 : 8;
  const bool aligned = ((((uintptr_t)out) | ((uintptr_t)res_out) | ((uintptr_t)x) | ((uintptr_t)res) | ((uintptr_t)w)) & 15) == 0;
  if (dtype == wdtype && aligned && hidden % per16 == 0 && hidden / per16 <= NORM_THREADS * NORM_MAX_CHUNKS) {
    if (dtype == 0)
      rmsnorm_row_kernel<float><<<grid, block, 0, stream>>>((float*)out, (float*)res_out, (const float*)x,
                                                            (const float*)res, (const float*)w, rows, hidden, eps);
    else if (dtype == 1)
      rmsnorm_row_kernel<bf16_t><<<grid, block, 0, stream>>>((bf16_t*)out, (bf16_t*)res_out, (const bf16_t*)x,
                                                             (const bf16_t*)res, (const bf16_t*)w, rows, hidden, eps);
    else
      return TS_BAD_DTYPE;
    return ts_check_launch();
  }
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
// Rotate-half RoPE on q and k from a 32-bit [max_pos, rot] table ([cos | sin] halves), fused with the
// scatter of rotated k and of v into their cache slots. rot <= head_dim is the rotated width: dimension
// j < rot / 2 of a head turns with dimension j + rot / 2, the dimensions from rot on pass as they are.
//   qkv   [T, (nh + 2*nkv) * hd]   one token's q heads, then k heads, then v heads
//   q_out [T, nh * hd]
//   key element address:   page * kp + offset * ks + head * kh + d          (d dense)
//   value element address: page * vp + offset * vs + head * vh + d * vd     (any layout: the engine
//                          keeps values transposed inside a page, vs = 1 and vd = page_size)
//   page = slot / page_size, offset = slot % page_size; slot -1 writes nothing.
// k_cache == null: this layer does not own a cache; only q is rotated.
// A workgroup takes ROPE_TOK consecutive tokens and one of gridDim.y slices of their elements
// (few tokens are spread over more workgroups); value elements are assigned token-fastest so that
// neighbouring threads write neighbouring slots of a transposed page.
// ------------------------------------------------------------------------------------------
#define ROPE_TOK 16
#define ROPE_VTILE 256     // value elements of a token that pass through LDS at a time

template <typename T>
__global__ void rope_store_kernel(T* __restrict__ q_out, T* __restrict__ k_cache, T* __restrict__ v_cache,
                                  const T* __restrict__ qkv, const float* __restrict__ cos_sin,
                                  const int32_t* __restrict__ positions, const int32_t* __restrict__ slots,
                                  int num_tokens, int nh, int nkv, int hd, int rot, int rotate, int page_size, int64_t kp,
                                  int64_t ks, int64_t kh, int64_t vp, int64_t vs, int64_t vh, int64_t vd, int vec, int vtile,
                                  int v_slices) {
  const int t0 = blockIdx.x * ROPE_TOK;
  const int nt = num_tokens - t0 < ROPE_TOK ? num_tokens - t0 : ROPE_TOK;
  const int half = rot / 2, rest = hd - rot;          // pairs that turn, and dimensions that pass
  // v_slices > 0: the last v_slices of the gridDim.y slices write the values, the others rotate q
  // and k (the two are independent chains of loads and stores: side by side they take half the
  // time); v_slices == 0: every workgroup does its slice of both
  int by = blockIdx.y, ny = gridDim.y;
  bool do_qk = true, do_v = true;
  if (v_slices > 0) {
    const int qk_slices = gridDim.y - v_slices;
    if (by < qk_slices) { do_v = false; ny = qk_slices; }
    else { do_qk = false; by -= qk_slices; ny = v_slices; }
  }
  // slot -> (page, offset) in 32-bit arithmetic; a shift where the page size is a power of two
  const int page_shift = (page_size & (page_size - 1)) == 0 ? __builtin_ctz(page_size) : -1;
  auto page_of = [&](int slot) { return page_shift >= 0 ? slot >> page_shift : slot / page_size; };
  const int row = (nh + 2 * nkv) * hd;
  const int per_head_items = half + rest;             // a pair or a passing dimension each
  const int qpairs = nh * per_head_items, kpairs = nkv * per_head_items;
  // q and k items of every token of the group: this workgroup's slice of them
  const int npairs = nt * (qpairs + kpairs);
  constexpr int V = 16 / sizeof(T);
  if (!do_qk) {
  } else if (vec) {
    // 16 bytes of each half of a head's rotated part at a time, then 16 bytes of what passes
    const int turning = half / V, per_head = turning + rest / V;
    const int npieces = nt * (nh + nkv) * per_head;
    const int pbeg = (int)((int64_t)npieces * by / ny), pend = (int)((int64_t)npieces * (by + 1) / ny);
    for (int i = pbeg + threadIdx.x; i < pend; i += blockDim.x) {
      const int tl = i / ((nh + nkv) * per_head), e = i - tl * ((nh + nkv) * per_head);
      const int t = t0 + tl;
      const int h = e / per_head, piece = e - h * per_head;
      const bool is_k = h >= nh, passes = piece >= turning;
      const int j = passes ? rot + (piece - turning) * V : piece * V;
      if (is_k && !k_cache) continue;
      // the token's slot and position and both pieces are asked for together (a piece that passes asks for
      // itself twice), then the table's rows for the position: two trips to memory, not four
      const T* src = qkv + (int64_t)t * row + h * hd;      // k heads follow the q heads in a row
      const int slot = k_cache ? slots[t] : 0, position = positions[t];
      const uint4 raw1 = *(const uint4*)(src + j), raw2 = *(const uint4*)(src + (passes ? j : j + half));
      float x1[V], x2[V];
      Pack16<T>::unpack(raw1, x1);
      Pack16<T>::unpack(raw2, x2);
      if (rotate && !passes) {
        const float* cs = cos_sin + (int64_t)position * rot + j;      // (16-byte aligned: rot and j are multiples of V)
        float c[V], sn[V];
#pragma unroll
        for (int k = 0; k < V; k += 4) {
          const float4 cv = *(const float4*)(cs + k), sv = *(const float4*)(cs + half + k);
          c[k] = cv.x; c[k + 1] = cv.y; c[k + 2] = cv.z; c[k + 3] = cv.w;
          sn[k] = sv.x; sn[k + 1] = sv.y; sn[k + 2] = sv.z; sn[k + 3] = sv.w;
        }
#pragma unroll
        for (int k = 0; k < V; ++k) {
          const float y1 = x1[k] * c[k] - x2[k] * sn[k], y2 = x2[k] * c[k] + x1[k] * sn[k];
          x1[k] = y1;
          x2[k] = y2;
        }
      }
      if (is_k && slot < 0) continue;
      T* dst;
      if (is_k) {
        const int pg = page_of(slot);
        dst = k_cache + (int64_t)pg * kp + (int64_t)(slot - pg * page_size) * ks + (int64_t)(h - nh) * kh;
      } else {
        dst = q_out + ((int64_t)t * nh + h) * hd;
      }
      Pack16<T>::st(dst + j, x1);
      if (!passes) Pack16<T>::st(dst + j + half, x2);
    }
  } else {
  const int pbeg = (int)((int64_t)npairs * by / ny), pend = (int)((int64_t)npairs * (by + 1) / ny);
  for (int i = pbeg + threadIdx.x; i < pend; i += blockDim.x) {
    const int tl = i / (qpairs + kpairs), e = i - tl * (qpairs + kpairs);
    const int t = t0 + tl;
    const bool is_k = e >= qpairs;
    const int pe = is_k ? e - qpairs : e;
    const int h = pe / per_head_items, item = pe - h * per_head_items;
    const bool passes = item >= half;
    const int j = passes ? rot + (item - half) : item;
    const T* src = qkv + (int64_t)t * row + (is_k ? nh * hd : 0) + h * hd;
    if (is_k && (!k_cache || slots[t] < 0)) continue;
    const float x1 = Num<T>::ld(src + j), x2 = passes ? 0.f : Num<T>::ld(src + j + half);
    float y1 = x1, y2 = x2;
    if (rotate && !passes) {
      const float* cs = cos_sin + (int64_t)positions[t] * rot;
      const float c = cs[j], sn = cs[half + j];
      y1 = x1 * c - x2 * sn;
      y2 = x2 * c + x1 * sn;
    }
    T* dst;
    if (is_k) {
      const int slot = slots[t], pg = page_of(slot);
      dst = k_cache + (int64_t)pg * kp + (int64_t)(slot - pg * page_size) * ks + (int64_t)h * kh;
    } else {
      dst = q_out + ((int64_t)t * nh + h) * hd;
    }
    Num<T>::st(dst + j, y1);
    if (!passes) Num<T>::st(dst + j + half, y2);
  }
  }
  if (!k_cache || !do_v) return;
  const int vel = nkv * hd;
  if (vtile) {
    // values through LDS: rows of the step are read 16 bytes at a time, then every thread takes one
    // (head, dimension) and writes its 8 consecutive tokens as one 16-byte piece of a transposed
    // page where their slots are consecutive, aligned and inside one page
    __shared__ T tile[ROPE_TOK][ROPE_VTILE];
    __shared__ int base_slot[ROPE_TOK / 8];          // first slot of each run of 8 tokens, or -1: no fast path
    __shared__ int slot_of[ROPE_TOK];                // the group's slots (tokens that are not there: -1), fetched once
    constexpr int VP = 16 / sizeof(T);                // elements of a 16-byte piece
    static_assert(VP == 8 || sizeof(T) == 4, "runs of 8 tokens are pieces of bfloat16");
    if (threadIdx.x < ROPE_TOK / 8) {
      // a thread per run of 8 tokens: their slots (tokens that are not there: -1), kept for the slow path, and
      // whether they are consecutive, aligned and inside one page
      const int first = 8 * threadIdx.x;
      int sl[8];
#pragma unroll
      for (int k = 0; k < 8; ++k) sl[k] = slots[t0 + min(first + k, nt - 1)];      // (no test between the loads: one trip)
#pragma unroll
      for (int k = 0; k < 8; ++k) sl[k] = first + k < nt ? sl[k] : -1;
      int s0 = sl[0];
      bool ok = s0 >= 0 && s0 % 8 == 0 && s0 % page_size + 7 < page_size;
#pragma unroll
      for (int k = 1; k < 8; ++k) ok = ok & (sl[k] == s0 + k);
#pragma unroll
      for (int k = 0; k < 8; ++k) slot_of[first + k] = sl[k];
      base_slot[threadIdx.x] = ok ? s0 : -1;
    }
    const int ebeg = (int)((int64_t)(vel / VP) * by / ny) * VP;
    const int eend = (int)((int64_t)(vel / VP) * (by + 1) / ny) * VP;
    for (int eb = ebeg; eb < eend; eb += ROPE_VTILE) {
      __syncthreads();                                // the previous tile has been read (and base_slot written)
      for (int p = threadIdx.x; p < ROPE_TOK * (ROPE_VTILE / VP); p += blockDim.x) {
        const int tl = p / (ROPE_VTILE / VP), e = eb + (p % (ROPE_VTILE / VP)) * VP;
        if (tl < nt && e < eend)
          *(uint4*)&tile[tl][e - eb] = *(const uint4*)(qkv + (int64_t)(t0 + tl) * row + (nh + nkv) * hd + e);
      }
      __syncthreads();
      // (two loops, chosen by the workgroup as a whole: with the scattered stores inside the fast loop the compiler
      // works out all sixteen tokens' pages before it looks whether it needs them)
      bool all_runs = sizeof(T) == 2;
#pragma unroll
      for (int run = 0; run < ROPE_TOK / 8; ++run) all_runs = all_runs && base_slot[run] >= 0;
      if (all_runs) {
        for (int el = threadIdx.x; el < ROPE_VTILE && eb + el < eend; el += blockDim.x) {
          const int e = eb + el, h = e / hd, d = e - h * hd;
#pragma unroll
          for (int run = 0; run < ROPE_TOK / 8; ++run) {
            const int s0 = base_slot[run];
            uint32_t w[4];
#pragma unroll
            for (int k = 0; k < 4; ++k)
              w[k] = (uint32_t)(*(const uint16_t*)&tile[8 * run + 2 * k][el]) |
                     ((uint32_t)(*(const uint16_t*)&tile[8 * run + 2 * k + 1][el]) << 16);
            const int pg = page_of(s0);
            *(uint4*)(v_cache + (int64_t)pg * vp + (s0 - pg * page_size) + (int64_t)h * vh + (int64_t)d * vd) =
                make_uint4(w[0], w[1], w[2], w[3]);
          }
        }
      } else {
        // tokens of different requests, or a run that is not whole: a store per token, its slot out of LDS
        for (int el = threadIdx.x; el < ROPE_VTILE && eb + el < eend; el += blockDim.x) {
          const int e = eb + el, h = e / hd, d = e - h * hd;
#pragma unroll
          for (int tl = 0; tl < ROPE_TOK; ++tl) {
            const int slot = slot_of[tl];
            if (slot < 0) continue;
            const int pg = page_of(slot);
            v_cache[(int64_t)pg * vp + (int64_t)(slot - pg * page_size) * vs + (int64_t)h * vh + (int64_t)d * vd] = tile[tl][el];
          }
        }
      }
    }
    return;
  }
  // values: thread -> (element, token), token fastest
  const int vbeg = (int)((int64_t)vel * by / ny) * ROPE_TOK;
  const int vend = (int)((int64_t)vel * (by + 1) / ny) * ROPE_TOK;
  for (int i = vbeg + threadIdx.x; i < vend; i += blockDim.x) {
    const int tl = i % ROPE_TOK, e = i / ROPE_TOK;
    if (tl >= nt) continue;
    const int t = t0 + tl;
    const int slot = slots[t];
    if (slot < 0) continue;
    const int h = e / hd, d = e - h * hd, pg = page_of(slot);
    v_cache[(int64_t)pg * vp + (int64_t)(slot - pg * page_size) * vs + (int64_t)h * vh + (int64_t)d * vd] =
        qkv[(int64_t)t * row + (nh + nkv) * hd + e];
  }
}

extern "C" int ts_rope_store(void* q_out, void* k_cache, void* v_cache, const void* qkv, const float* cos_sin,
                             const int32_t* positions, const int32_t* slots, int num_tokens, int nh, int nkv,
                             int hd, int rot, int rotate, int page_size, int64_t kp, int64_t ks, int64_t kh, int64_t vp,
                             int64_t vs, int64_t vh, int64_t vd, int dtype, hipStream_t stream) {
  if (num_tokens <= 0) return TS_OK;
  if (hd <= 0 || rot % 2 || rot < 0 || rot > hd || nh <= 0 || nkv < 0 || page_size <= 0) return TS_BAD_SHAPE;
  if (!rotate) rot = hd - hd % 2;                     // (nothing turns: the split into pairs is free)
  const int groups = (num_tokens + ROPE_TOK - 1) / ROPE_TOK;
  int slices = 2048 / groups;                       // enough workgroups to hide the loads' latency
  if (slices < 1) slices = 1;
  if (slices > 32) slices = 32;
  // (no more slices than give each of a workgroup's threads a piece of q or k)
  const int group_pieces = ROPE_TOK * (nh + nkv) * ((hd + (dtype == 0 ? 4 : 8) - 1) / (dtype == 0 ? 4 : 8)) / 2;
  if (slices > (group_pieces + 255) / 256) slices = (group_pieces + 255) / 256;
  dim3 blocks(groups, slices);
  // 16-byte pieces need halves of whole pieces and aligned rows everywhere
  const int per16 = dtype == 0 ? 4 : 8;
  const int row = (nh + 2 * nkv) * hd;
  const int vec = (rot / 2) % per16 == 0 && (hd - rot) % per16 == 0 && hd % per16 == 0 && row % per16 == 0 && kp % per16 == 0 && ks % per16 == 0 && kh % per16 == 0 &&
                  ((((uintptr_t)q_out) | ((uintptr_t)k_cache) | ((uintptr_t)qkv) | ((uintptr_t)cos_sin)) & 15) == 0;
  // values through LDS: bfloat16 steps of several tokens into transposed pages (slot stride 1) whose
  // 8-slot pieces are 16-byte aligned
  const int vtile = dtype == 1 && num_tokens >= 8 && v_cache && vs == 1 && row % 8 == 0 && ((nh + nkv) * hd) % 8 == 0 &&
                    (nkv * hd) % 8 == 0 && page_size % 8 == 0 && vp % 8 == 0 && vh % 8 == 0 && vd % 8 == 0 &&
                    ((((uintptr_t)v_cache) | ((uintptr_t)qkv)) & 15) == 0;
  int v_slices = 0;
  if (vtile) {                                        // values are a sixth or so of the work
    v_slices = slices / 4 > 0 ? slices / 4 : 1;
    blocks.y = slices + v_slices;
  }
  if (dtype == 0)
    rope_store_kernel<float><<<blocks, 256, 0, stream>>>((float*)q_out, (float*)k_cache, (float*)v_cache,
                                                         (const float*)qkv, cos_sin, positions, slots, num_tokens, nh,
                                                         nkv, hd, rot, rotate, page_size, kp, ks, kh, vp, vs, vh, vd, vec, 0, 0);
  else if (dtype == 1)
    rope_store_kernel<bf16_t><<<blocks, 256, 0, stream>>>((bf16_t*)q_out, (bf16_t*)k_cache, (bf16_t*)v_cache,
                                                          (const bf16_t*)qkv, cos_sin, positions, slots, num_tokens,
                                                          nh, nkv, hd, rot, rotate, page_size, kp, ks, kh, vp, vs, vh, vd, vec, vtile, v_slices);
  else
    return TS_BAD_DTYPE;
  return ts_check_launch();
}

// ------------------------------------------------------------------------------------------
// SiLU gate: out[t, i] = silu(gu[t, i]) * gu[t, inter + i]  (gate in the first half of a row)
// ------------------------------------------------------------------------------------------
// silu(g) for a result that is stored in 32 bits: the library's exponential and a true division. For bfloat16
// results the hardware's 2^x and reciprocal, each good to a unit in the last place of 32 bits (what the
// projections' gate epilogue uses): a piece of 8 elements costs a fifth of the instructions.
template <typename T> struct Gate;
template <> struct Gate<float> {
  static __device__ __forceinline__ float silu(float g) { return g / (1.0f + expf(-g)); }
};
template <> struct Gate<bf16_t> {
  static __device__ __forceinline__ float silu(float g) {
    return g * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.44269504088896340736f * g));
  }
};

template <typename T>
__global__ void silu_mul_kernel(T* __restrict__ out, const T* __restrict__ gu, int64_t total, int inter) {
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (int64_t)gridDim.x * blockDim.x) {
    const int64_t t = idx / inter;
    const int i = (int)(idx - t * inter);
    const float g = Num<T>::ld(gu + t * 2 * inter + i);
    const float u = Num<T>::ld(gu + t * 2 * inter + inter + i);
    Num<T>::st(out + idx, Gate<T>::silu(g) * u);
  }
}

// 16 bytes of gate and of up at a time, SILU_PIECES such pieces a thread (a workgroup's threads side by side in
// each), all of them asked for before the first is used; for widths that are whole numbers of pieces. A workgroup
// works on one token (blockIdx.x) and on 256 SILU_PIECES pieces of its row (blockIdx.y): nothing is divided.
#define SILU_PIECES 4
template <typename T>
__global__ void __launch_bounds__(256)
silu_mul_vec_kernel(T* __restrict__ out, const T* __restrict__ gu, int inter) {
  constexpr int N = Pack16<T>::N;
  const int per_row = inter / N;
  const T* row = gu + (int64_t)blockIdx.x * 2 * inter;
  T* orow = out + (int64_t)blockIdx.x * inter;
  const int first = blockIdx.y * (256 * SILU_PIECES) + threadIdx.x;
  uint4 graw[SILU_PIECES], uraw[SILU_PIECES];
#pragma unroll
  for (int p = 0; p < SILU_PIECES; ++p) {
    // (a piece past the row's end is its last piece once more: loads without a test between them all go out at once)
    const int i = min(first + p * 256, per_row - 1) * N;
    graw[p] = *(const uint4*)(row + i);
    uraw[p] = *(const uint4*)(row + inter + i);
  }
#pragma unroll
  for (int p = 0; p < SILU_PIECES; ++p) {
    float g[N], u[N];
    Pack16<T>::unpack(graw[p], g);
    Pack16<T>::unpack(uraw[p], u);
#pragma unroll
    for (int k = 0; k < N; ++k) g[k] = Gate<T>::silu(g[k]) * u[k];
    if (first + p * 256 < per_row) Pack16<T>::st(orow + (int64_t)(first + p * 256) * N, g);
  }
}

extern "C" int ts_silu_mul(void* out, const void* gu, int num_tokens, int inter, int dtype, hipStream_t stream) {
  const int64_t total = (int64_t)num_tokens * inter;
  if (total <= 0) return TS_OK;
  if (dtype != 0 && dtype != 1) return TS_BAD_DTYPE;
  const int per16 = dtype == 0 ? 4 : 8;
  if (inter % per16 == 0 && ((((uintptr_t)out) | ((uintptr_t)gu)) & 15) == 0) {
    const int chunks = (inter / per16 + 256 * SILU_PIECES - 1) / (256 * SILU_PIECES);
    if (chunks > 65535) return TS_BAD_SHAPE;
    const dim3 blocks(num_tokens, chunks);
    if (dtype == 0)
      silu_mul_vec_kernel<float><<<blocks, 256, 0, stream>>>((float*)out, (const float*)gu, inter);
    else
      silu_mul_vec_kernel<bf16_t><<<blocks, 256, 0, stream>>>((bf16_t*)out, (const bf16_t*)gu, inter);
    return ts_check_launch();
  }
  int64_t blocks = (total + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  if (dtype == 0)
    silu_mul_kernel<float><<<(int)blocks, 256, 0, stream>>>((float*)out, (const float*)gu, total, inter);
  else
    silu_mul_kernel<bf16_t><<<(int)blocks, 256, 0, stream>>>((bf16_t*)out, (const bf16_t*)gu, total, inter);
  return ts_check_launch();
}

// ------------------------------------------------------------------------------------------
// Copy the leading part of every run of page `src` to page `dst`. A page of a pool is `runs` runs of
// `run_units` 2-byte units; the first `copy_units` of each run are copied. For keys
// [pages, layers, heads, page_size, head_dim] a run is one head's slots and the leading part is the
// first n slots; for transposed values [pages, layers, heads, head_dim, page_size] a run is one
// dimension's slots.
// ------------------------------------------------------------------------------------------
__global__ void copy_slots_kernel(uint16_t* __restrict__ pool, int64_t page_units, int64_t run_units,
                                  int64_t copy_units, int64_t total, int src, int dst) {
  const uint16_t* s = pool + src * page_units;
  uint16_t* d = pool + dst * page_units;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t run = i / copy_units, o = i - run * copy_units;
    d[run * run_units + o] = s[run * run_units + o];
  }
}

extern "C" int ts_copy_slots(void* pool, int64_t runs, int64_t run_bytes, int64_t copy_bytes, int src, int dst,
                             hipStream_t stream) {
  if (copy_bytes <= 0 || runs <= 0) return TS_OK;
  if (copy_bytes > run_bytes || run_bytes % 2 || copy_bytes % 2 || src == dst || src < 0 || dst < 0)
    return TS_BAD_SHAPE;
  const int64_t total = runs * (copy_bytes / 2);
  int64_t blocks = (total + 255) / 256;
  if (blocks > 4096) blocks = 4096;
  copy_slots_kernel<<<(int)blocks, 256, 0, stream>>>((uint16_t*)pool, runs * (run_bytes / 2), run_bytes / 2,
                                                     copy_bytes / 2, total, src, dst);
  return ts_check_launch();
}
