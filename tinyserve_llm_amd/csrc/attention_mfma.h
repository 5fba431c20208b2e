// Building blocks of the matrix-core attention kernels (bfloat16): 32 keys at a time,
//     S^T[key, row] = K[key, :] · Q[row, :]        v_mfma_f32_16x16x16_bf16, keys as rows
//     online softmax per row (32-bit, in units of log2), P = 2^(S - max)
//     O[row, :]    += P[row, key] · V[key, :]
// for a tile of 16 rows, a row being one (token, query head) pair of one key/value head's group.
// The result layout of the first product is the operand layout of the second, so P never leaves
// its registers. Keys are read as 16-byte pieces of their rows; values are read from pages that
// hold them transposed ([head_dim, page_size] per head), so that the consecutive keys an operand
// needs lie side by side in memory.
#pragma once
#include "common.h"

typedef short short4_t __attribute__((ext_vector_type(4)));
typedef float float4_t __attribute__((ext_vector_type(4)));

static __device__ __forceinline__ short4_t lo_half(const uint4& v) {
  return __builtin_bit_cast(short4_t, make_uint2(v.x, v.y));
}
static __device__ __forceinline__ short4_t hi_half(const uint4& v) {
  return __builtin_bit_cast(short4_t, make_uint2(v.z, v.w));
}
// probabilities are finite and in [0, 1]: round to nearest even without the NaN case
static __device__ __forceinline__ short4_t pack_bf16(float a, float b, float c, float d) {
  const float f[4] = {a, b, c, d};
  short4_t r;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const uint32_t u = __float_as_uint(f[i]);
    r[i] = (short)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
  }
  return r;
}

// 2^x by the hardware's exponential; scores are kept in units of log2 so that one multiply
// (scale * log2 e) is all the softmax needs besides it
static __device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

struct PageMath {   // key -> (page index in the table, slot inside the page)
  int size, shift;  // shift >= 0: the page size is 2^shift
  __device__ __forceinline__ int page(int key) const { return shift >= 0 ? key >> shift : key / size; }
  __device__ __forceinline__ int slot(int key, int pg) const { return key - pg * size; }
};

template <int HD> struct KVTile {
  uint4 k[2][HD / 32];   // two 16-key tiles as A operands: row i of tile tau is key kb + 8 (i / 4) + 4 tau + i % 4
  uint4 v[HD / 16];      // transposed values: keys kb + 8 g .. + 7 of dimension 16 db + r
};

template <int HD>
static __device__ __forceinline__ void load_tile(KVTile<HD>& T, int kb, int r, int g, int lo, int pos, int kvh,
                                                 const int32_t* __restrict__ table, const PageMath pm,
                                                 const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
                                                 int64_t kp, int64_t ks, int64_t kh, int64_t vp, int64_t vh,
                                                 int64_t vd) {
  constexpr int NC = HD / 32, NDB = HD / 16;
#pragma unroll
  for (int tau = 0; tau < 2; ++tau) {
    const int key = kb + 8 * (r >> 2) + 4 * tau + (r & 3);
#pragma unroll
    for (int c = 0; c < NC; ++c) T.k[tau][c] = make_uint4(0, 0, 0, 0);
    if (key <= pos && key >= lo) {
      const int pg = pm.page(key);
      const bf16_t* kr = k_cache + (int64_t)table[pg] * kp + (int64_t)pm.slot(key, pg) * ks + (int64_t)kvh * kh + 8 * g;
#pragma unroll
      for (int c = 0; c < NC; ++c) T.k[tau][c] = *(const uint4*)(kr + 32 * c);
    }
  }
  const int vkey = kb + 8 * g;
#pragma unroll
  for (int db = 0; db < NDB; ++db) T.v[db] = make_uint4(0, 0, 0, 0);
  if (vkey <= pos && vkey + 7 >= lo) {
    const int pg = pm.page(vkey);
    const bf16_t* vr = v_cache + (int64_t)table[pg] * vp + pm.slot(vkey, pg) + (int64_t)kvh * vh + (int64_t)r * vd;
#pragma unroll
    for (int db = 0; db < NDB; ++db) T.v[db] = *(const uint4*)(vr + (int64_t)(16 * db) * vd);
  }
}

// One 32-key step of the online softmax for the 16 rows that `qreg` holds (lane r = row r of the
// score tile; output row 4 g + j). `m` is the running max in units of log2, `l` the running sum.
template <int HD>
static __device__ __forceinline__ void use_tile(const KVTile<HD>& T, int kb, int g, int lo, int pos,
                                                const uint4 (&qreg)[HD / 32], float scale2, float& m, float& l,
                                                float4_t (&o)[HD / 16]) {
  constexpr int NC = HD / 32, NDB = HD / 16;
  float4_t s[2];
#pragma unroll
  for (int tau = 0; tau < 2; ++tau) {
    s[tau] = (float4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      s[tau] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(lo_half(T.k[tau][c]), lo_half(qreg[c]), s[tau], 0, 0, 0);
      s[tau] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(hi_half(T.k[tau][c]), hi_half(qreg[c]), s[tau], 0, 0, 0);
    }
  }
  // this lane: row r, keys kb + 8 g + 4 tau + j
  float sv[2][4];
  float mloc = -INFINITY;
#pragma unroll
  for (int tau = 0; tau < 2; ++tau)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int key = kb + 8 * g + 4 * tau + j;
      sv[tau][j] = (key <= pos && key >= lo) ? s[tau][j] * scale2 : -INFINITY;
      mloc = fmaxf(mloc, sv[tau][j]);
    }
  mloc = fmaxf(mloc, __shfl_xor(mloc, 16, TS_WAVE));
  mloc = fmaxf(mloc, __shfl_xor(mloc, 32, TS_WAVE));
  const float m_new = fmaxf(m, mloc);
  const float m_safe = m_new == -INFINITY ? 0.f : m_new;   // nothing visible yet: every term below is 0
  const float alpha = fast_exp2(m - m_safe);
  float p[2][4];
  float lsum = 0.f;
#pragma unroll
  for (int tau = 0; tau < 2; ++tau)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      p[tau][j] = fast_exp2(sv[tau][j] - m_safe);
      lsum += p[tau][j];
    }
  lsum += __shfl_xor(lsum, 16, TS_WAVE);
  lsum += __shfl_xor(lsum, 32, TS_WAVE);
  l = l * alpha + lsum;
  m = m_new;
  // output row 4 g + j belongs to score row 4 g + j, whose alpha lane 4 g + j holds
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const float aj = __shfl(alpha, 4 * g + j, TS_WAVE);
#pragma unroll
    for (int db = 0; db < NDB; ++db) o[db][j] *= aj;
  }
  const short4_t pa0 = pack_bf16(p[0][0], p[0][1], p[0][2], p[0][3]);
  const short4_t pa1 = pack_bf16(p[1][0], p[1][1], p[1][2], p[1][3]);
#pragma unroll
  for (int db = 0; db < NDB; ++db) {
    o[db] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(pa0, lo_half(T.v[db]), o[db], 0, 0, 0);
    o[db] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(pa1, hi_half(T.v[db]), o[db], 0, 0, 0);
  }
}

