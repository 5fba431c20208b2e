// Building blocks of the matrix-core attention kernels (bfloat16): 32 keys at a time,
//     S^T[key, row] = K[key, :] · Q[row, :]        v_mfma_f32_16x16x32_bf16, keys as rows
//     online softmax per row (32-bit, in units of log2), P = 2^(S - m)
//     O[row, :]    += P[row, key] · V[key, :]
// for a tile of 16 rows, a row being one (token, query head) pair of one key/value head's group.
// m follows the row's running maximum lazily: it is raised (and the sums rescaled) only when a score
// exceeds it by more than 2^8, so that most steps need no exchange between lanes; P stays below 2^8,
// the sums are 32-bit, and a row's m depends on that row's scores alone. Each lane sums the P of its
// own keys; the four lanes of a row add theirs up once, at the end (`row_sum`). Or, where the vector
// unit is what bounds the kernel (prompt portions), the matrix cores sum P as well: one more product,
// of P with a matrix of ones, gives every row's sum in the layout of the output rows.
// The result layout of the first product is the operand layout of the second, so P never leaves
// its registers. Keys are read as 16-byte pieces of their rows; values are read from pages that
// hold them transposed ([head_dim, page_size] per head), so that the consecutive keys an operand
// needs lie side by side in memory.
#pragma once
#include <type_traits>
#include "common.h"

typedef float float4_t __attribute__((ext_vector_type(4)));

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
// acc + A · B over 32 k: lane (r, g) gives eight consecutive k (8 g .. 8 g + 7) of row r of A and of
// column r of B, 16 bytes each (v_mfma_f32_16x16x32_bf16); lane (r, g) gets D[4 g + j][r], j = 0..3
static __device__ __forceinline__ float4_t mfma32(const uint4& a, const uint4& b, float4_t acc) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), acc, 0, 0, 0);
}
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float float2_t __attribute__((ext_vector_type(2)));
// two floats to a pair of bfloat16, round to nearest even (the hardware's packed conversion)
static __device__ __forceinline__ uint32_t pack_bf16(float a, float b) {
  return __builtin_bit_cast(uint32_t, __builtin_convertvector((float2_t){a, b}, bf16x2_t));
}

// 2^x by the hardware's exponential; scores are kept in units of log2 so that one multiply
// (scale * log2 e) is all the softmax needs besides it
static __device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

struct PageMath {   // key -> (page index in the request, slot inside the page)
  int size, shift;  // shift >= 0: the page size is 2^shift
  int run = 0;      // an entry of a request's page table names 2^run consecutive pages of the pool: entry e the pages
                    // e 2^run .. e 2^run + 2^run - 1 (the pools may be cut into shorter pages than the tables count in)
  __device__ __forceinline__ int page(int key) const { return shift >= 0 ? key >> shift : key / size; }
  __device__ __forceinline__ int slot(int key, int pg) const { return key - pg * size; }
  // the pool's page that is page pg of the request whose table this is
  __device__ __forceinline__ int64_t pool_page(const int32_t* __restrict__ table, int pg) const {
    return ((int64_t)table[pg >> run] << run) + (pg & ((1 << run) - 1));
  }
  // pages of a multiple of 32 keys: a 32-key step (kb a multiple of 32) lies inside one page, and
  // its table entry is one scalar lookup for the whole wave
  __device__ __forceinline__ bool whole_steps() const { return (size & 31) == 0; }
};

// the wave's index in its workgroup, as a scalar the compiler knows to be uniform
static __device__ __forceinline__ int wave_index() { return __builtin_amdgcn_readfirstlane(threadIdx.x / TS_WAVE); }

template <int HD> struct KVTile {
  uint4 k[2][HD / 32];   // two 16-key tiles as A operands: row i of tile tau is key kb + 8 (i / 4) + 4 tau + i % 4
  uint4 v[HD / 16];      // transposed values: keys kb + 8 g .. + 7 of dimension 16 db + r
  bool vok;              // whether any of this lane's eight keys of v is visible (else v may hold anything and counts as zeros)
};

// Exchanges between the four lanes (r, g = 0..3) that share a row, by the register swaps of the
// hardware: after v_permlane16_swap of x with itself one result holds the even rows of 16 lanes
// twice and the other the odd rows, after v_permlane32_swap the lower and the upper half.
static __device__ __forceinline__ float row_max(float x) {
  auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  x = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
  auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
static __device__ __forceinline__ float row_sum(float x) {
  auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  x = __uint_as_float(a[0]) + __uint_as_float(a[1]);
  auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

// Asks for the 32-key step at kb (a multiple of 32, kb <= pos) of one request's pages, straight into
// operand registers. Every lane loads, whatever its keys, from an address inside the request's pages
// (that of a visible key where its own is not), by the same instructions on every path: the compiler
// can then count the loads under way and wait for a step's own only, while the next step's are in
// flight. Keys outside [lo, pos] are masked by the softmax; values outside count as zeros (`vok`).
template <int HD>
static __device__ __forceinline__ void load_tile(KVTile<HD>& T, int kb, int r, int g, int lo, int pos, int kvh,
                                                 const int32_t* __restrict__ table, const PageMath pm,
                                                 const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
                                                 int64_t kp, int64_t ks, int64_t kh, int64_t vp, int64_t vh,
                                                 int64_t vd) {
  constexpr int NC = HD / 32, NDB = HD / 16;
  int64_t koff[2], voff;      // (offsets, not pointers: the loads below are then plainly loads from the two caches)
  if (pm.whole_steps()) {
    // one page for the whole step: its base addresses are scalars, the lanes add fixed offsets
    // (the page is the request's since kb <= pos, and all its slots are memory of the pool)
    const int pg = pm.page(kb);
    const int64_t page = pm.pool_page(table, pg);
    const int slot = pm.slot(kb, pg);
    const int64_t kbase = page * kp + (int64_t)slot * ks + (int64_t)kvh * kh;
#pragma unroll
    for (int tau = 0; tau < 2; ++tau) koff[tau] = kbase + (int64_t)(8 * (r >> 2) + 4 * tau + (r & 3)) * ks + 8 * g;
    voff = page * vp + slot + (int64_t)kvh * vh + 8 * g + (int64_t)r * vd;
  } else {
#pragma unroll
    for (int tau = 0; tau < 2; ++tau) {
      const int key = min(max(kb + 8 * (r >> 2) + 4 * tau + (r & 3), lo), pos);     // a visible key, for the address
      const int pg = pm.page(key);
      koff[tau] = pm.pool_page(table, pg) * kp + (int64_t)pm.slot(key, pg) * ks + (int64_t)kvh * kh + 8 * g;
    }
    // page sizes are multiples of 8: the 8 keys share a page
    const int vkey = (kb + 8 * g <= pos && kb + 8 * g + 7 >= lo) ? kb + 8 * g : (pos & ~7);
    const int pg = pm.page(vkey);
    voff = pm.pool_page(table, pg) * vp + pm.slot(vkey, pg) + (int64_t)kvh * vh + (int64_t)r * vd;
  }
  T.vok = kb + 8 * g <= pos && kb + 8 * g + 7 >= lo;
#pragma unroll
  for (int tau = 0; tau < 2; ++tau)
#pragma unroll
    for (int c = 0; c < NC; ++c) T.k[tau][c] = *(const uint4*)(k_cache + koff[tau] + 32 * c);
#pragma unroll
  for (int db = 0; db < NDB; ++db) T.v[db] = *(const uint4*)(v_cache + voff + (int64_t)(16 * db) * vd);
}

#define TS_LAZY_MAX 8.0f     // a row's reference maximum is raised when a score exceeds it by more than this (log2 units)

// The scores of one 32-key step for the 16 rows that `qreg` holds: s[tau][j] = key kb + 8 g + 4 tau + j
// against row r (lane r = row r of the score tile), not yet scaled.
template <int HD>
static __device__ __forceinline__ void tile_scores(const uint4 (&k)[2][HD / 32], const uint4 (&qreg)[HD / 32], float4_t (&s)[2]) {
#pragma unroll
  for (int tau = 0; tau < 2; ++tau) {
    s[tau] = (float4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int c = 0; c < HD / 32; ++c) s[tau] = mfma32(k[tau][c], qreg[c], s[tau]);
  }
}

// The rest of the step: the online softmax of the scores `s` and the products with the values `v`
// (output row 4 g + j). `m` is the row's reference maximum in units of log2 (the same in the row's four
// lanes). `l`, a float: this lane's share of the row's sum; a float4_t: the sums of the output rows
// 4 g + j, made by the matrix cores from the rounded P that the output is made of. scale2 > 0.
// MASKED: rows mask the keys beyond their position and before their window (`vok`: whether any of
// this lane's eight keys of v is visible); without it every key of the step is visible to every row
// (the caller has checked).
template <int HD, bool MASKED, typename L>
static __device__ __forceinline__ void tile_softmax_values(float4_t (&s)[2], const uint4 (&v)[HD / 16], bool vok, int kb, int r,
                                                           int g, int lo, int pos, float scale2, float& m, L& l,
                                                           float4_t (&o)[HD / 16]) {
  constexpr int NDB = HD / 16;
  constexpr bool SUMS_BY_MFMA = std::is_same<L, float4_t>::value;
  // this lane: row r, keys kb + 8 g + 4 tau + j
  float mloc = -INFINITY;
#pragma unroll
  for (int tau = 0; tau < 2; ++tau)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (MASKED) {
        const int key = kb + 8 * g + 4 * tau + j;
        if (!(key <= pos && key >= lo)) s[tau][j] = -INFINITY;
      }
      mloc = fmaxf(mloc, s[tau][j]);
    }
  mloc *= scale2;
  const uint64_t hit = __builtin_amdgcn_ballot_w64(mloc > m + TS_LAZY_MAX);
  if (hit) {
    // some row's scores have outgrown its reference: those rows move it to their maximum so far
    const float mrow = row_max(mloc);
    const bool mine = ((hit >> r) & 0x0001000100010001ull) != 0;   // a lane of this lane's row
    const float m_new = mine ? fmaxf(m, mrow) : m;                 // finite where it changes
    const float alpha = m_new == m ? 1.0f : fast_exp2(m - m_new);
    if constexpr (!SUMS_BY_MFMA) l *= alpha;
    // output row 4 g + j belongs to score row 4 g + j, whose alpha lane 4 g + j holds
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float aj = __shfl(alpha, 4 * g + j, TS_WAVE);
      if constexpr (SUMS_BY_MFMA) l[j] *= aj;
#pragma unroll
      for (int db = 0; db < NDB; ++db) o[db][j] *= aj;
    }
    m = m_new;
  }
  const float neg_m = (MASKED && m == -INFINITY) ? 0.f : -m;   // nothing visible yet: every term below is 0
  float p[2][4];
#pragma unroll
  for (int tau = 0; tau < 2; ++tau)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      p[tau][j] = fast_exp2(fmaf(s[tau][j], scale2, neg_m));
      if constexpr (!SUMS_BY_MFMA) l += p[tau][j];
    }
  // this lane's eight keys kb + 8 g .. + 7, in the order the value registers hold them
  const uint4 pa = make_uint4(pack_bf16(p[0][0], p[0][1]), pack_bf16(p[0][2], p[0][3]), pack_bf16(p[1][0], p[1][1]),
                              pack_bf16(p[1][2], p[1][3]));
#pragma unroll
  for (int db = 0; db < NDB; ++db) o[db] = mfma32(pa, (MASKED && !vok) ? make_uint4(0, 0, 0, 0) : v[db], o[db]);
  if constexpr (SUMS_BY_MFMA) {
    const uint32_t ones = 0x3f803f80u;                 // 1.0 twice (a masked key's P is 0 already)
    l = mfma32(pa, make_uint4(ones, ones, ones, ones), l);
  }
}

// One 32-key step whole: the scores, then the softmax and the values.
template <int HD, bool MASKED, typename L>
static __device__ __forceinline__ void use_tile(const KVTile<HD>& T, int kb, int r, int g, int lo, int pos,
                                                const uint4 (&qreg)[HD / 32], float scale2, float& m, L& l,
                                                float4_t (&o)[HD / 16]) {
  float4_t s[2];
  tile_scores<HD>(T.k, qreg, s);
  tile_softmax_values<HD, MASKED, L>(s, T.v, T.vok, kb, r, g, lo, pos, scale2, m, l, o);
}

// The same, choosing the variant: `pmin` and `lomax` are the smallest position and the largest
// window start among the wave's rows (wave-uniform).
template <int HD>
static __device__ __forceinline__ void use_tile_auto(const KVTile<HD>& T, int kb, int r, int g, int lo, int pos,
                                                     int pmin, int lomax, const uint4 (&qreg)[HD / 32], float scale2,
                                                     float& m, float& l, float4_t (&o)[HD / 16]) {
  if (kb + 31 <= pmin && kb >= lomax) use_tile<HD, false, float>(T, kb, r, g, lo, pos, qreg, scale2, m, l, o);
  else use_tile<HD, true, float>(T, kb, r, g, lo, pos, qreg, scale2, m, l, o);
}

// out[t, h, :] from the chunks' partial results part_o [tokens, nh, num_splits, hd] and part_ml
// [tokens, nh, num_splits, 2] (reference maximum in units of log2, sum), over the chunks that hold
// keys visible from positions[t] (defined in attention_decode.hip).
int ts_launch_attention_combine(void* out, const float* part_o, const float* part_ml, const int32_t* positions,
                                int num_tokens, int nh, int hd, int num_splits, int chunk, int window,
                                hipStream_t stream);
