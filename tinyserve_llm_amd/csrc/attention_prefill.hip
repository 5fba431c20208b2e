// Paged attention on the matrix cores for steps that bring portions of prompts (and whatever
// decoded tokens ride along), bfloat16. The step's (token, query head) pairs of one key/value head
// are cut into tiles of 16 rows: 16 / G consecutive tokens of one request with the G heads of the
// group. A wave owns a tile and walks the request's keys from the first position any of its rows
// may see to the last, 32 keys at a time, with the next step's loads in flight; every row masks
// the keys beyond its own position (and before its window). Nothing is split and nothing is
// combined: a row's sums run over the keys in ascending order, whatever the batch.
//
// The host lists the tiles: tiles[2 i] = index of the tile's first token in the step,
// tiles[2 i + 1] = number of its tokens (at most 16 / G, all of one request).
#include "attention_mfma.h"

#define PRE_WAVES 4

template <int HD>
__global__ void __launch_bounds__(PRE_WAVES * TS_WAVE)
attn_prefill_mfma_kernel(bf16_t* __restrict__ out, const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_cache,
                         const bf16_t* __restrict__ v_cache, const int32_t* __restrict__ block_tables,
                         const int32_t* __restrict__ seq_of_token, const int32_t* __restrict__ positions,
                         const int32_t* __restrict__ tiles, int num_tiles, int nh, int G, int page_size,
                         int page_shift, int64_t kp, int64_t ks, int64_t kh, int64_t vp, int64_t vh, int64_t vd,
                         int max_blocks, float scale2, int window) {
  constexpr int NC = HD / 32, NDB = HD / 16;
  const int wave = threadIdx.x / TS_WAVE, lane = threadIdx.x & (TS_WAVE - 1);
  const int r = lane & 15, g = lane >> 4;
  // the longest tiles (the last tokens of long prompts) are listed last: hand them out first
  const int tile = num_tiles - 1 - (blockIdx.x * PRE_WAVES + wave);
  const int kvh = blockIdx.y;
  if (tile < 0) return;                      // whole wave; no workgroup barrier below
  const int t0 = tiles[2 * tile], ntok = tiles[2 * tile + 1];
  const int32_t* table = block_tables + (int64_t)seq_of_token[t0] * max_blocks;
  const PageMath pm{page_size, page_shift};

  // lane r carries row r of the score tile: token t0 + r / G, head r % G of the group
  const int tk = r / G, hh = r - tk * G;
  const bool row_ok = tk < ntok;
  const int pos = row_ok ? positions[t0 + tk] : -1;          // -1: no key is visible, the row stays empty
  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  // the tile's key range
  int pmax = pos, lmin = row_ok ? lo : 0x7fffffff;
#pragma unroll
  for (int off = 1; off < TS_WAVE; off <<= 1) {
    pmax = max(pmax, __shfl_xor(pmax, off, TS_WAVE));
    lmin = min(lmin, __shfl_xor(lmin, off, TS_WAVE));
  }

  uint4 qreg[NC];
#pragma unroll
  for (int c = 0; c < NC; ++c) qreg[c] = make_uint4(0, 0, 0, 0);
  if (row_ok) {
    const bf16_t* qrow = q + ((int64_t)(t0 + tk) * nh + (int64_t)kvh * G + hh) * HD + 8 * g;
#pragma unroll
    for (int c = 0; c < NC; ++c) qreg[c] = *(const uint4*)(qrow + 32 * c);
  }
  float m = -INFINITY, l = 0.f;
  float4_t o[NDB];
#pragma unroll
  for (int db = 0; db < NDB; ++db) o[db] = (float4_t){0.f, 0.f, 0.f, 0.f};

  int kb = lmin & ~31;
  const int kend = pmax + 1;
#define TS_LOAD(T, KB) load_tile<HD>(T, KB, r, g, lmin, pmax, kvh, table, pm, k_cache, v_cache, kp, ks, kh, vp, vh, vd)
#define TS_USE(T, KB) use_tile<HD>(T, KB, g, lo, pos, qreg, scale2, m, l, o)
  if (kb < kend) {
    KVTile<HD> A, B;
    TS_LOAD(A, kb);
    while (true) {
      const bool more_b = kb + 32 < kend;
      if (more_b) TS_LOAD(B, kb + 32);
      TS_USE(A, kb);
      if (!more_b) break;
      kb += 32;
      const bool more_a = kb + 32 < kend;
      if (more_a) TS_LOAD(A, kb + 32);
      TS_USE(B, kb);
      if (!more_a) break;
      kb += 32;
    }
  }
#undef TS_LOAD
#undef TS_USE
  // output row 4 g + j: token t0 + (4 g + j) / G, head (4 g + j) % G; its sum sits in lane 4 g + j
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int row = 4 * g + j;
    const float lj = __shfl(l, row, TS_WAVE);
    const int rtk = row / G, rhh = row - rtk * G;
    if (rtk < ntok && lj > 0.f) {
      const float inv = 1.0f / lj;
      bf16_t* orow = out + ((int64_t)(t0 + rtk) * nh + (int64_t)kvh * G + rhh) * HD;
#pragma unroll
      for (int db = 0; db < NDB; ++db) orow[16 * db + r] = f2bf(o[db][j] * inv);
    }
  }
}

// Keys: rows dense in head_dim, strides kp/ks/kh (page, slot, head). Values: transposed pages,
// slot stride 1, strides vp/vh/vd (page, head, dimension).
extern "C" int ts_paged_attention_prefill(void* out, const void* q, const void* k_cache, const void* v_cache,
                                          const int32_t* block_tables, const int32_t* seq_of_token,
                                          const int32_t* positions, const int32_t* tiles, int num_tiles, int nh,
                                          int nkv, int hd, int page_size, int64_t kp, int64_t ks, int64_t kh,
                                          int64_t vp, int64_t vh, int64_t vd, int max_blocks, float scale, int window,
                                          hipStream_t stream) {
  if (num_tiles <= 0) return TS_OK;
  if (nkv <= 0 || nh % nkv || page_size <= 0 || page_size % 8 || max_blocks <= 0) return TS_BAD_SHAPE;
  const int G = nh / nkv;
  if (G > 16 || nkv > 65535) return TS_BAD_SHAPE;
  if ((kp % 8) || (ks % 8) || (kh % 8) || (vp % 8) || (vh % 8) || (vd % 8)) return TS_BAD_SHAPE;
  if ((((uintptr_t)q) | ((uintptr_t)k_cache) | ((uintptr_t)v_cache)) & 15) return TS_BAD_SHAPE;
  int page_shift = -1;
  if ((page_size & (page_size - 1)) == 0) {
    page_shift = 0;
    while ((1 << page_shift) < page_size) ++page_shift;
  }
  dim3 grid((num_tiles + PRE_WAVES - 1) / PRE_WAVES, nkv);
#define TS_PRE(HH)                                                                                              \
  attn_prefill_mfma_kernel<HH><<<grid, PRE_WAVES * TS_WAVE, 0, stream>>>(                                       \
      (bf16_t*)out, (const bf16_t*)q, (const bf16_t*)k_cache, (const bf16_t*)v_cache, block_tables,             \
      seq_of_token, positions, tiles, num_tiles, nh, G, page_size, page_shift, kp, ks, kh, vp, vh, vd,          \
      max_blocks, scale * 1.44269504088896340736f, window)
  switch (hd) {
    case 32: TS_PRE(32); break;
    case 64: TS_PRE(64); break;
    case 96: TS_PRE(96); break;
    case 128: TS_PRE(128); break;
    default: return TS_BAD_SHAPE;
  }
#undef TS_PRE
  return ts_check_launch();
}
