// Paged attention on the matrix cores for steps that bring portions of prompts, bfloat16. The
// step's (token, query head) pairs of one key/value head are cut into tiles of 16 rows: 16 / G
// consecutive tokens of one request with the G heads of the group. A workgroup of four waves takes
// up to 4 RT such tiles of consecutive tokens (RT per wave) and walks the request's keys from the
// first position any of its rows may see to the last, 32 keys at a time. Each step's keys and
// values are fetched from the pages once per workgroup: every wave loads a quarter of the operand
// registers, leaves them in LDS in the order the lanes use them, and all four waves read the whole
// step back from there, two steps ahead of the loads in flight. A row masks the keys beyond its own
// position (and before its window); steps that lie wholly inside every row's range skip the masks.
// Normally nothing is split and nothing is combined: a row's sums run over the keys in ascending
// order, whatever the batch. A step of few tokens over a long context has too few tiles to fill the
// chip: then the keys are cut into chunks (num_splits > 1), a workgroup walks one chunk for its
// tile and leaves the rows' partial results (part_o, part_ml, as the decode kernel does), and the
// decode kernel's combining kernel sums the chunks in ascending order.
//
// The host lists the tiles: tiles[2 i] = index of the tile's first token in the step,
// tiles[2 i + 1] = number of its tokens (at most 4 RT (16 / G), all of one request), in ascending
// order of the number of keys a tile walks. There is one workgroup per (key/value head, tile), and
// the long tiles start first. The chip hands consecutive workgroups to its eight dies in turn, and
// each die has a cache of its own, so the kernel maps workgroups to work such that those which walk
// one head's keys sit on as few dies as possible: with eight heads (or a multiple) each die works
// on heads of its own and reads their keys from memory once.
#include <type_traits>
#include "attention_mfma.h"

#define PRE_MAX_WAVES 8

// Where the steps of a walk lie (whole steps only: pages of a multiple of 32 keys): a ring of PRE_PLACES steps, refilled
// by halves, that holds for step i what its page and slot add to a lane's fixed place in the keys' pool and in the
// values'. The walk reads a step's entry instead of looking its page up and multiplying.
#define PRE_PLACES 256
template <int HD>
struct PrefillLds {
  uint4 stage[2][HD / 8][TS_WAVE];   // two steps of operand registers, [register][lane]
  int range[4][PRE_MAX_WAVES];
  int64_t place[2][PRE_PLACES];      // [keys | values][step mod PRE_PLACES], in elements
};

// PRE_WAVES: 4, or 8 (heads of 64 or 128 dimensions): the same tokens a workgroup in tiles half as
// large a wave, so that a step's vector work is spread over twice the waves; the longest tiles of a
// short prompt, which run alone at the end, then take a shorter step (2,048 tokens at head size 64:
// 48.9 µs against 51.3; over long contexts the doubled reads of LDS cost more than that gains).
// WHOLE: a page holds a multiple of 32 keys, so that every step lies in one page.
template <int HD, int RT, int PRE_WAVES, bool WHOLE>
static __device__ __forceinline__ void
prefill_tile(PrefillLds<HD>& lds, int tile, int kvh, bf16_t* __restrict__ out, const bf16_t* __restrict__ q,
             const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
             const int32_t* __restrict__ block_tables, const int32_t* __restrict__ seq_of_token,
             const int32_t* __restrict__ positions, const int32_t* __restrict__ tiles, int nh, int G, int page_size,
             int page_shift, int page_run, int64_t kp, int64_t ks, int64_t kh, int64_t vp, int64_t vh, int64_t vd, int max_blocks,
             float scale2, int window, float* __restrict__ part_o, float* __restrict__ part_ml, int num_splits,
             int chunk, int split) {
  constexpr int NC = HD / 32, NDB = HD / 16;   // operand registers of a 32-key step: 2 NC of K, NDB of V
  auto& stage = lds.stage;
  auto& wg_range = lds.range;
  const int wave = wave_index(), lane = threadIdx.x & (TS_WAVE - 1);
  const int r = lane & 15, g = lane >> 4;
  const int t0 = tiles[2 * tile], ntok = tiles[2 * tile + 1];
  const int32_t* table = block_tables + (int64_t)seq_of_token[t0] * max_blocks;
  const PageMath pm{page_size, page_shift, page_run};
  const int tpt = 16 / G;                                   // tokens per row tile

  // lane r carries row r of each of its wave's score tiles: token tk[j], head r % G of the group
  const int hh = r % G;
  int pos[RT], lo[RT], tk[RT];
  int pmax = -1, lmin = 0x7fffffff;
#pragma unroll
  for (int j = 0; j < RT; ++j) {
    tk[j] = (wave * RT + j) * tpt + r / G;
    const bool ok = r / G < tpt && tk[j] < ntok;
    pos[j] = ok ? positions[t0 + tk[j]] : -1;               // -1: no key is visible, the row stays empty
    lo[j] = (window > 0 && pos[j] - window + 1 > 0) ? pos[j] - window + 1 : 0;
    if (!ok) tk[j] = -1;
    pmax = max(pmax, pos[j]);
    lmin = min(lmin, ok ? lo[j] : 0x7fffffff);
  }
  // per row tile: the smallest position and largest window start of its rows (wave-uniform)
  // (tile_vpmin: the smallest position among the rows that exist; rows that do not are never stored)
  int tile_lomax[RT], tile_pmax[RT], tile_lomin[RT], tile_vpmin[RT];
#pragma unroll
  for (int j = 0; j < RT; ++j) {
    tile_lomax[j] = lo[j]; tile_pmax[j] = pos[j];
    tile_lomin[j] = tk[j] >= 0 ? lo[j] : 0x7fffffff;
    tile_vpmin[j] = tk[j] >= 0 ? pos[j] : 0x7fffffff;
  }
#pragma unroll
  for (int off = 1; off < TS_WAVE; off <<= 1) {
    pmax = max(pmax, __shfl_xor(pmax, off, TS_WAVE));
    lmin = min(lmin, __shfl_xor(lmin, off, TS_WAVE));
#pragma unroll
    for (int j = 0; j < RT; ++j) {
      tile_vpmin[j] = min(tile_vpmin[j], __shfl_xor(tile_vpmin[j], off, TS_WAVE));
      tile_pmax[j] = max(tile_pmax[j], __shfl_xor(tile_pmax[j], off, TS_WAVE));
      tile_lomax[j] = max(tile_lomax[j], __shfl_xor(tile_lomax[j], off, TS_WAVE));
      tile_lomin[j] = min(tile_lomin[j], __shfl_xor(tile_lomin[j], off, TS_WAVE));
    }
  }
  // the workgroup's key range [wlo, whi], and the range every one of its rows sees whole: [wfull_lo, wfull_hi]
  if (lane == 0) {
    int pmin = 0x7fffffff, lomax = 0;
#pragma unroll
    for (int j = 0; j < RT; ++j) { pmin = min(pmin, tile_vpmin[j]); lomax = max(lomax, tile_lomax[j]); }
    wg_range[0][wave] = lmin; wg_range[1][wave] = pmax; wg_range[2][wave] = pmin; wg_range[3][wave] = lomax;
  }
  __syncthreads();
  int wlo = wg_range[0][0], whi = wg_range[1][0], wfull_hi = wg_range[2][0], wfull_lo = wg_range[3][0];
#pragma unroll
  for (int w = 1; w < PRE_WAVES; ++w) {
    wlo = min(wlo, wg_range[0][w]); whi = max(whi, wg_range[1][w]);
    wfull_hi = min(wfull_hi, wg_range[2][w]); wfull_lo = max(wfull_lo, wg_range[3][w]);
  }
  if (num_splits > 1) {
    // this workgroup walks one chunk of the keys only (chunks are multiples of 32 keys, so no step
    // straddles two); what the rows see of it is combined with the other chunks afterwards
    // (the last chunk has no upper end, so every position is in some chunk whatever the caller chose)
    wlo = max(wlo, split * chunk);
    wfull_lo = max(wfull_lo, split * chunk);
    if (split + 1 < num_splits) {
      whi = min(whi, split * chunk + chunk - 1);
      if (wfull_hi != 0x7fffffff) wfull_hi = min(wfull_hi, split * chunk + chunk - 1);
    }
  }
  // every lane holds the same values: say so, and loop control and page lookups become scalar
  wlo = __builtin_amdgcn_readfirstlane(wlo);
  whi = __builtin_amdgcn_readfirstlane(whi);
  wfull_lo = __builtin_amdgcn_readfirstlane(wfull_lo);
  wfull_hi = __builtin_amdgcn_readfirstlane(wfull_hi);
#pragma unroll
  for (int j = 0; j < RT; ++j) {
    tile_pmax[j] = __builtin_amdgcn_readfirstlane(tile_pmax[j]);
    tile_lomax[j] = __builtin_amdgcn_readfirstlane(tile_lomax[j]);
    tile_lomin[j] = __builtin_amdgcn_readfirstlane(tile_lomin[j]);
  }

  uint4 qreg[RT][NC];
  float m[RT];
  float4_t l[RT];                 // the sums of the output rows 4 g + i, made by the matrix cores
  float4_t o[RT][NDB];
#pragma unroll
  for (int j = 0; j < RT; ++j) {
    m[j] = -INFINITY; l[j] = (float4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int c = 0; c < NC; ++c) qreg[j][c] = make_uint4(0, 0, 0, 0);
    if (tk[j] >= 0) {
      const bf16_t* qrow = q + ((int64_t)(t0 + tk[j]) * nh + (int64_t)kvh * G + hh) * HD + 8 * g;
#pragma unroll
      for (int c = 0; c < NC; ++c) qreg[j][c] = *(const uint4*)(qrow + 32 * c);
    }
#pragma unroll
    for (int db = 0; db < NDB; ++db) o[j][db] = (float4_t){0.f, 0.f, 0.f, 0.f};
  }

  // This wave's share of a step's operand registers, PER of the 4 NC: register q < 2 NC is piece q % NC
  // of the 16-key tile q / NC of K, register 2 NC + db is dimension block db of V.
  constexpr int PER = 4 * NC / PRE_WAVES;
  static_assert(PER >= 1 && PER * PRE_WAVES == 4 * NC, "the waves share a step's operand registers evenly");
  uint4 fetched[PER];
  const bool loads_k = wave * PER < 2 * NC;           // (a wave's registers are all of K or all of V)
  const int tau = (wave * PER) / NC, c0 = (wave * PER) % NC, db0 = wave * PER - 2 * NC;
  const int kbeg = wlo & ~31;
  const int kend = whi + 1;
  // Whole steps: a lane's pieces lie at the same places of every page, so what the lane adds to a step's
  // place is worked out once, and the steps' places come from the ring in LDS.
  const int koff = 8 * (r >> 2) + 4 * tau + (r & 3);
  const bf16_t* const lane_base = loads_k ? k_cache + ((int64_t)kvh * kh + (int64_t)koff * ks + 8 * g + 32 * c0)
                                          : v_cache + ((int64_t)kvh * vh + 8 * g + (int64_t)(db0 * 16 + r) * vd);
  const int64_t piece = loads_k ? 32 : 16 * vd;
  const int lane_first = loads_k ? koff : 8 * g, lane_last = loads_k ? koff : 8 * g + 7;   // the keys a piece holds
  const int64_t* const places = lds.place[loads_k ? 0 : 1];
  // the places of the walk's steps first .. first + count - 1 go into the ring (steps beyond the last one: the
  // last one's, whose page is the request's as well)
  auto fill_places = [&](int first, int count) {
    for (int i = threadIdx.x; i < count; i += PRE_WAVES * TS_WAVE) {
      const int kb = min(kbeg + 32 * (first + i), whi & ~31);
      const int pg = pm.page(kb);
      const int64_t page = pm.pool_page(table, pg);
      const int slot = pm.slot(kb, pg);
      lds.place[0][(first + i) & (PRE_PLACES - 1)] = page * kp + (int64_t)slot * ks;
      lds.place[1][(first + i) & (PRE_PLACES - 1)] = page * vp + slot;
    }
  };
  auto place_of = [&](int kb) { return places[((kb - kbeg) >> 5) & (PRE_PLACES - 1)]; };
  // asks for the step at kb, which lies at `place` (whole steps; kb may lie beyond the walk: nothing is loaded then)
  auto fetch_at = [&](int kb, int64_t place) {
    const bf16_t* src = lane_base + place;
    if (kb >= wlo && kb + 31 <= whi) {              // nearly every step: nothing to leave out, nothing to clear
#pragma unroll
      for (int c = 0; c < PER; ++c) fetched[c] = *(const uint4*)(src + c * piece);
    } else {
      const bool ok = kb + lane_first <= whi && kb + lane_last >= wlo;
#pragma unroll
      for (int c = 0; c < PER; ++c) fetched[c] = ok ? *(const uint4*)(src + c * piece) : make_uint4(0, 0, 0, 0);
    }
  };
  auto fetch = [&](int kb) {
    if constexpr (WHOLE) {
      fetch_at(kb, place_of(kb));
      return;
    }
#pragma unroll
    for (int c = 0; c < PER; ++c) fetched[c] = make_uint4(0, 0, 0, 0);
    if (loads_k) {
      const int key = kb + 8 * (r >> 2) + 4 * tau + (r & 3);
      if (key <= whi && key >= wlo) {
        const int pg = pm.page(key);
        const bf16_t* kr = k_cache + pm.pool_page(table, pg) * kp + (int64_t)pm.slot(key, pg) * ks + (int64_t)kvh * kh + 8 * g + 32 * c0;
#pragma unroll
        for (int c = 0; c < PER; ++c) fetched[c] = *(const uint4*)(kr + 32 * c);
      }
    } else {
      const int vkey = kb + 8 * g;
      if (vkey <= whi && vkey + 7 >= wlo) {
        const int pg = pm.page(vkey);
        const bf16_t* vr = v_cache + pm.pool_page(table, pg) * vp + pm.slot(vkey, pg) + (int64_t)kvh * vh +
                           (int64_t)(db0 * 16 + r) * vd;
#pragma unroll
        for (int c = 0; c < PER; ++c) fetched[c] = *(const uint4*)(vr + (int64_t)(16 * c) * vd);
      }
    }
  };
  auto put = [&](int buf) {
#pragma unroll
    for (int c = 0; c < PER; ++c) stage[buf][wave * PER + c][lane] = fetched[c];
  };

  // The walk has three stretches: steps that some row sees in part (before the last window start),
  // steps that every row of the workgroup sees whole, and the steps around the rows' own positions.
  // The middle one, nearly all of a long walk, runs without masks and without the test whether a
  // tile has anything to do; each stretch is a loop of its own so that the accumulators stay in
  // their registers from one step to the next.
  const int full_lo = min(max((wfull_lo + 31) & ~31, kbeg), kend);
  const int full_hi = min(max(wfull_hi == 0x7fffffff ? 0 : ((wfull_hi + 1) & ~31), full_lo), kend);
  int buf = 0;
  int64_t place_next = 0;                    // whole steps: the place of the step two ahead, read a step early
  auto walk = [&](int from, int to, auto masked) {
    for (int kb = from; kb < to; kb += 32, buf ^= 1) {
      int64_t place_now = 0;
      if constexpr (WHOLE) {
        // every half turn of the ring the half that the walk has left behind takes the places of the steps
        // a turn ahead (first read half a turn from now, many barriers later)
        const int step = (kb - kbeg) >> 5;
        if ((step & (PRE_PLACES / 2 - 1)) == 0 && step) fill_places(step + PRE_PLACES / 2, PRE_PLACES / 2);
        place_now = place_next;
        place_next = place_of(kb + 96);
      }
      KVTile<HD> T;
#pragma unroll
      for (int c = 0; c < NC; ++c) { T.k[0][c] = stage[buf][c][lane]; T.k[1][c] = stage[buf][NC + c][lane]; }
#pragma unroll
      for (int db = 0; db < NDB; ++db) T.v[db] = stage[buf][2 * NC + db][lane];
      T.vok = true;                          // (what lies outside the range went into LDS as zeros)
      if constexpr (WHOLE) {
        // (no tests for the walk's end: past it zeros are put where nobody reads, and nothing is asked for)
        put(buf ^ 1);                        // the other buffer was last read before the previous barrier
        fetch_at(kb + 64, place_now);
      } else {
        if (kb + 32 < kend) put(buf ^ 1);
        if (kb + 64 < kend) fetch(kb + 64);
      }
#pragma unroll
      for (int j = 0; j < RT; ++j) {
        if constexpr (decltype(masked)::value) {
          // a step wholly beyond the tile's last position, or wholly before all its windows, has nothing for it
          if (kb <= tile_pmax[j] && kb + 31 >= tile_lomin[j])
            use_tile<HD, true, float4_t>(T, kb, r, g, lo[j], pos[j], qreg[j], scale2, m[j], l[j], o[j]);
        } else {
          use_tile<HD, false, float4_t>(T, kb, r, g, lo[j], pos[j], qreg[j], scale2, m[j], l[j], o[j]);
        }
      }
      __syncthreads();
    }
  };
  if (kbeg < kend) {                         // uniform over the workgroup
    if constexpr (WHOLE) {
      fill_places(0, PRE_PLACES);
      __syncthreads();
      place_next = place_of(kbeg + 64);
    }
    fetch(kbeg);
    put(0);
    if (kbeg + 32 < kend) fetch(kbeg + 32);
    __syncthreads();
    walk(kbeg, full_lo, std::true_type{});
    walk(full_lo, full_hi, std::false_type{});
    walk(full_hi, kend, std::true_type{});
  }
  // output row 4 g + i of row tile j: its token and head, and its sum
#pragma unroll
  for (int j = 0; j < RT; ++j)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int row = 4 * g + i;
      const float lj = l[j][i];
      const int rtk = (wave * RT + j) * tpt + row / G, rhh = row % G;
      if (num_splits > 1) {
        // the chunk's share of the row, not normalised: sums, and the reference maximum they are relative to
        const float mj = __shfl(m[j], row, TS_WAVE);
        if (row / G < tpt && rtk < ntok) {
          const int64_t at = (((int64_t)(t0 + rtk) * nh + (int64_t)kvh * G + rhh) * num_splits + split);
#pragma unroll
          for (int db = 0; db < NDB; ++db) part_o[at * HD + 16 * db + r] = o[j][db][i];
          if (r == 0) { part_ml[at * 2] = mj; part_ml[at * 2 + 1] = lj; }
        }
        continue;
      }
      if (row / G < tpt && rtk < ntok && lj > 0.f) {
        const float inv = 1.0f / lj;
        bf16_t* orow = out + ((int64_t)(t0 + rtk) * nh + (int64_t)kvh * G + rhh) * HD;
#pragma unroll
        for (int db = 0; db < NDB; ++db) orow[16 * db + r] = f2bf(o[j][db][i] * inv);
      }
    }
}

template <int HD, int RT, int PRE_WAVES, bool WHOLE>
__global__ void __launch_bounds__(PRE_WAVES * TS_WAVE)
attn_prefill_mfma_kernel(bf16_t* __restrict__ out, const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_cache,
                         const bf16_t* __restrict__ v_cache, const int32_t* __restrict__ block_tables,
                         const int32_t* __restrict__ seq_of_token, const int32_t* __restrict__ positions,
                         const int32_t* __restrict__ tiles, int num_tiles, int nh, int G, int dies_per_group,
                         int heads_per_group, int page_size, int page_shift, int page_run, int64_t kp, int64_t ks, int64_t kh,
                         int64_t vp, int64_t vh, int64_t vd, int max_blocks, float scale2, int window,
                         float* __restrict__ part_o, float* __restrict__ part_ml, int num_splits, int chunk) {
  __shared__ PrefillLds<HD> lds;
  // die = workgroup index mod 8. The dies form `groups` groups of `dies_per_group`, the heads as
  // many groups of `heads_per_group`; a group's (tile, head) pairs go round its dies, long tiles first.
  const int die = blockIdx.x % 8, turn = blockIdx.x / 8;
  const int item = turn * dies_per_group + die % dies_per_group;
  if (item >= num_tiles * heads_per_group) return;
  const int tile = num_tiles - 1 - item / heads_per_group;
  const int kvh = (die / dies_per_group) * heads_per_group + item % heads_per_group;
  prefill_tile<HD, RT, PRE_WAVES, WHOLE>(lds, tile, kvh, out, q, k_cache, v_cache, block_tables, seq_of_token, positions, tiles, nh,
                       G, page_size, page_shift, page_run, kp, ks, kh, vp, vh, vd, max_blocks, scale2, window, part_o, part_ml,
                       num_splits, chunk, blockIdx.y);
}

// Keys: rows dense in head_dim, strides kp/ks/kh (page, slot, head). Values: transposed pages,
// slot stride 1, strides vp/vh/vd (page, head, dimension). tile_tokens: the most tokens a listed
// tile holds, waves x RT (16 / G) for RT of 1, 2 or 4 row tiles a wave and 4 waves, or 8 waves with one or two
// (heads of 64 or 128 dimensions). num_splits > 1: chunk (a multiple of 32; the last chunk
// takes every key from its start on) and the float workspaces part_o [num_tokens, nh, num_splits, hd] and
// part_ml [num_tokens, nh, num_splits, 2]; every token from first_token on must then be in a tile (the ones
// before it keep what `out` held). An entry of block_tables names 2^page_run consecutive pages of page_size keys.
extern "C" int ts_paged_attention_prefill(void* out, const void* q, const void* k_cache, const void* v_cache,
                                          const int32_t* block_tables, const int32_t* seq_of_token,
                                          const int32_t* positions, const int32_t* tiles, int num_tiles,
                                          int tile_tokens, int waves, int nh, int nkv, int hd, int page_size, int64_t kp,
                                          int64_t ks, int64_t kh, int64_t vp, int64_t vh, int64_t vd, int max_blocks,
                                          float scale, int window, int first_token, int num_tokens, int num_splits,
                                          int chunk, float* part_o, float* part_ml, int page_run, hipStream_t stream) {
  if (num_tiles <= 0) return TS_OK;
  if (num_splits < 1 || num_splits > 65535) return TS_BAD_SHAPE;
  if (num_splits > 1 && (chunk <= 0 || chunk % 32 || !part_o || !part_ml || first_token < 0 || num_tokens <= first_token))
    return TS_BAD_SHAPE;
  if (nkv <= 0 || nh % nkv || page_size <= 0 || page_size % 8 || max_blocks <= 0 || page_run < 0 || page_run > 16) return TS_BAD_SHAPE;
  const int G = nh / nkv;
  if (G > 16) return TS_BAD_SHAPE;
  if (waves != 4 && !(waves == 8 && (hd == 64 || hd == 128))) return TS_BAD_SHAPE;
  const int per_wave = waves * (16 / G);
  if (tile_tokens != per_wave && tile_tokens != 2 * per_wave && !(tile_tokens == 4 * per_wave && waves == 4)) return TS_BAD_SHAPE;
  const int rt = tile_tokens / per_wave;
  if ((kp % 8) || (ks % 8) || (kh % 8) || (vp % 8) || (vh % 8) || (vd % 8)) return TS_BAD_SHAPE;
  if ((((uintptr_t)q) | ((uintptr_t)k_cache) | ((uintptr_t)v_cache)) & 15) return TS_BAD_SHAPE;
  int page_shift = -1;
  if ((page_size & (page_size - 1)) == 0) {
    page_shift = 0;
    while ((1 << page_shift) < page_size) ++page_shift;
  }
  int groups = 8;                                   // gcd(nkv, 8)
  while (nkv % groups) groups /= 2;
  const int dies_per_group = 8 / groups, heads_per_group = nkv / groups;
  const int64_t turns = ((int64_t)num_tiles * heads_per_group + dies_per_group - 1) / dies_per_group;
  if (turns * 8 > 0x7fffffff) return TS_BAD_SHAPE;
  dim3 grid((unsigned)(8 * turns), num_splits);
#define TS_PRE_W(HH, RR, WW)                                                                                    \
  if (page_size % 32 == 0) TS_PRE_P(HH, RR, WW, true); else TS_PRE_P(HH, RR, WW, false)
#define TS_PRE_P(HH, RR, WW, PP)                                                                                \
  attn_prefill_mfma_kernel<HH, RR, WW, PP><<<grid, WW * TS_WAVE, 0, stream>>>(                                  \
      (bf16_t*)out, (const bf16_t*)q, (const bf16_t*)k_cache, (const bf16_t*)v_cache, block_tables,             \
      seq_of_token, positions, tiles, num_tiles, nh, G, dies_per_group, heads_per_group, page_size, page_shift, page_run, kp,  \
      ks, kh, vp, vh, vd, max_blocks, scale * 1.44269504088896340736f, window, part_o, part_ml, num_splits, chunk)
#define TS_PRE_RT(HH)                                                                                           \
  if (rt == 1) TS_PRE_W(HH, 1, 4); else if (rt == 2) TS_PRE_W(HH, 2, 4); else TS_PRE_W(HH, 4, 4)
#define TS_PRE_RT8(HH)                                                                                          \
  if (rt == 1) TS_PRE_W(HH, 1, 8); else TS_PRE_W(HH, 2, 8)
  if (waves == 8) {
    switch (hd) {
      case 64: TS_PRE_RT8(64); break;
      case 128: TS_PRE_RT8(128); break;
      default: return TS_BAD_SHAPE;       // (96: twelve registers a step do not go round eight waves)
    }
  } else {
    switch (hd) {
      case 32: TS_PRE_RT(32); break;
      case 64: TS_PRE_RT(64); break;
      case 96: TS_PRE_RT(96); break;
      case 128: TS_PRE_RT(128); break;
      default: return TS_BAD_SHAPE;
    }
  }
#undef TS_PRE_RT8
#undef TS_PRE_RT
#undef TS_PRE_W
#undef TS_PRE_P
  const int rc = ts_check_launch();
  if (rc || num_splits == 1) return rc;
  const int64_t skip = (int64_t)first_token * nh;     // rows of the tokens before the first listed one
  return ts_launch_attention_combine((bf16_t*)out + skip * hd, part_o + skip * num_splits * hd,
                                     part_ml + skip * num_splits * 2, positions + first_token,
                                     num_tokens - first_token, nh, hd, num_splits, chunk, window, stream);
}
