// y[M, N] = e(f(x)[M, K] · W[N, K]^T) for bfloat16 with few rows of x (decoding: M up to 32), where
// time goes to reading W once from HBM. A workgroup owns 16 to 64 rows of W over the whole of K;
// each of its waves takes a slice of K of 256 or 512 and issues every load of its slice of W before
// it uses the first, so that a cold matrix streams at memory speed; the rows go straight from the
// 16-byte loads into MFMA operands (v_mfma_f32_16x16x32_bf16: W rows are the A matrix, x^T the B
// matrix), and the waves' partial tiles are summed in LDS in a fixed order. Accumulation is 32-bit;
// the result is rounded once.
//
// x is read through the caches (it is tiny and shared by every workgroup). What precedes and
// follows the product in a layer can ride along, so that no separate kernel has to run:
//   MODE_NORM  residual + RMSNorm on the way in (up to 16 rows): the operand is T((x + res) * nw) and
//              the row's scale rsqrt(mean((x + res)^2) + eps), 32-bit, multiplies the finished sums
//              (the separate norm kernel rounds (x + res) * scale first and the product with nw
//              again: the same value up to the rounding of the storage type); workgroup 0 also writes
//              T(x + res) as the new residual
//   EPI_GLU    W = [gate rows | up rows]; a workgroup takes matching rows of both and writes
//              silu(gate) * up, y being [M, N / 2]
//   EPI_ROPE   W = [q heads | k heads | v heads] of head_dim columns each; a 16-row tile holds 8
//              columns of the first half of a head (matrix rows r < 8) and the 8 that rotate with
//              them (rows r >= 8: head_dim / 2 further on), so a workgroup of one tile has both
//              halves of a rotation and a matrix of 3,072 columns gives 192 workgroups; it rounds the
//              products as y would hold them, rotates q and k by the token's position, and writes q
//              to its own tensor and k and v into their cache slots: y itself is never stored
#include "skinny_ops.h"

struct SkinnyArgs {
  const bf16_t* x;      // [M, K] (MODE_GATE: [M, 2K])
  const bf16_t* res;    // MODE_NORM: residual [M, K] or null
  const bf16_t* nw;     // MODE_NORM: norm weight [K]
  bf16_t* res_out;      // MODE_NORM with res: new residual [M, K]
  const bf16_t* w;      // [N, K]
  void* y;              // [M, N]
  int M, N, K, packed;
  int64_t ldx, ldw, ldy;
  float eps;
  // EPI_ROPE: N = (nh + 2 nkv) * hd; cos_sin [max_pos, hd] 32-bit, [cos | sin] halves; slot -1 stores nothing.
  // key element: page * kp + offset * ks + head * kh + d; value element: page * vp + offset * vs + head * vh + d * vd
  const float* cos_sin;
  const int32_t* positions;
  const int32_t* slots;
  bf16_t* q_out;        // [M, nh * hd]
  bf16_t* k_cache;      // null: this layer owns no cache, only q is produced
  bf16_t* v_cache;
  int nh, nkv, hd, rotate, page_size;
  int64_t kp, ks, kh, vp, vs, vh, vd;
};

// RT: 16-row tiles of W per workgroup; CB: 16-row blocks of x; STEPS: 32-wide k steps per wave;
// MAXT: most threads a workgroup of this instance is launched with (it bounds the registers)
template <int RT, int CB, int STEPS, int MODE, int EPI, int MAXT, typename OUT>
__global__ void __launch_bounds__(MAXT)
gemm_skinny_kernel(const SkinnyArgs a) {
  constexpr bool GLU = EPI == EPI_GLU, ROPE = EPI == EPI_ROPE, PAIRS = EPI != EPI_NONE;
  static_assert(MODE == MODE_PLAIN || CB == 1, "the fused norm serves one block of rows");
  static_assert(!GLU || RT % 2 == 0, "gate and up tiles come in pairs");
  // steps of x fetched at a time: fewer where more blocks of x, more row tiles of W or a larger workgroup leave fewer registers
  constexpr int SK_XBATCH = CB >= 4 ? 4 : (CB == 2 && (MAXT > 512 || RT >= 4)) ? 4 : 8;
  extern __shared__ __align__(16) float smem[];
  const int nwaves = blockDim.x / TS_WAVE;
  float* part = smem;                                   // [nwaves][RT][CB][256]
  float* ssq = smem + (size_t)nwaves * RT * CB * 256;   // [nwaves][16]
  const int wave = threadIdx.x / TS_WAVE, lane = threadIdx.x & (TS_WAVE - 1);
  const int r = lane & 15, g = lane >> 4;
  // GLU: tiles 0 .. RT/2-1 are gate rows n0 + 16 t, tiles RT/2 .. RT-1 the up rows N/2 below them.
  // ROPE: tile j of the matrix holds rows 8 (j % (hd / 16)) .. + 7 of head j / (hd / 16) in its rows
  // r < 8 and the rows hd / 2 below them in its rows r >= 8.
  constexpr int OT = GLU ? RT / 2 : RT;                 // 16-column tiles of the output per workgroup
  const int n0 = blockIdx.x * 16 * OT;
  const int half = a.N / 2;
  const int kbeg = wave * STEPS * SK_KSTEP + 8 * g;     // this lane's first k

  const bf16_t* xrow[CB];
  bool xok[CB];
#pragma unroll
  for (int b = 0; b < CB; ++b) {
    const int m = b * 16 + r;
    xok[b] = m < a.M;
    xrow[b] = a.x + (int64_t)(xok[b] ? m : 0) * a.ldx + kbeg;
  }
  // ---- MODE_NORM: this wave's slice of x, the residual and the norm weight are asked for before W.
  // Loads come back in the order they were issued, and these are short and hit the cache: the norm
  // is computed while W is still streaming in.
  // (Up to 8 waves a workgroup: 16 waves have no registers for it, and their callers run the norm
  // as a kernel of its own.)
  static_assert(MODE != MODE_NORM || MAXT <= 512, "the fused norm needs the registers of a workgroup of 8 waves");
  uint4 xraw[MODE == MODE_NORM ? STEPS : 1], rraw[MODE == MODE_NORM ? STEPS : 1], nraw[MODE == MODE_NORM ? STEPS : 1];
  if (MODE == MODE_NORM) {
    // unconditional loads from addresses that always exist (rows past M read row 0, a missing
    // residual reads x again): what does not count is dropped after it has arrived
    const bf16_t* rrow = a.res ? a.res + (int64_t)(xok[0] ? r : 0) * a.K + kbeg : xrow[0];
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
      xraw[s] = *(const uint4*)(xrow[0] + s * SK_KSTEP);
      rraw[s] = *(const uint4*)(rrow + s * SK_KSTEP);
      nraw[s] = *(const uint4*)(a.nw + kbeg + s * SK_KSTEP);
    }
    __builtin_amdgcn_sched_barrier(0);                  // the compiler keeps these loads ahead of W's
  }

  // ---- every load of this wave's slice of W, at once
  uint4 wreg[RT][STEPS];
#pragma unroll
  for (int t = 0; t < RT; ++t) {
    int n = GLU ? (t < OT ? n0 + t * 16 + r : half + n0 + (t - OT) * 16 + r) : n0 + t * 16 + r;
    int limit = GLU ? (t < OT ? half : a.N) : a.N;
    if (ROPE) {
      const int per_head = a.hd / 16, j = blockIdx.x * RT + t;
      n = (j / per_head) * a.hd + 8 * (j % per_head) + (r & 7) + (r >> 3) * (a.hd / 2);
      limit = a.N;
    }
    if (a.packed) {
      // W in 1 KB blocks [16-row tile][32-wide k step][lane][8 k]: one load of a wave is one
      // contiguous kilobyte and a wave's slice of a tile a contiguous run of them (rows past N are
      // zeros in the last tile; tiles past the last are computed from it and not stored)
      int tile_n = ROPE ? blockIdx.x * RT + t : (n - r) / 16;   // (ROPE: the packed copy holds the tiles as described above)
      const int last = (a.N - 1) / 16;
      if (tile_n > last) tile_n = last;
      const bf16_t* wblk = a.w + (((int64_t)tile_n * (a.K / SK_KSTEP) + (int64_t)wave * STEPS) * 64 + lane) * 8;
#pragma unroll
      for (int s = 0; s < STEPS; ++s) wreg[t][s] = *(const uint4*)(wblk + (int64_t)s * 512);
    } else {
      if (n >= limit) n = limit - 1;                    // rows past the end are computed and not stored
      const bf16_t* wrow = a.w + (int64_t)n * a.ldw + kbeg;
#pragma unroll
      for (int s = 0; s < STEPS; ++s) wreg[t][s] = *(const uint4*)(wrow + s * SK_KSTEP);
    }
  }
  // all of W's loads are in flight before anything waits: left to itself the compiler interleaves
  // them with the products to save registers, and the matrix no longer streams at memory speed
  __builtin_amdgcn_sched_barrier(0);

  float4_t acc[RT][CB];
#pragma unroll
  for (int t = 0; t < RT; ++t)
#pragma unroll
    for (int b = 0; b < CB; ++b) acc[t][b] = (float4_t){0.f, 0.f, 0.f, 0.f};

  float sq = 0.f;                                       // MODE_NORM: this lane's share of its row's sum of squares
  if (MODE == MODE_NORM) {
    // ---- (x + res) * nw of this wave's slice, rounded, is the operand. The row's scale
    // rsqrt(mean((x + res)^2) + eps) is a number per row: it multiplies the finished sums on the way
    // out instead of every operand on the way in, so no wave waits for the others' squares first.
    const bool has_res = a.res != nullptr;
    uint4 xb[STEPS];
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
      // (both loads are used whatever the case, so that neither moves behind the loads of W)
      float xs[8], rv[8], nv[8];
      sk_unpack(xraw[s], xs);
      sk_unpack(rraw[s], rv);
      sk_unpack(nraw[s], nv);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float sum = xs[i] + (has_res ? rv[i] : 0.f);
        xs[i] = xok[0] ? sum : 0.f;                      // rows past M count as zeros
      }
      if (has_res && blockIdx.x == 0 && xok[0]) *(uint4*)(a.res_out + (int64_t)r * a.K + kbeg + s * SK_KSTEP) = sk_pack(xs);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        sq = fmaf(xs[i], xs[i], sq);
        xs[i] *= nv[i];
      }
      xb[s] = sk_pack(xs);
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int s = 0; s < STEPS; ++s)
#pragma unroll
      for (int t = 0; t < RT; ++t) acc[t][0] = sk_mfma(wreg[t][s], xb[s], acc[t][0]);
    sq += __shfl_xor(sq, 16, TS_WAVE);
    sq += __shfl_xor(sq, 32, TS_WAVE);
    if (g == 0) ssq[wave * 16 + r] = sq;
  } else {
    // ---- x in batches of steps, then the products
#pragma unroll
    for (int s0 = 0; s0 < STEPS; s0 += SK_XBATCH) {
      uint4 xb[CB][SK_XBATCH];
#pragma unroll
      for (int b = 0; b < CB; ++b)
#pragma unroll
        for (int s = 0; s < SK_XBATCH; ++s)
          xb[b][s] = *(const uint4*)(xrow[b] + (s0 + s) * SK_KSTEP);   // rows past M repeat row 0 and are not stored
      __builtin_amdgcn_sched_barrier(0);                // the batch is asked for at once
#pragma unroll
      for (int s = 0; s < SK_XBATCH; ++s)
#pragma unroll
        for (int t = 0; t < RT; ++t)
#pragma unroll
          for (int b = 0; b < CB; ++b) acc[t][b] = sk_mfma(wreg[t][s0 + s], xb[b][s], acc[t][b]);
    }
  }
  // acc[t][b][j] = sum over this wave's k of W[row 16 t + 4 g + j of the workgroup, k] * f(x)[16 b + r, k]
#pragma unroll
  for (int t = 0; t < RT; ++t)
#pragma unroll
    for (int b = 0; b < CB; ++b)
#pragma unroll
      for (int j = 0; j < 4; ++j) part[(((size_t)wave * RT + t) * CB + b) * 256 + r * 16 + 4 * g + j] = acc[t][b][j];
  __syncthreads();
  // part[.][t][b][m_local * 16 + n_local]: a thread sums 4 consecutive n of one m over the waves in order
  OUT* y = (OUT*)a.y;
  const int ncols = GLU ? half : a.N;
  // ROPE: a tile gives 8 columns of a head's first half (n_local 0 .. 7) and their partners (n_local 8 .. 15): 32 items of 4
  constexpr int PER_TILE = ROPE ? 32 : 64;
  for (int idx = threadIdx.x; idx < OT * CB * PER_TILE; idx += blockDim.x) {
    const int tile = idx / PER_TILE, e = idx - tile * PER_TILE;
    const int t = tile / CB, b = tile - t * CB;
    const int ml = ROPE ? e >> 1 : e >> 2, nl = ROPE ? (e & 1) * 4 : (e & 3) * 4;
    const int m = b * 16 + ml, n = n0 + t * 16 + nl;
    if (m >= a.M) continue;
    float s[4] = {0.f, 0.f, 0.f, 0.f}, u[4] = {0.f, 0.f, 0.f, 0.f};
    for (int wv = 0; wv < nwaves; ++wv) {
      const float* p = part + (((size_t)wv * RT + t) * CB + b) * 256 + ml * 16 + nl;
#pragma unroll
      for (int j = 0; j < 4; ++j) s[j] += p[j];
      if (PAIRS) {
        const float* pu = ROPE ? p + 8 : part + (((size_t)wv * RT + t + OT) * CB + b) * 256 + ml * 16 + nl;
#pragma unroll
        for (int j = 0; j < 4; ++j) u[j] += pu[j];
      }
    }
    if (MODE == MODE_NORM) {                              // the row's scale, from every wave's squares
      float total = 0.f;
      for (int wv = 0; wv < nwaves; ++wv) total += ssq[wv * 16 + ml];
      const float inv = 1.0f / sqrtf(total / (float)a.K + a.eps);
#pragma unroll
      for (int j = 0; j < 4; ++j) { s[j] *= inv; u[j] *= inv; }
    }
    if (ROPE) {
      const int per_head = a.hd / 16, jb = blockIdx.x * RT + t, hdh = a.hd / 2;
      const int head = jb / per_head, d0 = 8 * (jb % per_head) + nl;    // d0 .. d0 + 3 of the head's first half
      if (head >= a.nh + 2 * a.nkv) continue;
      float y1[4], y2[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {                       // as the product would be stored
        y1[j] = __uint_as_float(sk_round(s[j]) << 16);
        y2[j] = __uint_as_float(sk_round(u[j]) << 16);
      }
      if (a.rotate && head < a.nh + a.nkv) {
        const float* cs = a.cos_sin + (int64_t)a.positions[m] * a.hd + d0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float c = cs[j], sn = cs[hdh + j];
          const float r1 = y1[j] * c - y2[j] * sn, r2 = y2[j] * c + y1[j] * sn;
          y1[j] = r1;
          y2[j] = r2;
        }
      }
      const uint2 o1 = make_uint2(sk_round(y1[0]) | (sk_round(y1[1]) << 16), sk_round(y1[2]) | (sk_round(y1[3]) << 16));
      const uint2 o2 = make_uint2(sk_round(y2[0]) | (sk_round(y2[1]) << 16), sk_round(y2[2]) | (sk_round(y2[3]) << 16));
      if (head < a.nh) {
        bf16_t* dst = a.q_out + ((int64_t)m * a.nh + head) * a.hd + d0;
        *(uint2*)dst = o1;
        *(uint2*)(dst + hdh) = o2;
        continue;
      }
      const int64_t slot = a.slots ? a.slots[m] : -1;
      if (!a.k_cache || slot < 0) continue;
      const int64_t page = slot / a.page_size, off = slot - page * a.page_size;
      if (head < a.nh + a.nkv) {
        bf16_t* dst = a.k_cache + page * a.kp + off * a.ks + (int64_t)(head - a.nh) * a.kh + d0;
        *(uint2*)dst = o1;
        *(uint2*)(dst + hdh) = o2;
      } else {
        bf16_t* dst = a.v_cache + page * a.vp + off * a.vs + (int64_t)(head - a.nh - a.nkv) * a.vh + (int64_t)d0 * a.vd;
        const uint32_t w1[2] = {o1.x, o1.y}, w2[2] = {o2.x, o2.y};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          dst[(int64_t)j * a.vd] = (bf16_t)(w1[j >> 1] >> (16 * (j & 1)));
          dst[(int64_t)(hdh + j) * a.vd] = (bf16_t)(w2[j >> 1] >> (16 * (j & 1)));
        }
      }
      continue;
    }
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (n + j < ncols) Num<OUT>::st(y + (int64_t)m * a.ldy + n + j, GLU ? sk_silu(s[j]) * u[j] : s[j]);
  }
}

template <int RT, int CB, int STEPS, int MODE, int GLU, typename OUT>
static int sk_launch(const SkinnyArgs& a, hipStream_t stream) {
  const int nwaves = a.K / (STEPS * SK_KSTEP);
  const size_t smem = sizeof(float) * ((size_t)nwaves * RT * CB * 256 + (size_t)nwaves * 16);
  constexpr int OT = GLU == EPI_GLU ? RT / 2 : RT;
  const int ncols = GLU == EPI_GLU ? a.N / 2 : a.N;     // (EPI_ROPE: a 16-row tile of the matrix per 8 columns and their partners)
  dim3 grid((ncols + 16 * OT - 1) / (16 * OT)), block(nwaves * TS_WAVE);
  if (nwaves <= 8) {
    gemm_skinny_kernel<RT, CB, STEPS, MODE, GLU, 512, OUT><<<grid, block, smem, stream>>>(a);
  } else {
    // a workgroup of 16 waves has 128 registers a lane: one or two row tiles, and no fused norm
    if constexpr (MODE == MODE_PLAIN && (RT == 1 || (RT == 2 && CB == 1)))
      gemm_skinny_kernel<RT, CB, STEPS, MODE, GLU, 1024, OUT><<<grid, block, smem, stream>>>(a);
    else return TS_BAD_SHAPE;
  }
  return ts_check_launch();
}

// Picks the instance: slices of 256 k while that needs at most 16 waves, else slices of 512; more
// rows of W per workgroup for wide matrices once that still leaves a workgroup per compute unit
// (fewer workgroups repeat less of the work on x).
template <int MODE, int GLU, typename OUT>
static int sk_dispatch(const SkinnyArgs& a, hipStream_t stream) {
  const int steps = (a.K % 256 == 0 && a.K / 256 <= 16) ? 8 : 16;
  if (a.K % (steps * SK_KSTEP) || a.K / (steps * SK_KSTEP) > 16) return TS_BAD_SHAPE;
  const int nwaves = a.K / (steps * SK_KSTEP);
  const int cb = (a.M + 15) / 16;
  if (MODE == MODE_NORM && cb != 1) return TS_BAD_SHAPE;
  const int ncols = GLU ? a.N / 2 : a.N;
#define SK_GO(RT, CB, ST) return sk_launch<RT, CB, ST, MODE, GLU, OUT>(a, stream)
  if constexpr (MODE == MODE_NORM || GLU != 0) {
    // the instances that hold x + res or four row tiles need the registers of a workgroup of 8 waves
    if (steps != 8) return TS_BAD_SHAPE;
    if constexpr (MODE == MODE_PLAIN && GLU != 0) {
      // the gate for 17 to 64 rows of x: two or four blocks of rows against the same registers of W
      if (cb > 1 && nwaves > 8) return TS_BAD_SHAPE;
      if (cb == 2) { if (ncols >= 4096) SK_GO(4, 2, 8); else SK_GO(2, 2, 8); }
      if (cb > 2) SK_GO(2, 4, 8);
    }
    if (nwaves <= 8) {
      if (ncols >= 4096 * (GLU ? 1 : 2)) SK_GO(4, 1, 8);
      if (GLU || ncols >= 4096) SK_GO(2, 1, 8);
    }
    if constexpr (GLU == 0) SK_GO(1, 1, 8);
    if constexpr (MODE == MODE_PLAIN) SK_GO(2, 1, 8);   // the gate alone, in a workgroup of up to 16 waves
    return TS_BAD_SHAPE;
  } else {
    const bool two = a.N >= 8192 && (nwaves <= 8 || cb == 1);
    if (steps == 8) {
      if (two) { if (cb == 1) SK_GO(2, 1, 8); else SK_GO(2, 2, 8); }
      if (cb == 1) SK_GO(1, 1, 8); else SK_GO(1, 2, 8);
    }
    if (cb == 1) SK_GO(1, 1, 16); else SK_GO(1, 2, 16);
  }
#undef SK_GO
}

// ---- up to 8 rows of x, narrow matrices ------------------------------------------------------------
// With at most 8 rows of x, half of a 16 x 16 x 32 matrix instruction would multiply rows that do not
// exist. Here it multiplies 8 rows of W by 8 rows of x over 64 k instead: lanes r < 8 of the A operand
// hold rows n0 .. n0 + 7 of W at k, lanes r >= 8 the same rows at k + 32 STEPS; the B operand holds
// the rows of x at k in its columns 0 .. 7 and at k + 32 STEPS in its columns 8 .. 15. Of the 16 x 16
// result the two 8 x 8 blocks on the diagonal are the two halves of the sum; the other two blocks mix
// the halves and are dropped. A workgroup then owns 8 rows of W, not 16: a matrix of 2,048 rows
// gives 256 workgroups, one per compute unit, and a reduction of 8,192 fits the 8 waves of one
// workgroup (a wave covers 64 STEPS of k), where the 16-row form needs 16 waves on half the chip.
// packed: W in the order of these loads, [N / 8 tiles][waves][STEPS][lane][8] (see hip.pack_weight8).
template <int STEPS, int MAXT, typename OUT>
__global__ void __launch_bounds__(MAXT)
gemm_skinny8_kernel(const SkinnyArgs a) {
  extern __shared__ __align__(16) float smem[];         // [nwaves][256]
  const int nwaves = blockDim.x / TS_WAVE;
  const int wave = threadIdx.x / TS_WAVE, lane = threadIdx.x & (TS_WAVE - 1);
  const int r = lane & 15, g = lane >> 4, row = r & 7, half = r >> 3;
  const int n0 = blockIdx.x * 8;
  const int kbeg = wave * (2 * STEPS * SK_KSTEP) + half * (STEPS * SK_KSTEP) + 8 * g;   // this lane's first k
  // x first where the registers allow it (workgroups of up to 8 waves): it is small and comes from the
  // cache, loads return in the order they were issued, and so the products start the moment W is there;
  // a larger workgroup has half the registers and fetches x in batches after W instead
  constexpr bool X_FIRST = MAXT <= 512;
  constexpr int XB = X_FIRST ? STEPS : (STEPS < 8 ? STEPS : 8);
  const bf16_t* xrow = a.x + (int64_t)(row < a.M ? row : 0) * a.ldx + kbeg;   // rows past M repeat row 0 and are not stored
  uint4 xb[XB];
  if (X_FIRST) {
#pragma unroll
    for (int s = 0; s < STEPS; ++s) xb[s] = *(const uint4*)(xrow + s * SK_KSTEP);
    __builtin_amdgcn_sched_barrier(0);
  }
  uint4 wreg[STEPS];
  if (a.packed) {
    const bf16_t* blk = a.w + ((((int64_t)blockIdx.x * nwaves + wave) * STEPS) * 64 + lane) * 8;
#pragma unroll
    for (int s = 0; s < STEPS; ++s) wreg[s] = *(const uint4*)(blk + (int64_t)s * 512);
  } else {
    const int n = n0 + row < a.N ? n0 + row : a.N - 1;    // rows past the end are computed and not stored
    const bf16_t* wrow = a.w + (int64_t)n * a.ldw + kbeg;
#pragma unroll
    for (int s = 0; s < STEPS; ++s) wreg[s] = *(const uint4*)(wrow + s * SK_KSTEP);
  }
  __builtin_amdgcn_sched_barrier(0);                    // all of W's loads are in flight before anything waits
  float4_t acc = {0.f, 0.f, 0.f, 0.f};
  if (X_FIRST) {
#pragma unroll
    for (int s = 0; s < STEPS; ++s) acc = sk_mfma(wreg[s], xb[s], acc);
  } else {
#pragma unroll
    for (int s0 = 0; s0 < STEPS; s0 += XB) {
#pragma unroll
      for (int s = 0; s < XB; ++s) xb[s] = *(const uint4*)(xrow + (s0 + s) * SK_KSTEP);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int s = 0; s < XB; ++s) acc = sk_mfma(wreg[s0 + s], xb[s], acc);
    }
  }
  // acc[j] = D[4 g + j][r]: W row (4 g + j) & 7 of half (4 g + j) >> 3 times x row r & 7 of half r >> 3
#pragma unroll
  for (int j = 0; j < 4; ++j) smem[wave * 256 + r * 16 + 4 * g + j] = acc[j];
  __syncthreads();
  if (threadIdx.x >= 64) return;
  const int m = threadIdx.x >> 3, nl = threadIdx.x & 7;  // x row, W row of the tile
  float sum = 0.f;
  for (int wv = 0; wv < nwaves; ++wv)                    // waves in order, within a wave the lower half of k first
    sum += smem[wv * 256 + m * 16 + nl] + smem[wv * 256 + (m + 8) * 16 + nl + 8];
  const int n = n0 + nl;
  if constexpr (sizeof(OUT) == 4) {
    if (m < a.M && n < a.N) ((float*)a.y)[(int64_t)m * a.ldy + n] = sum;
  } else {
    const uint32_t mine = sk_round(sum), next = __shfl_down(mine, 1, TS_WAVE);
    if (m < a.M && !(nl & 1)) {
      bf16_t* dst = (bf16_t*)a.y + (int64_t)m * a.ldy + n;
      if (n + 1 < a.N && !(((uintptr_t)dst) & 3)) *(uint32_t*)dst = mine | (next << 16);
      else {
        if (n < a.N) dst[0] = (bf16_t)mine;
        if (n + 1 < a.N) dst[1] = (bf16_t)next;
      }
    }
  }
}

template <typename OUT>
static int sk8_dispatch(const SkinnyArgs& a, hipStream_t stream) {
  // a wave covers 64 STEPS of k; 8 waves where the reduction allows it, never more than 16
  int steps = 0;
  for (int cand : {4, 8, 16})
    if (!steps && a.K % (64 * cand) == 0 && a.K / (64 * cand) <= 8) steps = cand;
  if (!steps && a.K % 1024 == 0 && a.K / 1024 <= 16) steps = 16;
  if (!steps) return TS_BAD_SHAPE;
  const int nwaves = a.K / (64 * steps);
  dim3 grid((a.N + 7) / 8), block(nwaves * TS_WAVE);
  const size_t smem = sizeof(float) * 256 * nwaves;
  if (steps == 4) gemm_skinny8_kernel<4, 512, OUT><<<grid, block, smem, stream>>>(a);
  else if (steps == 8) gemm_skinny8_kernel<8, 512, OUT><<<grid, block, smem, stream>>>(a);
  else if (nwaves <= 8) gemm_skinny8_kernel<16, 512, OUT><<<grid, block, smem, stream>>>(a);
  else gemm_skinny8_kernel<16, 1024, OUT><<<grid, block, smem, stream>>>(a);
  return ts_check_launch();
}

// y [M <= 8, N] = x · W^T by the 8-row form above: K a multiple of 256 up to 8,192 or of 1,024 up to
// 16,384; contiguous 16-byte aligned rows. out_dtype: 1 bfloat16, 0 float. packed: w is
// hip.pack_weight8(W) for this K, ldw unused, N a multiple of 8.
extern "C" int ts_gemm_skinny8_bf16(void* y, const void* x, const void* w, int M, int N, int K, int64_t ldx, int64_t ldw,
                                    int64_t ldy, int out_dtype, int packed, hipStream_t stream) {
  if (M <= 0 || N <= 0) return TS_OK;
  if (M > 8 || K <= 0 || ldx % 8 || ldx < K || ldy < N || (!packed && (ldw % 8 || ldw < K)) || (packed && N % 8)) return TS_BAD_SHAPE;
  if (((uintptr_t)x | (uintptr_t)w) & 15 || !y) return TS_BAD_SHAPE;
  SkinnyArgs a = {};
  a.x = (const bf16_t*)x; a.w = (const bf16_t*)w; a.y = y; a.M = M; a.N = N; a.K = K; a.ldx = ldx; a.ldw = ldw; a.ldy = ldy;
  a.packed = packed;
  if (out_dtype == 1) return sk8_dispatch<bf16_t>(a, stream);
  if (out_dtype == 0) return sk8_dispatch<float>(a, stream);
  return TS_BAD_DTYPE;
}

// mode: 0 plain, 1 residual + RMSNorm on the way in (M <= 16, K in steps of 256 up to 2048). glu: W holds
// gate rows then up rows, y is [M, N / 2] = silu(gate) * up (M <= 16, K up to 4096, 2048 with the norm). out_dtype: 1 bfloat16, 0 float
// (plain only). packed: w holds the matrix in the kernel's own order (see the loads of W), ldw is unused. Requires M <= 32 (the gate
// alone: M <= 64 for K up to 2048), K a multiple of 256 (up to 4096) or of 512 (up to 8192), contiguous
// 16-byte aligned rows; mode 1 takes x, res, res_out as dense [M, K].
extern "C" int ts_gemm_skinny_bf16(void* y, const void* x, const void* w, const void* res, const void* nw,
                                   void* res_out, int M, int N, int K, int64_t ldx, int64_t ldw, int64_t ldy,
                                   float eps, int mode, int glu, int out_dtype, int packed, hipStream_t stream) {
  if (M <= 0 || N <= 0) return TS_OK;
  if (M > (glu && mode == MODE_PLAIN ? 64 : 32) || K <= 0 || ldx % 8 || ldw % 8 || ldx < K || ldw < K || ldy < (glu ? N / 2 : N)) return TS_BAD_SHAPE;
  if (glu && (N % 2 || (N / 2) % 16)) return TS_BAD_SHAPE;
  if (((uintptr_t)x | (uintptr_t)w | (uintptr_t)res | (uintptr_t)nw | (uintptr_t)res_out) & 15) return TS_BAD_SHAPE;
  if (mode == MODE_NORM && (!nw || (res && !res_out))) return TS_BAD_SHAPE;
  SkinnyArgs a = {};
  a.x = (const bf16_t*)x; a.res = (const bf16_t*)res; a.nw = (const bf16_t*)nw; a.res_out = (bf16_t*)res_out;
  a.w = (const bf16_t*)w; a.y = y; a.M = M; a.N = N; a.K = K; a.ldx = ldx; a.ldw = ldw; a.ldy = ldy; a.eps = eps; a.packed = packed;
  if (out_dtype == 1) {
    if (mode == MODE_PLAIN && !glu) return sk_dispatch<MODE_PLAIN, 0, bf16_t>(a, stream);
    if (mode == MODE_PLAIN && glu) return sk_dispatch<MODE_PLAIN, 1, bf16_t>(a, stream);
    if (mode == MODE_NORM && !glu) return sk_dispatch<MODE_NORM, 0, bf16_t>(a, stream);
    if (mode == MODE_NORM && glu) return sk_dispatch<MODE_NORM, 1, bf16_t>(a, stream);
    return TS_BAD_SHAPE;
  }
  if (out_dtype == 0 && mode == MODE_PLAIN && !glu) return sk_dispatch<MODE_PLAIN, 0, float>(a, stream);
  return TS_BAD_DTYPE;
}

// The qkv projection of an attention layer with the rotation and the cache write on the way out:
// q_out [M, nh * hd] gets the rotated queries, the rotated keys and the values go to the slots
// `slots[m]` of the pages (see SkinnyArgs); w is [(nh + 2 nkv) * hd, K]. mode as above. Requires
// M <= 16 (without the norm: M <= 64 for K up to 2048), hd a multiple of 32, K a multiple of 256 up to 4096
// (2048 with the norm), 8-byte aligned cache strides.
extern "C" int ts_gemm_skinny_rope_bf16(void* q_out, const void* x, const void* w, const void* res, const void* nw,
                                        void* res_out, int M, int K, int64_t ldx, int64_t ldw, float eps, int mode,
                                        int packed, const float* cos_sin, const int32_t* positions, const int32_t* slots,
                                        void* k_cache, void* v_cache, int nh, int nkv, int hd, int rotate,
                                        int page_size, int64_t kp, int64_t ks, int64_t kh, int64_t vp, int64_t vs,
                                        int64_t vh, int64_t vd, hipStream_t stream) {
  if (M <= 0) return TS_OK;
  if (M > (mode == MODE_PLAIN && K <= 2048 ? 64 : 16) || K <= 0 || K % 256 || K / 256 > (mode == MODE_NORM ? 8 : 16) || ldx % 8 || ldw % 8 || ldx < K || ldw < K) return TS_BAD_SHAPE;
  if (nh <= 0 || nkv < 0 || hd <= 0 || hd % 32 || page_size <= 0) return TS_BAD_SHAPE;
  if (((uintptr_t)x | (uintptr_t)w | (uintptr_t)res | (uintptr_t)nw | (uintptr_t)res_out | (uintptr_t)q_out) & 15)
    return TS_BAD_SHAPE;
  if (mode == MODE_NORM && (!nw || (res && !res_out))) return TS_BAD_SHAPE;
  if (rotate && (!cos_sin || !positions)) return TS_BAD_SHAPE;
  if (k_cache && (!v_cache || !slots || (kp % 4) || (ks % 4) || (kh % 4) || (((uintptr_t)k_cache) & 7))) return TS_BAD_SHAPE;
  SkinnyArgs a = {};
  a.x = (const bf16_t*)x; a.res = (const bf16_t*)res; a.nw = (const bf16_t*)nw; a.res_out = (bf16_t*)res_out;
  a.w = (const bf16_t*)w; a.y = nullptr; a.M = M; a.N = (nh + 2 * nkv) * hd; a.K = K; a.ldx = ldx; a.ldw = ldw;
  a.ldy = 0; a.eps = eps; a.packed = packed;
  a.cos_sin = cos_sin; a.positions = positions; a.slots = slots; a.q_out = (bf16_t*)q_out;
  a.k_cache = (bf16_t*)k_cache; a.v_cache = (bf16_t*)v_cache; a.nh = nh; a.nkv = nkv; a.hd = hd; a.rotate = rotate;
  a.page_size = page_size; a.kp = kp; a.ks = ks; a.kh = kh; a.vp = vp; a.vs = vs; a.vh = vh; a.vd = vd;
  if (mode == MODE_PLAIN && M > 32) return sk_launch<1, 4, 8, MODE_PLAIN, EPI_ROPE, bf16_t>(a, stream);
  if (mode == MODE_PLAIN && M > 16) return sk_launch<1, 2, 8, MODE_PLAIN, EPI_ROPE, bf16_t>(a, stream);
  if (mode == MODE_PLAIN) return sk_launch<1, 1, 8, MODE_PLAIN, EPI_ROPE, bf16_t>(a, stream);
  if (mode == MODE_NORM) return sk_launch<1, 1, 8, MODE_NORM, EPI_ROPE, bf16_t>(a, stream);
  return TS_BAD_SHAPE;
}
