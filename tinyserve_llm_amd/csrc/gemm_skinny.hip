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
//   MODE_PREP  the norm on the way in, half done already by the kernel that made x (EPI_NEXT below):
//              x is the operand T((h + res) * nw) as it stands, and the row's scale comes from the
//              partial sums of squares that kernel left, one per row and column tile, added up in
//              the tiles' order; any number of 16-row blocks of x
//   EPI_NEXT   what follows a projection whose result goes into a residual sum and a norm: with
//              t = T(y) + res, the kernel writes T(t) as the new residual, T(t * nw) as the next
//              projection's operand and, per row and 16-column tile (8 in the 8-row form), the sum of
//              t^2 over the tile's columns; y itself is not stored
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
  // Up to 8 rows in the order the 8-row form's lanes read them, [K / (64 steps)][steps][64 lanes][8]: lane
  // r + 16 g of (wave, step) holds row r % 8 at k = 64 steps wave + 32 steps (r / 8) + 32 step + 8 g .. + 7, so
  // that a load is a contiguous kilobyte instead of 64 bytes of each of 8 rows in two places (the down
  // projection of 8 rows over 8,192: 10.8 -> 9.2 us). y_pack8 > 0: the gated product is stored that way for a
  // reader of y_pack8 steps; x_packed8: x comes that way (ldx is unused). Lanes of rows past M hold anything.
  int x_packed8, y_pack8;
  // x_packed8 == 2: the 8-row form for one token (M = 1), x not given but made on the way in from the parts that the
  // split-key attention kernel has left (the combining kernel's sums, bit for bit): x is the token's heads side by
  // side, head h of it sum_s o[h, s, :] 2^(m_s - M) / sum_s l_s 2^(m_s - M) over the chunks s that hold keys it
  // sees. Its operands travel in fields that the 8-row form leaves unused otherwise, so that the block of arguments
  // which every kernel of this file fetches stays as short as it is (see SkinnyParts).
  int64_t ldx, ldw, ldy;
  float eps;
  // MODE_PREP: sums of squares [M, ssq_parts] of the rows of h + res, in parts (K is their width)
  const float* ssq_in;
  int ssq_parts;
  // EPI_NEXT: res [M, N] or null, next norm's weight [N], outputs [M, N] dense and [M, tiles of the grid]
  const bf16_t* next_res;
  const bf16_t* next_nw;
  bf16_t* next_res_out;
  bf16_t* next_op;
  float* ssq_out;
  // EPI_ROPE: N = (nh + 2 nkv) * hd; cos_sin [max_pos, hd] 32-bit, [cos | sin] halves; slot -1 stores nothing.
  // key element: page * kp + offset * ks + head * kh + d; value element: page * vp + offset * vs + head * vh + d * vd
  const float* cos_sin;
  const int32_t* positions;
  const int32_t* slots;
  bf16_t* q_out;        // [M, nh * hd]
  bf16_t* k_cache;      // null: this layer owns no cache, only q is produced
  bf16_t* v_cache;
  int nh, nkv, hd, rotate, page_size;
  int table_vec;        // cos_sin is 16-byte aligned: four of its values go in one load
  int64_t kp, ks, kh, vp, vs, vh, vd;
};

// RT: 16-row tiles of W per workgroup; CB: 16-row blocks of x; STEPS: 32-wide k steps per wave;
// MAXT: most threads a workgroup of this instance is launched with (it bounds the registers)
template <int RT, int CB, int STEPS, int MODE, int EPI, int MAXT, typename OUT>
__global__ void __launch_bounds__(MAXT)
gemm_skinny_kernel(const SkinnyArgs a) {
  constexpr bool GLU = EPI == EPI_GLU, ROPE = EPI == EPI_ROPE, PAIRS = GLU || ROPE, NEXT = EPI == EPI_NEXT;
  static_assert(MODE != MODE_NORM || CB == 1, "the fused norm serves one block of rows");
  static_assert(!GLU || RT % 2 == 0, "gate and up tiles come in pairs");
  // steps of x fetched at a time: fewer where more blocks of x, more row tiles of W or a larger workgroup leave fewer registers
  constexpr int SK_XBATCH = CB >= 4 ? 4 : (CB == 2 && (MAXT > 512 || RT >= 4)) ? 4 : 8;
  ts_fetch_arguments<sizeof(SkinnyArgs)>();
  extern __shared__ __align__(16) float smem[];
  const int nwaves = blockDim.x / TS_WAVE;
  float* part = smem;                                   // [nwaves][RT][CB][256]
  float* ssq = smem + (size_t)nwaves * RT * CB * 256;   // MODE_NORM: [nwaves][16]; MODE_PREP: [CB][nwaves][16]
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

  // ---- MODE_PLAIN with room in the registers: all of this wave's x is asked for before W. It is
  // small and comes from the cache, loads come back in the order they were issued, and so the products
  // can start the moment W has arrived; asked for after W, every batch of x would wait behind all of W
  // and then for its own trip to the cache.
  constexpr bool X_FIRST = MODE != MODE_NORM && MAXT <= 512 && (CB * STEPS + RT * STEPS) <= 48;
  // ---- with more than one block of rows the loads of x outnumber W's, and a load that gathers 64 bytes of each
  // of 16 rows costs far more than one of long pieces (q|k|v of 64 rows: 10.9 us, 8.0 with contiguous loads):
  // the wave then fetches its slice of a block's rows whole (STEPS 64 bytes of a row side by side, 64 / (4 STEPS)
  // rows a load) and turns them into operand order through LDS once W's loads are out (sk_place). (Not where a
  // wave has more row tiles of W than blocks of x: the gate|up product of 24 rows, 4 tiles against 2 blocks, takes
  // 16.7 us that way and 16.5 as it is.)
  constexpr bool X_TURNED = X_FIRST && CB >= 2 && CB >= RT;
  constexpr int X_LANES = 4 * STEPS <= TS_WAVE ? 4 * STEPS : TS_WAVE;     // lanes that share a row of such a load
  static_assert(!X_TURNED || 4 * STEPS <= TS_WAVE, "a wave's slice of a row is at most a kilobyte");
  uint4 xall[X_FIRST ? CB : 1][X_FIRST ? STEPS : 1];
  if constexpr (X_TURNED) {
    const int lr = lane / X_LANES, piece = lane % X_LANES;
#pragma unroll
    for (int b = 0; b < CB; ++b)
#pragma unroll
      for (int j = 0; j < STEPS; ++j) {
        const int m = b * 16 + j * (TS_WAVE / X_LANES) + lr;              // rows past M repeat row 0 and are not stored
        xall[b][j] = *(const uint4*)(a.x + (int64_t)(m < a.M ? m : 0) * a.ldx + wave * STEPS * SK_KSTEP + 8 * piece);
      }
    __builtin_amdgcn_sched_barrier(0);
  } else if constexpr (X_FIRST) {
#pragma unroll
    for (int b = 0; b < CB; ++b)
#pragma unroll
      for (int s = 0; s < STEPS; ++s) xall[b][s] = *(const uint4*)(xrow[b] + s * SK_KSTEP);   // rows past M repeat row 0 and are not stored
    __builtin_amdgcn_sched_barrier(0);
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

  // ---- MODE_PREP: the rows' sums of squares, from the parts the kernel before left. The parts of a
  // row are dealt out in runs to the 4 x nwaves lanes that hold the row (lane (r, g) of wave w adds up
  // run 4 w + g of row 16 b + r), and the runs' sums meet in LDS as the waves' squares do in MODE_NORM.
  // The parts are asked for here, right behind W (whose addresses are in registers when the wave
  // starts, while the address of the parts has to be fetched first: asked for ahead of W they would
  // hold W back), and added up after the products. (Runs longer than the registers set aside hold,
  // as short reductions with their few waves have, are fetched and added after the products.)
  constexpr int PREP_VECS = 2;                          // 16-byte pieces of a run that a lane holds
  float4 pv[MODE == MODE_PREP ? CB : 1][MODE == MODE_PREP ? PREP_VECS : 1];
  // parts of a row per lane, in whole pieces of four
  const int prep_run = MODE == MODE_PREP ? (a.ssq_parts + 16 * nwaves - 1) / (16 * nwaves) * 4 : 0;
  const bool prep_early = MODE == MODE_PREP && prep_run <= 4 * PREP_VECS && a.ssq_parts % 4 == 0;
  if constexpr (MODE == MODE_PREP) {
    if (prep_early) {
      const int first = (4 * wave + g) * prep_run;
#pragma unroll
      for (int b = 0; b < CB; ++b)
#pragma unroll
        for (int i = 0; i < PREP_VECS; ++i)
          pv[b][i] = (xok[b] && 4 * i < prep_run && first + 4 * i < a.ssq_parts)
                         ? *(const float4*)(a.ssq_in + (int64_t)(16 * b + r) * a.ssq_parts + first + 4 * i)
                         : make_float4(0.f, 0.f, 0.f, 0.f);
    }
    __builtin_amdgcn_sched_barrier(0);
  }

  // ---- EPI_NEXT: the residual and the next norm's weight of the four columns this thread will finish
  // are asked for right behind W (where every thread finishes at most one item and the columns are
  // whole), so that the way out does not wait for a trip to the cache
  constexpr int NEXT_ITEMS = (EPI == EPI_GLU ? RT / 2 : RT) * CB * 64;
  const bool next_early = NEXT && NEXT_ITEMS <= (int)blockDim.x && a.N % 4 == 0;
  uint2 pre_res = make_uint2(0, 0), pre_nw = make_uint2(0, 0);
  if constexpr (NEXT) {
    if (next_early && (int)threadIdx.x < NEXT_ITEMS) {
      const int tile = threadIdx.x / 64, e = threadIdx.x - tile * 64;
      const int t = tile / CB, b = tile - t * CB, m = b * 16 + (e >> 2), n = n0 + t * 16 + (e & 3) * 4;
      if (m < a.M && n < a.N) {
        pre_nw = *(const uint2*)(a.next_nw + n);
        if (a.next_res) pre_res = *(const uint2*)(a.next_res + (int64_t)m * a.N + n);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
  }

  // ---- EPI_ROPE: the position and the slot of the token this thread will finish are asked for right
  // behind W as well, and the table's values of that position after the products, ahead of the
  // waves' meeting, so that neither trip to the cache is made on the way out
  constexpr int ROPE_ITEMS = RT * CB * 32;
  const bool rope_early = ROPE && ROPE_ITEMS <= (int)blockDim.x && a.table_vec;
  int pre_pos = 0;
  int pre_slot = -1;
  // (the same for what else the way out needs and the products do not give: which head and which of its
  // dimensions this thread finishes, where its parts lie in LDS and where its values go. A wave has nothing
  // to do while W is on its way; after the waves' meeting every instruction is waited for.)
  int way_kind = 0;                                     // 0 nothing, 1 a query or a key (two pieces half a head apart), 2 a value
  int way_part = 0, way_ssq = 0, way_head = 0, way_d0 = 0;
  bf16_t* way_dst = nullptr;
  float inv_k = 1.0f / (float)a.K;
  if constexpr (ROPE) {
    if (rope_early && (int)threadIdx.x < ROPE_ITEMS) {
      const int tile = threadIdx.x / 32, t = tile / CB, b = tile - t * CB, ml = (threadIdx.x & 31) >> 1, nl = (threadIdx.x & 1) * 4;
      const int m = b * 16 + ml;
      const int per_head = a.hd / 16, jb = blockIdx.x * RT + t;
      way_head = jb / per_head;
      way_d0 = 8 * (jb % per_head) + nl;
      way_part = (t * CB + b) * 256 + ml * 16 + nl;
      way_ssq = (MODE == MODE_PREP ? b * nwaves : 0) * 16 + ml;
      if (m < a.M && way_head < a.nh + 2 * a.nkv) {
        if (a.rotate) pre_pos = a.positions[m];
        if (a.slots) pre_slot = a.slots[m];
        way_kind = way_head < a.nh + a.nkv ? 1 : 2;
        if (way_head < a.nh) way_dst = a.q_out + ((int64_t)m * a.nh + way_head) * a.hd + way_d0;
      }
    }
    asm volatile("" : "+v"(way_kind), "+v"(way_part), "+v"(way_ssq), "+v"(way_dst), "+v"(inv_k));
    __builtin_amdgcn_sched_barrier(0);
  }
  // ---- EPI_GLU in bfloat16, four whole columns a thread and at most one item a thread: likewise
  constexpr int GLU_ITEMS = OT * CB * 64;
  const bool glu_early = GLU && sizeof(OUT) == 2 && GLU_ITEMS <= (int)blockDim.x &&
                         (a.y_pack8 || (half % 4 == 0 && a.ldy % 4 == 0 && !(((uintptr_t)a.y) & 7)));
  if constexpr (GLU && sizeof(OUT) == 2) {
    if (glu_early && (int)threadIdx.x < GLU_ITEMS) {
      const int tile = threadIdx.x / 64, e = threadIdx.x & 63, t = tile / CB, b = tile - t * CB, ml = e >> 2, nl = (e & 3) * 4;
      const int m = b * 16 + ml, n = n0 + t * 16 + nl;
      way_part = (t * CB + b) * 256 + ml * 16 + nl;
      way_ssq = (MODE == MODE_PREP ? b * nwaves : 0) * 16 + ml;
      if (m < a.M && n < half) {
        way_kind = 1;
        if (a.y_pack8) {
          // the four columns are four neighbouring k of the reader's lane (the host has checked the widths)
          const int S = a.y_pack8, w = n / (64 * S), in_wave = n - w * 64 * S, hf = in_wave / (32 * S), in_half = in_wave - hf * 32 * S;
          way_dst = (bf16_t*)a.y + (((int64_t)w * S + (in_half >> 5)) * 64 + m + 8 * hf + 16 * ((in_half & 31) >> 3)) * 8 + (n & 7);
        } else {
          way_dst = (bf16_t*)a.y + (int64_t)m * a.ldy + n;
        }
      }
    }
    asm volatile("" : "+v"(way_kind), "+v"(way_part), "+v"(way_ssq), "+v"(way_dst), "+v"(inv_k));
    __builtin_amdgcn_sched_barrier(0);
  }

  // ---- EPI_NEXT with whole columns and at most one item a thread: likewise (way_dst the new residual's place,
  // way_op the next operand's, way_sq the place of the tile's share of the row's squares)
  bf16_t* way_op = nullptr;
  float* way_sq = nullptr;
  if constexpr (NEXT) {
    if (next_early && (int)threadIdx.x < NEXT_ITEMS) {
      const int tile = threadIdx.x / 64, e = threadIdx.x & 63, t = tile / CB, b = tile - t * CB, ml = e >> 2, nl = (e & 3) * 4;
      const int m = b * 16 + ml, n = n0 + t * 16 + nl;
      way_part = (t * CB + b) * 256 + ml * 16 + nl;
      way_ssq = (MODE == MODE_PREP ? b * nwaves : 0) * 16 + ml;
      if (m < a.M) {
        way_kind = n < a.N ? 1 : 2;                     // 2: past the last column, only its zero goes into the row's squares
        way_dst = a.next_res_out + (int64_t)m * a.N + n;
        way_op = a.next_op + (int64_t)m * a.N + n;
        way_sq = a.ssq_out + (int64_t)m * gridDim.x * OT + (int64_t)blockIdx.x * OT + t;
      }
    }
    asm volatile("" : "+v"(way_kind), "+v"(way_part), "+v"(way_ssq), "+v"(way_dst), "+v"(way_op), "+v"(way_sq), "+v"(inv_k));
    __builtin_amdgcn_sched_barrier(0);
  }

  if constexpr (X_TURNED) {
    // a block at a time through this wave's STEPS kilobytes (a wave's LDS operations keep their order)
    uint4* turn = (uint4*)smem + (size_t)wave * STEPS * TS_WAVE;
    const int lr = lane / X_LANES, piece = lane % X_LANES;
#pragma unroll
    for (int b = 0; b < CB; ++b) {
#pragma unroll
      for (int j = 0; j < STEPS; ++j)
        turn[(piece >> 2) * TS_WAVE + sk_place(j * (TS_WAVE / X_LANES) + lr, piece >> 2, piece & 3)] = xall[b][j];
#pragma unroll
      for (int s = 0; s < STEPS; ++s) xall[b][s] = turn[s * TS_WAVE + sk_place(r, s, g)];
    }
    __syncthreads();            // the kilobytes are the waves' partial sums from here on
  }

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
  } else if constexpr (X_FIRST) {
#pragma unroll
    for (int s = 0; s < STEPS; ++s)
#pragma unroll
      for (int t = 0; t < RT; ++t)
#pragma unroll
        for (int b = 0; b < CB; ++b) acc[t][b] = sk_mfma(wreg[t][s], xall[b][s], acc[t][b]);
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
  if constexpr (MODE == MODE_PREP) {
    const int first = (4 * wave + g) * prep_run;
#pragma unroll
    for (int b = 0; b < CB; ++b) {
      float run = 0.f;
      if (prep_early) {
#pragma unroll
        for (int i = 0; i < PREP_VECS; ++i) run += (pv[b][i].x + pv[b][i].y) + (pv[b][i].z + pv[b][i].w);
      } else if (xok[b]) {
        for (int i = first; i < first + prep_run && i < a.ssq_parts; ++i) run += a.ssq_in[(int64_t)(16 * b + r) * a.ssq_parts + i];
      }
      run += __shfl_xor(run, 16, TS_WAVE);
      run += __shfl_xor(run, 32, TS_WAVE);
      if (g == 0) ssq[(b * nwaves + wave) * 16 + r] = run;
    }
  }
  float4 pre_cos = make_float4(1.f, 1.f, 1.f, 1.f), pre_sin = make_float4(0.f, 0.f, 0.f, 0.f);
  if constexpr (ROPE) {
    if (rope_early && way_kind) {
      if (a.rotate && way_kind == 1) {
        const float* cs = a.cos_sin + (int64_t)pre_pos * a.hd + way_d0;
        pre_cos = *(const float4*)cs;
        pre_sin = *(const float4*)(cs + a.hd / 2);
      }
      if (way_head >= a.nh) {                           // a key or a value: its place in the pools, or nowhere
        if (!a.k_cache || pre_slot < 0) way_kind = 0;
        else {
          const int64_t page = pre_slot / a.page_size, off = pre_slot - page * a.page_size;
          way_dst = way_kind == 1 ? a.k_cache + page * a.kp + off * a.ks + (int64_t)(way_head - a.nh) * a.kh + way_d0
                                  : a.v_cache + page * a.vp + off * a.vs + (int64_t)(way_head - a.nh - a.nkv) * a.vh + (int64_t)way_d0 * a.vd;
        }
      }
    }
    asm volatile("" : "+v"(way_kind), "+v"(way_dst));
    __builtin_amdgcn_sched_barrier(0);
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
  if constexpr (NEXT) {
    if (next_early) {                                   // every thread finishes at most one item, and has prepared it
      if ((int)threadIdx.x >= NEXT_ITEMS) return;       // (whole waves: an item's four threads stay together)
      constexpr int WAVE_PARTS = RT * CB * 256;
      float s[4] = {0.f, 0.f, 0.f, 0.f};
      for (int wv = 0; wv < nwaves; ++wv) {
        const float4 ps = *(const float4*)(part + wv * WAVE_PARTS + way_part);
        s[0] += ps.x; s[1] += ps.y; s[2] += ps.z; s[3] += ps.w;
      }
      if (MODE != MODE_PLAIN) {
        float total = 0.f;
        for (int wv = 0; wv < nwaves; ++wv) total += ssq[way_ssq + wv * 16];
        const float inv = __builtin_amdgcn_rsqf(total * inv_k + a.eps);
#pragma unroll
        for (int j = 0; j < 4; ++j) s[j] *= inv;
      }
      // t = T(y) + res; the new residual T(t), the next operand T(t * nw), and the tile's share of the row's sum of t^2
      float sq = 0.f, tv[4], ov[4];
      const uint32_t early_res[2] = {pre_res.x, pre_res.y}, early_nw[2] = {pre_nw.x, pre_nw.y};
#pragma unroll
      for (int j = 0; j < 4; ++j) {                       // (the low half of a word is the even column)
        const float rj = __uint_as_float((early_res[j >> 1] >> (16 * (j & 1))) << 16);
        const float nj = __uint_as_float((early_nw[j >> 1] >> (16 * (j & 1))) << 16);
        const float sum = __uint_as_float(sk_round(s[j]) << 16) + rj;
        tv[j] = sum;
        ov[j] = sum * nj;
        sq = way_kind == 1 ? fmaf(sum, sum, sq) : sq;
      }
      sq += __shfl_xor(sq, 1, TS_WAVE);
      sq += __shfl_xor(sq, 2, TS_WAVE);
      if (way_kind && !(threadIdx.x & 3)) *way_sq = sq;
      if (way_kind == 1) {
        *(uint2*)way_dst = make_uint2(sk_round(tv[0]) | (sk_round(tv[1]) << 16), sk_round(tv[2]) | (sk_round(tv[3]) << 16));
        *(uint2*)way_op = make_uint2(sk_round(ov[0]) | (sk_round(ov[1]) << 16), sk_round(ov[2]) | (sk_round(ov[3]) << 16));
      }
      return;
    }
  }
  if constexpr (GLU && sizeof(OUT) == 2) {
    if (glu_early) {                                    // every thread finishes at most one item, and has prepared it
      if (!way_kind) return;
      constexpr int WAVE_PARTS = RT * CB * 256, PAIR = OT * CB * 256;
      float s[4] = {0.f, 0.f, 0.f, 0.f}, u[4] = {0.f, 0.f, 0.f, 0.f};
      for (int wv = 0; wv < nwaves; ++wv) {
        const float4 ps = *(const float4*)(part + wv * WAVE_PARTS + way_part), pu = *(const float4*)(part + wv * WAVE_PARTS + way_part + PAIR);
        s[0] += ps.x; s[1] += ps.y; s[2] += ps.z; s[3] += ps.w;
        u[0] += pu.x; u[1] += pu.y; u[2] += pu.z; u[3] += pu.w;
      }
      if (MODE != MODE_PLAIN) {
        float total = 0.f;
        for (int wv = 0; wv < nwaves; ++wv) total += ssq[way_ssq + wv * 16];
        const float inv = __builtin_amdgcn_rsqf(total * inv_k + a.eps);
#pragma unroll
        for (int j = 0; j < 4; ++j) { s[j] *= inv; u[j] *= inv; }
      }
      float v[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) v[j] = sk_silu(s[j]) * u[j];
      if (a.y_pack8) *(uint2*)way_dst = make_uint2(sk_round(v[0]) | (sk_round(v[1]) << 16), sk_round(v[2]) | (sk_round(v[3]) << 16));
      else *(uint2*)way_dst = make_uint2(f2bf(v[0]) | ((uint32_t)f2bf(v[1]) << 16), f2bf(v[2]) | ((uint32_t)f2bf(v[3]) << 16));
      return;
    }
  }
  if constexpr (ROPE) {
    if (rope_early) {                                   // every thread finishes at most one item, and has prepared it
      if (!way_kind) return;
      constexpr int WAVE_PARTS = RT * CB * 256;
      float s[4] = {0.f, 0.f, 0.f, 0.f}, u[4] = {0.f, 0.f, 0.f, 0.f};
      for (int wv = 0; wv < nwaves; ++wv) {
        const float4 ps = *(const float4*)(part + wv * WAVE_PARTS + way_part), pu = *(const float4*)(part + wv * WAVE_PARTS + way_part + 8);
        s[0] += ps.x; s[1] += ps.y; s[2] += ps.z; s[3] += ps.w;
        u[0] += pu.x; u[1] += pu.y; u[2] += pu.z; u[3] += pu.w;
      }
      if (MODE != MODE_PLAIN) {
        float total = 0.f;
        for (int wv = 0; wv < nwaves; ++wv) total += ssq[way_ssq + wv * 16];
        const float inv = __builtin_amdgcn_rsqf(total * inv_k + a.eps);
#pragma unroll
        for (int j = 0; j < 4; ++j) { s[j] *= inv; u[j] *= inv; }
      }
      float y1[4], y2[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {                       // as the product would be stored
        y1[j] = __uint_as_float(sk_round(s[j]) << 16);
        y2[j] = __uint_as_float(sk_round(u[j]) << 16);
      }
      if (a.rotate && way_kind == 1) {
        const float ce[4] = {pre_cos.x, pre_cos.y, pre_cos.z, pre_cos.w}, se[4] = {pre_sin.x, pre_sin.y, pre_sin.z, pre_sin.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float r1 = y1[j] * ce[j] - y2[j] * se[j], r2 = y2[j] * ce[j] + y1[j] * se[j];
          y1[j] = r1;
          y2[j] = r2;
        }
      }
      const uint2 o1 = make_uint2(sk_round(y1[0]) | (sk_round(y1[1]) << 16), sk_round(y1[2]) | (sk_round(y1[3]) << 16));
      const uint2 o2 = make_uint2(sk_round(y2[0]) | (sk_round(y2[1]) << 16), sk_round(y2[2]) | (sk_round(y2[3]) << 16));
      const int hdh = a.hd / 2;
      if (way_kind == 1) {
        *(uint2*)way_dst = o1;
        *(uint2*)(way_dst + hdh) = o2;
      } else {
        const uint32_t w1[2] = {o1.x, o1.y}, w2[2] = {o2.x, o2.y};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          way_dst[(int64_t)j * a.vd] = (bf16_t)(w1[j >> 1] >> (16 * (j & 1)));
          way_dst[(int64_t)(hdh + j) * a.vd] = (bf16_t)(w2[j >> 1] >> (16 * (j & 1)));
        }
      }
      return;
    }
  }
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
    if (MODE != MODE_PLAIN) {                             // the row's scale, from every wave's squares (MODE_PREP: from the row's total)
      float total = 0.f;
      for (int wv = 0; wv < nwaves; ++wv) total += ssq[((MODE == MODE_PREP ? b : 0) * nwaves + wv) * 16 + ml];
      const float inv = __builtin_amdgcn_rsqf(total * inv_k + a.eps);   // (the hardware's reciprocal square root: within a rounding)
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
      const int slot = a.slots ? a.slots[m] : -1;
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
    if constexpr (NEXT) {
      // t = T(y) + res; the new residual T(t), the next operand T(t * nw), and the tile's share of the row's
      // sum of t^2: the four threads that hold a row's 16 columns of a tile are neighbours in a wave
      float sq = 0.f, tv[4], ov[4];
      const uint32_t early_res[2] = {pre_res.x, pre_res.y}, early_nw[2] = {pre_nw.x, pre_nw.y};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const bool in = n + j < a.N;
        const int64_t at = (int64_t)m * a.N + (in ? n + j : 0);
        // (fetched at the start where that was possible: the low half of a word is the even column)
        const float rj = next_early ? __uint_as_float((early_res[j >> 1] >> (16 * (j & 1))) << 16)
                                    : (a.next_res ? bf2f(a.next_res[at]) : 0.f);
        const float nj = next_early ? __uint_as_float((early_nw[j >> 1] >> (16 * (j & 1))) << 16) : bf2f(a.next_nw[in ? n + j : 0]);
        const float sum = __uint_as_float(sk_round(s[j]) << 16) + rj;
        tv[j] = sum;
        ov[j] = sum * nj;
        sq = in ? fmaf(sum, sum, sq) : sq;
      }
      sq += __shfl_xor(sq, 1, TS_WAVE);
      sq += __shfl_xor(sq, 2, TS_WAVE);
      if (!(e & 3)) a.ssq_out[(int64_t)m * gridDim.x * OT + (int64_t)blockIdx.x * OT + t] = sq;
      if (a.N % 4 == 0 && n + 3 < a.N) {
        *(uint2*)(a.next_res_out + (int64_t)m * a.N + n) = make_uint2(sk_round(tv[0]) | (sk_round(tv[1]) << 16), sk_round(tv[2]) | (sk_round(tv[3]) << 16));
        *(uint2*)(a.next_op + (int64_t)m * a.N + n) = make_uint2(sk_round(ov[0]) | (sk_round(ov[1]) << 16), sk_round(ov[2]) | (sk_round(ov[3]) << 16));
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j)
          if (n + j < a.N) {
            a.next_res_out[(int64_t)m * a.N + n + j] = (bf16_t)sk_round(tv[j]);
            a.next_op[(int64_t)m * a.N + n + j] = (bf16_t)sk_round(ov[j]);
          }
      }
      continue;
    }
    if constexpr (GLU && sizeof(OUT) == 2) {
      if (a.y_pack8) {
        // the four columns are four neighbouring k of the reader's lane (the host has checked the widths)
        const int S = a.y_pack8, w = n / (64 * S), in_wave = n - w * 64 * S, hf = in_wave / (32 * S), in_half = in_wave - hf * 32 * S;
        bf16_t* dst = (bf16_t*)a.y + (((int64_t)w * S + (in_half >> 5)) * 64 + m + 8 * hf + 16 * ((in_half & 31) >> 3)) * 8 + (n & 7);
        float v[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] = sk_silu(s[j]) * u[j];
        *(uint2*)dst = make_uint2(sk_round(v[0]) | (sk_round(v[1]) << 16), sk_round(v[2]) | (sk_round(v[3]) << 16));
        continue;
      }
    }
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (n + j < ncols) Num<OUT>::st(y + (int64_t)m * a.ldy + n + j, GLU ? sk_silu(s[j]) * u[j] : s[j]);
  }
}

// The LDS a workgroup may ask for on the current device (asked of the runtime once per device).
static size_t sk_lds_limit() {
  static int limit[16] = {0};
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 16) return 65536;
  if (!limit[device]) {
    int v = 0;
    if (hipDeviceGetAttribute(&v, hipDeviceAttributeMaxSharedMemoryPerBlock, device) != hipSuccess || v <= 0) v = 65536;
    limit[device] = v;
  }
  return (size_t)limit[device];
}

template <int RT, int CB, int STEPS, int MODE, int GLU, typename OUT>
static int sk_launch(const SkinnyArgs& a, hipStream_t stream) {
  const int nwaves = a.K / (STEPS * SK_KSTEP);
  size_t smem = sizeof(float) * ((size_t)nwaves * RT * CB * 256 + (size_t)nwaves * 16 * CB);
  // (the kilobytes through which a wave turns its rows of x, where it does: X_TURNED of the kernel)
  if (CB >= 2 && CB >= RT && MODE != MODE_NORM && nwaves <= 8 && (CB * STEPS + RT * STEPS) <= 48 && smem < (size_t)nwaves * STEPS * 1024)
    smem = (size_t)nwaves * STEPS * 1024;
  constexpr int OT = GLU == EPI_GLU ? RT / 2 : RT;
  const int ncols = GLU == EPI_GLU ? a.N / 2 : a.N;     // (EPI_ROPE: a 16-row tile of the matrix per 8 columns and their partners)
  if (smem > sk_lds_limit()) return TS_BAD_SHAPE;       // (the largest instances ask for a little more than 64 KB)
  dim3 grid((ncols + 16 * OT - 1) / (16 * OT)), block(nwaves * TS_WAVE);
  if (nwaves <= 8) {
    gemm_skinny_kernel<RT, CB, STEPS, MODE, GLU, 512, OUT><<<grid, block, smem, stream>>>(a);
  } else {
    // a workgroup of 16 waves has 128 registers a lane: one or two row tiles, and no fused norm
    if constexpr (MODE != MODE_NORM && (RT == 1 || (RT == 2 && CB == 1)))
      gemm_skinny_kernel<RT, CB, STEPS, MODE, GLU, 1024, OUT><<<grid, block, smem, stream>>>(a);
    else return TS_BAD_SHAPE;
  }
  return ts_check_launch();
}

// Picks the instance: slices of 256 k while that needs at most 16 waves, else slices of 512; more
// rows of W per workgroup for wide matrices once that still leaves a workgroup per compute unit
// (fewer workgroups repeat less of the work on x).
#ifndef SK_GLU_SMALL_ROWS
#define SK_GLU_SMALL_ROWS 4
#endif
template <int MODE, int EPI, typename OUT>
static int sk_dispatch(const SkinnyArgs& a, hipStream_t stream) {
  constexpr bool GLU = EPI == EPI_GLU, NORM = MODE == MODE_NORM;
  const int steps = (a.K % 256 == 0 && a.K / 256 <= 16) ? 8 : 16;
  if (a.K % (steps * SK_KSTEP) || a.K / (steps * SK_KSTEP) > 16) return TS_BAD_SHAPE;
  const int nwaves = a.K / (steps * SK_KSTEP);
  const int cb = (a.M + 15) / 16;
  if (NORM && cb != 1) return TS_BAD_SHAPE;
  const int ncols = GLU ? a.N / 2 : a.N;
#define SK_GO(RT, CB, ST) return sk_launch<RT, CB, ST, MODE, EPI, OUT>(a, stream)
  if constexpr (NORM || GLU) {
    // the instances that hold x + res or four row tiles need the registers of a workgroup of 8 waves
    if (steps != 8) return TS_BAD_SHAPE;
    if constexpr (!NORM && GLU) {
      // the gate for 17 to 64 rows of x: two or four blocks of rows against the same registers of W
      if (cb > 1 && nwaves > 8) return TS_BAD_SHAPE;
      if (cb == 2) { if (ncols >= 4096) SK_GO(4, 2, 8); else SK_GO(2, 2, 8); }
      if (cb > 2) SK_GO(2, 4, 8);
    }
    if (nwaves <= 8) {
      // (the gate for up to four rows of x: 512 workgroups of two row tiles stream faster than 256 of four, which
      //  repeat less of the work on x with more rows: a decode step at batch 1 0.747 -> 0.741 ms, at batch 4
      //  0.819 -> 0.816, at batch 6 0.837 -> 0.840)
      if (ncols >= 4096 * (GLU ? (a.M <= SK_GLU_SMALL_ROWS ? 4 : 1) : 2)) SK_GO(4, 1, 8);
      if (GLU || ncols >= 4096) SK_GO(2, 1, 8);
    }
    if constexpr (!GLU) SK_GO(1, 1, 8);
    if constexpr (!NORM) SK_GO(2, 1, 8);                // the gate alone, in a workgroup of up to 16 waves
    return TS_BAD_SHAPE;
  } else {
    if (cb > 2) {                                       // 33 to 64 rows of x: reductions of up to 2048 in 8 waves
      if (steps == 8 && nwaves <= 8) SK_GO(1, 4, 8);
      return TS_BAD_SHAPE;
    }
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
#define SK_COMB_CHUNKS 16     // most chunks that the instance which makes its x from an attention's parts adds up
// The operands of that instance, out of the fields they travel in.
struct SkinnyParts {
  const float* o;            // [K / hd heads, splits, hd]: the chunks' weighted values            (SkinnyArgs::x)
  const float* ml;           // [heads, splits, 2]: a chunk's running maximum (log2 units) and sum   (ssq_in)
  const int32_t* pos;        // [1]: the token's position                                            (positions)
  int splits, chunk, window, hd;   //                                                                (nh, nkv, rotate, hd)
  __device__ __host__ SkinnyParts(const SkinnyArgs& a)
      : o((const float*)a.x), ml(a.ssq_in), pos(a.positions), splits(a.nh), chunk(a.nkv), window(a.rotate), hd(a.hd) {}
};
template <int STEPS, int MAXT, typename OUT, bool NEXT = false, bool COMB = false>
__global__ void __launch_bounds__(MAXT)
gemm_skinny8_kernel(const SkinnyArgs a) {
  static_assert(!COMB || (STEPS == 4 && MAXT <= 512 && sizeof(OUT) == 2), "x from parts: a wave's 256 k of one token fit its kilobyte of LDS");
  ts_fetch_arguments<sizeof(SkinnyArgs)>();
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
  // rows past M repeat row 0 (in the packed order: hold anything) and are not stored
  const bf16_t* xrow = a.x_packed8 ? a.x + ((int64_t)wave * STEPS * 64 + lane) * 8 : a.x + (int64_t)(row < a.M ? row : 0) * a.ldx + kbeg;
  const int xstep = a.x_packed8 ? 512 : SK_KSTEP;       // from a step's piece to the next step's
  uint4 xb[XB];
  // COMB: lane l makes the wave's k 4 l .. 4 l + 3 (they lie in one head). Every chunk's maximum, sum and four
  // values are asked for here, ahead of W (a chunk that holds nothing the token sees reads the last that does, and
  // counts with weight zero); they are added up once W's loads are out.
  float2 c_ml[COMB ? SK_COMB_CHUNKS : 1];
  float4 c_po[COMB ? SK_COMB_CHUNKS : 1];
  int c_s0 = 0, c_s1 = 0;
  if constexpr (COMB) {
    const SkinnyParts parts(a);
    const int pos = parts.pos[0];
    const int lo = (parts.window > 0 && pos - parts.window + 1 > 0) ? pos - parts.window + 1 : 0;
    c_s0 = min(lo / parts.chunk, parts.splits - 1);
    c_s1 = min(pos / parts.chunk, parts.splits - 1);
    const int k4 = wave * (2 * STEPS * SK_KSTEP) + 4 * lane, head = k4 / parts.hd, d = k4 - head * parts.hd;
    const float* ml = parts.ml + (int64_t)head * parts.splits * 2;
    const float* po = parts.o + (int64_t)head * parts.splits * parts.hd + d;
#pragma unroll
    for (int i = 0; i < SK_COMB_CHUNKS; ++i) {
      const int c = c_s0 + i <= c_s1 ? c_s0 + i : c_s1;
      c_ml[i] = *(const float2*)(ml + 2 * c);
      c_po[i] = *(const float4*)(po + (int64_t)c * parts.hd);
    }
    __builtin_amdgcn_sched_barrier(0);
  } else if (X_FIRST) {
#pragma unroll
    for (int s = 0; s < STEPS; ++s) xb[s] = *(const uint4*)(xrow + s * xstep);
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
  // EPI_NEXT: the residual and the next norm's weight of the element this thread will finish, asked for right behind W
  // (and where its results go is worked out here, while W is on its way: after the waves' meeting every instruction is waited for)
  bf16_t pre_res = 0, pre_nw = 0;
  bf16_t *way_res = nullptr, *way_op = nullptr;
  float* way_sq = nullptr;
  int way_pair = 0;                                     // 1: this thread stores its column and the next as one word; 2: singly
  if constexpr (NEXT) {
    const int m = threadIdx.x >> 3, n = n0 + (threadIdx.x & 7);
    if (threadIdx.x < 64 && m < a.M && n < a.N) {
      pre_nw = a.next_nw[n];
      if (a.next_res) pre_res = a.next_res[(int64_t)m * a.N + n];
    }
    if (threadIdx.x < 64 && m < a.M) {
      way_res = a.next_res_out + (int64_t)m * a.N + n;
      way_op = a.next_op + (int64_t)m * a.N + n;
      way_sq = a.ssq_out + (int64_t)m * gridDim.x + blockIdx.x;
      if (!(threadIdx.x & 1)) way_pair = n + 1 < a.N && !((((uintptr_t)way_res) | ((uintptr_t)way_op)) & 3) ? 1 : 2;
    }
    asm volatile("" : "+v"(way_res), "+v"(way_op), "+v"(way_sq), "+v"(way_pair));
    __builtin_amdgcn_sched_barrier(0);
  }
  if constexpr (COMB) {
    float top = -INFINITY;
#pragma unroll
    for (int i = 0; i < SK_COMB_CHUNKS; ++i) top = c_s0 + i <= c_s1 ? fmaxf(top, c_ml[i].x) : top;
    // the chunks' sums as the combining kernel's wave adds them: chunk s0 + i in lane i, lanes 8, 4, 2 and 1 apart in turn
    float sum[SK_COMB_CHUNKS], v[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < SK_COMB_CHUNKS; ++i) {
      const bool has = c_s0 + i <= c_s1;
      const float w = has ? __builtin_amdgcn_exp2f(c_ml[i].x - top) : 0.f;
      sum[i] = has ? c_ml[i].y * w : 0.f;
      v[0] = has ? fmaf(c_po[i].x, w, v[0]) : v[0];
      v[1] = has ? fmaf(c_po[i].y, w, v[1]) : v[1];
      v[2] = has ? fmaf(c_po[i].z, w, v[2]) : v[2];
      v[3] = has ? fmaf(c_po[i].w, w, v[3]) : v[3];
    }
#pragma unroll
    for (int step = SK_COMB_CHUNKS / 2; step >= 1; step >>= 1)
#pragma unroll
      for (int i = 0; i < step; ++i) sum[i] += sum[i + step];
    const float inv = 1.0f / sum[0];
    // through this wave's kilobyte of LDS into operand order (a wave's LDS operations keep their order; the kilobyte
    // is the wave's partial sums afterwards)
    bf16_t* turn = (bf16_t*)(smem + wave * 256);
    *(uint2*)(turn + 4 * lane) = make_uint2(f2bf(v[0] * inv) | ((uint32_t)f2bf(v[1] * inv) << 16), f2bf(v[2] * inv) | ((uint32_t)f2bf(v[3] * inv) << 16));
#pragma unroll
    for (int s = 0; s < STEPS; ++s)
      xb[s] = row == 0 ? *(const uint4*)(turn + half * (STEPS * SK_KSTEP) + s * SK_KSTEP + 8 * g) : make_uint4(0, 0, 0, 0);
  }
  float4_t acc = {0.f, 0.f, 0.f, 0.f};
  if (X_FIRST) {
#pragma unroll
    for (int s = 0; s < STEPS; ++s) acc = sk_mfma(wreg[s], xb[s], acc);
  } else {
#pragma unroll
    for (int s0 = 0; s0 < STEPS; s0 += XB) {
#pragma unroll
      for (int s = 0; s < XB; ++s) xb[s] = *(const uint4*)(xrow + (s0 + s) * xstep);
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
  if constexpr (NEXT) {
    // EPI_NEXT (see the top of the file): the eight threads of a row hold the tile's eight columns
    const bool in = m < a.M && n < a.N;
    const float t = __uint_as_float(sk_round(sum) << 16) + bf2f(pre_res);
    float sq = in ? t * t : 0.f;
    sq += __shfl_xor(sq, 1, TS_WAVE);
    sq += __shfl_xor(sq, 2, TS_WAVE);
    sq += __shfl_xor(sq, 4, TS_WAVE);
    if (nl == 0 && m < a.M) *way_sq = sq;
    const uint32_t res_mine = sk_round(t), op_mine = sk_round(t * bf2f(pre_nw));
    const uint32_t res_next = __shfl_down(res_mine, 1, TS_WAVE), op_next = __shfl_down(op_mine, 1, TS_WAVE);
    if (way_pair == 1) {
      *(uint32_t*)way_res = res_mine | (res_next << 16);
      *(uint32_t*)way_op = op_mine | (op_next << 16);
    } else if (way_pair == 2) {
      if (n < a.N) { way_res[0] = (bf16_t)res_mine; way_op[0] = (bf16_t)op_mine; }
      if (n + 1 < a.N) { way_res[1] = (bf16_t)res_next; way_op[1] = (bf16_t)op_next; }
    }
  } else if constexpr (sizeof(OUT) == 4) {
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

template <typename OUT, bool NEXT = false>
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
  if (a.x_packed8 == 2) {
    if constexpr (sizeof(OUT) == 2) {
      if (steps != 4 || nwaves > 8 || a.M != 1 || SkinnyParts(a).splits > SK_COMB_CHUNKS) return TS_BAD_SHAPE;
      gemm_skinny8_kernel<4, 512, OUT, NEXT, true><<<grid, block, smem, stream>>>(a);
      return ts_check_launch();
    } else {
      return TS_BAD_SHAPE;
    }
  }
  if (steps == 4) gemm_skinny8_kernel<4, 512, OUT, NEXT><<<grid, block, smem, stream>>>(a);
  else if (steps == 8) gemm_skinny8_kernel<8, 512, OUT, NEXT><<<grid, block, smem, stream>>>(a);
  else if (nwaves <= 8) gemm_skinny8_kernel<16, 512, OUT, NEXT><<<grid, block, smem, stream>>>(a);
  else gemm_skinny8_kernel<16, 1024, OUT, NEXT><<<grid, block, smem, stream>>>(a);
  return ts_check_launch();
}

// The operands of EPI_NEXT, checked: the next norm's weight [N], the outputs [M, N] dense (the new residual
// and the next operand) and [M, parts] (sums of squares), an optional residual [M, N].
static bool sk_next_ok(const void* next_res, const void* next_nw, const void* next_res_out, const void* next_op,
                       const void* ssq_out) {
  if (!next_nw || !next_res_out || !next_op || !ssq_out) return false;
  return !((((uintptr_t)next_res) | ((uintptr_t)next_nw) | ((uintptr_t)next_res_out) | ((uintptr_t)next_op)) & 1) &&
         !(((uintptr_t)ssq_out) & 3);
}

// y [M <= 8, N] = x · W^T by the 8-row form above: K a multiple of 256 up to 8,192 or of 1,024 up to
// 16,384; contiguous 16-byte aligned rows. out_dtype: 1 bfloat16, 0 float. packed: w is
// hip.pack_weight8(W) for this K, ldw unused, N a multiple of 8. With next_nw (EPI_NEXT; bfloat16 only)
// y is not written: next_res_out, next_op [M, N] and ssq_out [M, (N + 7) / 8] are. x_packed8: x is given in
// the order the lanes read it (SkinnyArgs::x_packed8; K / 8 16-byte pieces of 64 lanes, whatever M), ldx unused.
// comb_o (x null, M = 1, bfloat16 out, K a multiple of 256 up to 2,048): x is made on the way in from the split-key
// attention kernel's parts (SkinnyParts; comb_hd a multiple of 32 that divides K, up to 16 chunks).
extern "C" int ts_gemm_skinny8_bf16(void* y, const void* x, const void* w, int M, int N, int K, int64_t ldx, int64_t ldw,
                                    int64_t ldy, int out_dtype, int packed, const void* next_res, const void* next_nw,
                                    void* next_res_out, void* next_op, void* ssq_out, int x_packed8, const float* comb_o,
                                    const float* comb_ml, const int32_t* comb_pos, int comb_splits, int comb_chunk,
                                    int comb_window, int comb_hd, hipStream_t stream) {
  if (M <= 0 || N <= 0) return TS_OK;
  if (comb_o) {
    if (x || x_packed8 || M != 1 || out_dtype != 1 || !comb_ml || !comb_pos || comb_splits < 1 || comb_splits > SK_COMB_CHUNKS ||
        comb_chunk <= 0 || comb_hd <= 0 || comb_hd % 32 || K % comb_hd || K % 256 || K > 2048 ||
        ((((uintptr_t)comb_o) | ((uintptr_t)comb_ml)) & 15))
      return TS_BAD_SHAPE;
    ldx = K;
  }
  if (M > 8 || K <= 0 || (!x_packed8 && (ldx % 8 || ldx < K)) || (!packed && (ldw % 8 || ldw < K)) || (packed && N % 8)) return TS_BAD_SHAPE;
  if (((uintptr_t)x | (uintptr_t)w) & 15) return TS_BAD_SHAPE;
  SkinnyArgs a = {};
  a.x = (const bf16_t*)x; a.w = (const bf16_t*)w; a.y = y; a.M = M; a.N = N; a.K = K; a.ldx = ldx; a.ldw = ldw; a.ldy = ldy;
  a.packed = packed;
  a.x_packed8 = x_packed8 != 0;
  if (comb_o) {                                         // (see SkinnyParts)
    a.x_packed8 = 2;
    a.x = (const bf16_t*)comb_o; a.ssq_in = comb_ml; a.positions = comb_pos;
    a.nh = comb_splits; a.nkv = comb_chunk; a.rotate = comb_window; a.hd = comb_hd;
  }
  if (next_nw) {
    if (out_dtype != 1 || !sk_next_ok(next_res, next_nw, next_res_out, next_op, ssq_out)) return TS_BAD_SHAPE;
    a.next_res = (const bf16_t*)next_res; a.next_nw = (const bf16_t*)next_nw; a.next_res_out = (bf16_t*)next_res_out;
    a.next_op = (bf16_t*)next_op; a.ssq_out = (float*)ssq_out;
    return sk8_dispatch<bf16_t, true>(a, stream);
  }
  if (!y || ldy < N) return TS_BAD_SHAPE;
  if (out_dtype == 1) return sk8_dispatch<bf16_t>(a, stream);
  if (out_dtype == 0) return sk8_dispatch<float>(a, stream);
  return TS_BAD_DTYPE;
}

// mode: 0 plain, 1 residual + RMSNorm on the way in (M <= 16, K in steps of 256 up to 2048), 2 the norm
// prepared by the kernel before (x is the operand as it stands; ssq_in [M, ssq_parts] the parts of the rows'
// sums of squares; eps). glu: W holds gate rows then up rows, y is [M, N / 2] = silu(gate) * up (M <= 16,
// K up to 4096, 2048 with the norm; without the norm of mode 1 M <= 64 for K up to 2048). out_dtype: 1 bfloat16,
// 0 float (plain only). packed: w holds the matrix in the kernel's own order (see the loads of W), ldw is
// unused. Requires M <= 32 (M <= 64 for K up to 2048 in 8 waves), K a multiple of 256 (up to 4096) or of 512
// (up to 8192), contiguous 16-byte aligned rows; mode 1 takes x, res, res_out as dense [M, K].
// With next_nw (EPI_NEXT; modes 0 and 2 without glu, bfloat16) y is not written: next_res_out, next_op
// [M, N] and ssq_out [M, tiles] are, tiles being the 16-column tiles the grid covers (ts_skinny_tiles).
// y_pack8 > 0 (glu, bfloat16, M <= 8, N / 2 a multiple of 64 y_pack8): y is not [M, N / 2] but the gated product in
// the order the 8-row form of y_pack8 steps reads its x (SkinnyArgs::x_packed8): N / 2 / 8 pieces of 64 lanes.
extern "C" int ts_gemm_skinny_bf16(void* y, const void* x, const void* w, const void* res, const void* nw,
                                   void* res_out, int M, int N, int K, int64_t ldx, int64_t ldw, int64_t ldy,
                                   float eps, int mode, int glu, int out_dtype, int packed, const void* ssq_in,
                                   int ssq_parts, const void* next_res, const void* next_nw, void* next_res_out,
                                   void* next_op, void* ssq_out, int y_pack8, hipStream_t stream) {
  if (M <= 0 || N <= 0) return TS_OK;
  // the gated product for the 8-row form: up to 8 rows, bfloat16, whole waves of the reader (64 y_pack8 of k each)
  if (y_pack8 && (!glu || out_dtype != 1 || M > 8 || (y_pack8 != 4 && y_pack8 != 8 && y_pack8 != 16) || (N / 2) % (64 * y_pack8))) return TS_BAD_SHAPE;
  const bool wide = mode != MODE_NORM && K <= 2048 && K % 256 == 0;        // 33 to 64 rows: see sk_dispatch
  if (M > (wide ? 64 : 32) || K <= 0 || ldx % 8 || ldw % 8 || ldx < K || ldw < K) return TS_BAD_SHAPE;
  if (glu && (N % 2 || (N / 2) % 16)) return TS_BAD_SHAPE;
  if (((uintptr_t)x | (uintptr_t)w | (uintptr_t)res | (uintptr_t)nw | (uintptr_t)res_out) & 15) return TS_BAD_SHAPE;
  if (mode == MODE_NORM && (!nw || (res && !res_out))) return TS_BAD_SHAPE;
  if (mode == MODE_PREP && (!ssq_in || ssq_parts <= 0 || (((uintptr_t)ssq_in) & 3))) return TS_BAD_SHAPE;
  SkinnyArgs a = {};
  a.x = (const bf16_t*)x; a.res = (const bf16_t*)res; a.nw = (const bf16_t*)nw; a.res_out = (bf16_t*)res_out;
  a.w = (const bf16_t*)w; a.y = y; a.M = M; a.N = N; a.K = K; a.ldx = ldx; a.ldw = ldw; a.ldy = ldy; a.eps = eps; a.packed = packed;
  a.ssq_in = (const float*)ssq_in; a.ssq_parts = ssq_parts;
  a.y_pack8 = y_pack8;
  if (next_nw) {
    if (glu || out_dtype != 1 || mode == MODE_NORM || !sk_next_ok(next_res, next_nw, next_res_out, next_op, ssq_out)) return TS_BAD_SHAPE;
    a.next_res = (const bf16_t*)next_res; a.next_nw = (const bf16_t*)next_nw; a.next_res_out = (bf16_t*)next_res_out;
    a.next_op = (bf16_t*)next_op; a.ssq_out = (float*)ssq_out;
    if (mode == MODE_PLAIN) return sk_dispatch<MODE_PLAIN, EPI_NEXT, bf16_t>(a, stream);
    return sk_dispatch<MODE_PREP, EPI_NEXT, bf16_t>(a, stream);
  }
  if (!y || ldy < (glu ? N / 2 : N)) return TS_BAD_SHAPE;
  if (out_dtype == 1) {
    if (mode == MODE_PLAIN && !glu) return sk_dispatch<MODE_PLAIN, EPI_NONE, bf16_t>(a, stream);
    if (mode == MODE_PLAIN && glu) return sk_dispatch<MODE_PLAIN, EPI_GLU, bf16_t>(a, stream);
    if (mode == MODE_NORM && !glu) return sk_dispatch<MODE_NORM, EPI_NONE, bf16_t>(a, stream);
    if (mode == MODE_NORM && glu) return sk_dispatch<MODE_NORM, EPI_GLU, bf16_t>(a, stream);
    if (mode == MODE_PREP && !glu) return sk_dispatch<MODE_PREP, EPI_NONE, bf16_t>(a, stream);
    if (mode == MODE_PREP && glu) return sk_dispatch<MODE_PREP, EPI_GLU, bf16_t>(a, stream);
    return TS_BAD_SHAPE;
  }
  if (out_dtype == 0 && mode == MODE_PLAIN && !glu) return sk_dispatch<MODE_PLAIN, EPI_NONE, float>(a, stream);
  return TS_BAD_DTYPE;
}

// The 16-column tiles that ts_gemm_skinny_bf16's grid covers for a matrix of N rows over K with M rows of x: the
// second dimension of ssq_out. (The workgroups own one, two or four tiles; the last may reach past N.)
extern "C" int ts_skinny_tiles(int M, int N, int K) {
  const int steps = (K % 256 == 0 && K / 256 <= 16) ? 8 : 16;
  const int nwaves = K / (steps * SK_KSTEP), cb = (M + 15) / 16;
  const int rt = (cb <= 2 && N >= 8192 && (nwaves <= 8 || cb == 1) && steps == 8) ? 2 : 1;
  return (N + 16 * rt - 1) / (16 * rt) * rt;
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
                                        int64_t vh, int64_t vd, const void* ssq_in, int ssq_parts, hipStream_t stream) {
  if (M <= 0) return TS_OK;
  if (mode == MODE_PREP && (!ssq_in || ssq_parts <= 0 || (((uintptr_t)ssq_in) & 3))) return TS_BAD_SHAPE;
  if (M > (mode != MODE_NORM && K <= 2048 ? 64 : 16) || K <= 0 || K % 256 || K / 256 > (mode == MODE_NORM ? 8 : 16) || ldx % 8 || ldw % 8 || ldx < K || ldw < K) return TS_BAD_SHAPE;
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
  a.table_vec = !(((uintptr_t)cos_sin) & 15);
  a.page_size = page_size; a.kp = kp; a.ks = ks; a.kh = kh; a.vp = vp; a.vs = vs; a.vh = vh; a.vd = vd;
  a.ssq_in = (const float*)ssq_in; a.ssq_parts = ssq_parts;
  if (mode == MODE_PREP && M > 32) return sk_launch<1, 4, 8, MODE_PREP, EPI_ROPE, bf16_t>(a, stream);
  if (mode == MODE_PREP && M > 16) return sk_launch<1, 2, 8, MODE_PREP, EPI_ROPE, bf16_t>(a, stream);
  if (mode == MODE_PREP) return sk_launch<1, 1, 8, MODE_PREP, EPI_ROPE, bf16_t>(a, stream);
  if (mode == MODE_PLAIN && M > 32) return sk_launch<1, 4, 8, MODE_PLAIN, EPI_ROPE, bf16_t>(a, stream);
  if (mode == MODE_PLAIN && M > 16) return sk_launch<1, 2, 8, MODE_PLAIN, EPI_ROPE, bf16_t>(a, stream);
  if (mode == MODE_PLAIN) return sk_launch<1, 1, 8, MODE_PLAIN, EPI_ROPE, bf16_t>(a, stream);
  if (mode == MODE_NORM) return sk_launch<1, 1, 8, MODE_NORM, EPI_ROPE, bf16_t>(a, stream);
  return TS_BAD_SHAPE;
}
