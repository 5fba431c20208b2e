// y[M, N] = e(f(x)[M, K] · W[N, K]^T) in bfloat16 for 17 to 128 rows of x and a wide W (the gate|up
// projection of a decode step of a few dozen requests), where time should go to reading W once.
//
// With so many rows the weight-streaming kernel of gemm_skinny.hip reads x from the second-level cache
// once per 32 rows of W, which is twice the bytes of W itself. Here a workgroup owns 64 rows of W and
// splits the work between two kinds of wave:
//   four compute waves, one 16-row tile of W each over the whole of K: the tile streams from memory
//   straight into MFMA operands, 16 steps of 32 k under way at any time (a step's register is asked for
//   again as soon as it has been used), and the four 16-row blocks of x come out of LDS;
//   four staging waves, which bring x into LDS in chunks of 256 k, one chunk ahead of the compute waves
//   (two buffers, a barrier per chunk). A staging wave takes a block of 16 rows, and each of its loads
//   512 contiguous bytes of two rows (an instruction that gathered 64 bytes of each of 16 rows, the
//   order in which the matrix instruction wants them, cost the gate|up product of 64 rows 1.7 of 20 us
//   and 7.5 of 62 at the 8B widths); the pieces go into LDS where the compute lanes look for them, with
//   the place inside a block of 16 rows turned by the piece's step and part of k so that neither the
//   writes nor the reads meet in a bank. Their loads hit the cache; in waves of their own they do not
//   queue behind the loads of W (a wave's loads come back in the order it asked).
// The gate can ride along as in gemm_skinny.hip:
//   GLU   W = [gate rows | up rows]: waves 0 and 1 take two gate tiles, waves 2 and 3 the up tiles
//         N / 2 rows below them, and y [M, N / 2] = silu(gate) * up
// (The norm on the way in, which every workgroup would have to repeat for all of x, was tried in the
// staging waves and costs more than the norm kernel it saves: 37 µs against 21 + 7 at 64 rows.)
// W comes as the 16-row packed copy ([N / 16 tiles][K / 32 steps][64 lanes][8]); K is a multiple of
// 1,024. A row of x meets W's k in ascending order in one accumulator, whatever the other rows are.
//
// A narrow W (the o and down projections: 2,048 to 4,096 rows) has too few 64-row tiles to give every
// compute unit a workgroup, so its reduction may be cut into slices (the grid's second dimension): the
// workgroup of slice s multiplies k = s K / slices .. (s + 1) K / slices and leaves its 32-bit sums in
// part s of y [slices][M][N]. rows64_finish_kernel then adds a column's parts in ascending order
// (always the same order: the result does not depend on which workgroup finished first) and either
// stores the product or finishes it into the residual sum and the norm that follow it, as EPI_NEXT of
// gemm_skinny.hip does: the new residual, the next projection's operand and the rows' sums of squares
// (whole: a workgroup of that kernel takes a row).
#include <type_traits>
#include "skinny_ops.h"

#define R64_CHUNK_STEPS 8         // 32-wide k steps per chunk of x in LDS
#define R64_RING 16               // steps of W a compute wave has under way (two chunks): with 32 the chip had 32 MB under way and
                                  // every load, x's among them, came back some 5 us later (the gate|up product of 64 rows 20.7 us, 19.7 with 16)
#define R64_STAGE_LOADS 8          // loads of a staging wave per chunk: two rows of its block each

struct Rows64Args {
  const bf16_t* x;       // [M, K], row stride ldx
  const bf16_t* w16;     // W [N, K], packed
  void* y;               // [M, N] (GLU: [M, N / 2]), row stride ldy
  int M, N, K;
  int64_t ldx, ldy;
  // the norm on the way in, prepared by the kernel that made x (see MODE_PREP in gemm_skinny.hip): x is
  // the operand as it stands and a row's scale rsqrt(sum of its ssq_parts parts / K + eps) multiplies
  // its finished sums; null: no scale
  const float* ssq_in;
  int ssq_parts;
  float eps;
  int slices;            // the reduction in this many slices (gridDim.y); more than one: y is float [slices][M][ldy]
};

// BLOCKS: blocks of 16 rows of x, 4 (up to 64 rows) or 8 (up to 128: the compute waves then take a chunk's
// steps one at a time instead of in pairs, for their registers' sake).
template <bool GLU, typename OUT, int BLOCKS>
__global__ void __launch_bounds__(512) gemm_rows64_kernel(const Rows64Args a) {
  // x as the B operands of the matrix instruction: [buffer][step][block of 16 rows][lane], lane r + 16 g
  // holding k = 8 g .. 8 g + 7 of row r (turned: sk_place)
  extern __shared__ __align__(16) uint4 xs_all[];
  auto xs = [&](int buf, int step, int b) { return xs_all + (((size_t)buf * R64_CHUNK_STEPS + step) * BLOCKS + b) * TS_WAVE; };
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / TS_WAVE), lane = threadIdx.x & (TS_WAVE - 1);
  const int r = lane & 15, g = lane >> 4;
  const int slice = blockIdx.y;
  const int nsteps = a.K / SK_KSTEP / a.slices, nchunks = nsteps / R64_CHUNK_STEPS;   // (steps: a multiple of the ring, chunks: even)
  const int64_t kfirst = (int64_t)slice * nsteps * SK_KSTEP;                  // the slice's first k

  if (wave >= 4) {
    // ---- staging waves: wave sw brings block sw of 16 rows, all the steps of every chunk. It asks for
    // the next chunk before it puts this one into LDS, so that a chunk costs the compute waves a barrier
    // and not a trip to the cache.
    const int sw = wave - 4;                              // this wave's blocks of 16 rows: sw BLOCKS / 4 ..
    constexpr int MINE = BLOCKS / 4, LOADS = R64_STAGE_LOADS * MINE;
    const int half = lane >> 5, kl = lane & 31;           // the row of a load's two, and the piece of its 256 k
    bool ok[LOADS];
    int64_t xoff[LOADS];
    int slot[LOADS];
#pragma unroll
    for (int j = 0; j < LOADS; ++j) {
      const int block = sw * MINE + j / R64_STAGE_LOADS, r = 2 * (j % R64_STAGE_LOADS) + half, m = 16 * block + r;
      ok[j] = m < a.M;                                    // rows past M read row 0 and count as zeros
      xoff[j] = (int64_t)(ok[j] ? m : 0) * a.ldx + kfirst + 8 * kl;
      slot[j] = ((kl >> 2) * BLOCKS + block) * TS_WAVE + sk_place(r, kl >> 2, kl & 3);      // in a buffer's [step][block][64]
    }
    auto ask = [&](int c, uint4 (&t)[LOADS]) {
      const int k0 = c * R64_CHUNK_STEPS * SK_KSTEP;      // first k of the chunk
#pragma unroll
      for (int j = 0; j < LOADS; ++j) t[j] = *(const uint4*)(a.x + xoff[j] + k0);
    };
    auto put = [&](int c, const uint4 (&t)[LOADS]) {
      uint4* buf = xs(c & 1, 0, 0);
#pragma unroll
      for (int j = 0; j < LOADS; ++j) buf[slot[j]] = ok[j] ? t[j] : make_uint4(0, 0, 0, 0);
    };
    uint4 A[LOADS], B[LOADS];
    ask(0, A);
    for (int c = 0; c < nchunks; c += 2) {
      ask(c + 1, B);
      put(c, A);
      __syncthreads();          // chunk c is there (and chunk c - 1 has been used: its buffer is the next one's)
      ask(min(c + 2, nchunks - 1), A);   // (past the end: the last chunk again, and nobody uses it)
      put(c + 1, B);
      __syncthreads();
    }
    __syncthreads();            // the compute waves' last chunk
    if (GLU) __syncthreads();   // their exchange
    return;
  }

  // ---- compute waves
  const int tile = GLU ? (wave < 2 ? 2 * blockIdx.x + wave : a.N / 32 + 2 * blockIdx.x + (wave - 2)) : 4 * blockIdx.x + wave;
  const bf16_t* wp = a.w16 + (((int64_t)tile * a.slices + slice) * nsteps * 64 + lane) * 8;      // the slice's step s at wp + 512 s
  uint4 wr[R64_RING];
  // (in this order and no other: the ring is used oldest first, and a wait is for the oldest load only if the
  // compiler sees the first loads come in the order of their use)
#pragma unroll
  for (int s = 0; s < R64_RING; ++s) {
    wr[s] = *(const uint4*)(wp + (int64_t)s * 512);
    __builtin_amdgcn_sched_barrier(0);
  }
  float4_t acc[BLOCKS];
#pragma unroll
  for (int b = 0; b < BLOCKS; ++b) acc[b] = (float4_t){0.f, 0.f, 0.f, 0.f};
  int at[4];                    // where this lane's piece of a step lies in a block, by the step's last two bits
#pragma unroll
  for (int i = 0; i < 4; ++i) at[i] = sk_place(r, i, g);
  // the scales of this lane's rows: the parts of a row's sum of squares in ascending order. The wait is for
  // loads that come back behind the ring's first turn, which the first products wait for anyway (in the
  // staging waves a wait for the parts held the second chunk's request back by a trip to memory).
  float scale[BLOCKS];
#pragma unroll
  for (int b = 0; b < BLOCKS; ++b) scale[b] = 1.f;
  if (a.ssq_in) {
#pragma unroll
    for (int b = 0; b < BLOCKS; ++b) {
      const int m = 16 * b + r;
      float total = 0.f;
      if (m < a.M) {
        total = a.ssq_in[(int64_t)m * a.ssq_parts];
        for (int q = 1; q < a.ssq_parts; ++q) total += a.ssq_in[(int64_t)m * a.ssq_parts + q];
      }
      scale[b] = 1.0f / sqrtf(total / (float)a.K + a.eps);
    }
  }
  __syncthreads();              // chunk 0 is there
  // a turn of the ring at a time, each register asked for again once it has been used; the last turn asks for nothing
  auto ring = [&](int base, auto more) {
#pragma unroll
    for (int h = 0; h < R64_RING / R64_CHUNK_STEPS; ++h) {
      // a chunk in batches of steps (pairs; single steps with 8 blocks of x): the next batch's operands leave
      // LDS while this batch's products run (left to itself the compiler reads two operands, waits,
      // multiplies, and so on)
      constexpr int PER = BLOCKS == 4 ? 2 : 1, BATCHES = R64_CHUNK_STEPS / PER;
      const int buf = (base / R64_CHUNK_STEPS + h) & 1;
      uint4 xb[2][PER][BLOCKS];
#pragma unroll
      for (int i = 0; i < PER; ++i)
#pragma unroll
        for (int b = 0; b < BLOCKS; ++b) xb[0][i][b] = xs(buf, i, b)[at[i & 3]];
#pragma unroll
      for (int q = 0; q < BATCHES; ++q) {
        if (q + 1 < BATCHES) {
#pragma unroll
          for (int i = 0; i < PER; ++i)
#pragma unroll
            for (int b = 0; b < BLOCKS; ++b) xb[(q + 1) & 1][i][b] = xs(buf, PER * (q + 1) + i, b)[at[(PER * (q + 1) + i) & 3]];
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < PER; ++i) {
          const int sl = R64_CHUNK_STEPS * h + PER * q + i;
#pragma unroll
          for (int b = 0; b < BLOCKS; ++b) acc[b] = sk_mfma(wr[sl], xb[q & 1][i][b], acc[b]);
          if (decltype(more)::value) wr[sl] = *(const uint4*)(wp + (int64_t)(base + R64_RING + sl) * 512);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      __syncthreads();
    }
  };
  int base = 0;
  for (; base + R64_RING < nsteps; base += R64_RING) ring(base, std::true_type{});
  ring(base, std::false_type{});
  // acc[b][j] = sum over k of W[row 16 tile + 4 g + j, k] * x[16 b + r, k]
  float4_t* ex = (float4_t*)xs_all;                      // [2 up waves][blocks][lane]; every read of x is behind the last barrier
  if (GLU) {
    if (wave >= 2) {
#pragma unroll
      for (int b = 0; b < BLOCKS; ++b) ex[((wave - 2) * BLOCKS + b) * TS_WAVE + lane] = acc[b];
    }
    __syncthreads();
    if (wave >= 2) return;
  }
  OUT* y = (OUT*)a.y + (int64_t)slice * a.M * a.ldy;
  const int n0 = GLU ? (2 * blockIdx.x + wave) * 16 + 4 * g : tile * 16 + 4 * g;
#pragma unroll
  for (int b = 0; b < BLOCKS; ++b) {
    const int m = 16 * b + r;
    if (m >= a.M) continue;
    float4_t u = {0.f, 0.f, 0.f, 0.f};
    if (GLU) u = ex[(wave * BLOCKS + b) * TS_WAVE + lane];
    acc[b] *= scale[b];
    u *= scale[b];
#pragma unroll
    for (int j = 0; j < 4; ++j) Num<OUT>::st(y + (int64_t)m * a.ldy + n0 + j, GLU ? sk_silu(acc[b][j]) * u[j] : acc[b][j]);
  }
}

#define R64_MAX_ROWS 128

template <bool GLU, typename OUT>
static int r64_launch(const Rows64Args& a, hipStream_t stream) {
  // 64 rows of W per workgroup; two buffers of a chunk of x in LDS: 64 KB for up to 64 rows, 128 KB beyond
  const dim3 grid(a.N / 64, a.slices);
  if (a.M <= 64) gemm_rows64_kernel<GLU, OUT, 4><<<grid, 512, 2 * R64_CHUNK_STEPS * 4 * TS_WAVE * sizeof(uint4), stream>>>(a);
  else gemm_rows64_kernel<GLU, OUT, 8><<<grid, 512, 2 * R64_CHUNK_STEPS * 8 * TS_WAVE * sizeof(uint4), stream>>>(a);
  return ts_check_launch();
}

static bool r64_operands_ok(const void* x, const void* w16, int M, int N, int K, int64_t ldx) {
  if (M > R64_MAX_ROWS || K <= 0 || ldx < K || (ldx % 8) || !x || !w16) return false;
  return !((((uintptr_t)x) | ((uintptr_t)w16)) & 15);
}

// x [M <= 128, K] (row stride ldx), w16: W [N, K] as its 16-row packed copy, y [M, N] or, with glu, [M, N / 2]
// (row stride ldy; out_f32: 32-bit sums instead of bfloat16). N a multiple of 64 (128 with glu), K of 1,024.
// ssq_in [M, ssq_parts] and eps: the prepared norm's scale per row (null: none).
extern "C" int ts_gemm_rows64_bf16(void* y, const void* x, const void* w16, int M, int N, int K, int64_t ldx, int64_t ldy,
                                   int glu, int out_f32, const void* ssq_in, int ssq_parts, float eps, hipStream_t stream) {
  if (M <= 0 || N <= 0) return TS_OK;
  if (N % (glu ? 128 : 64) || K % 1024 || !y || !r64_operands_ok(x, w16, M, N, K, ldx)) return TS_BAD_SHAPE;
  if (ldy < (glu ? N / 2 : N) || (((uintptr_t)y) & (out_f32 ? 3 : 1))) return TS_BAD_SHAPE;
  if (glu && out_f32) return TS_BAD_SHAPE;
  if (ssq_in && (ssq_parts <= 0 || (((uintptr_t)ssq_in) & 3))) return TS_BAD_SHAPE;
  Rows64Args a = {(const bf16_t*)x, (const bf16_t*)w16, y, M, N, K, ldx, ldy, (const float*)ssq_in, ssq_parts, eps, 1};
  if (glu) return r64_launch<true, bf16_t>(a, stream);
  if (out_f32) return r64_launch<false, float>(a, stream);
  return r64_launch<false, bf16_t>(a, stream);
}

// ---- a product in slices of its reduction, and what finishes it

#define R64_FINISH_THREADS 1024   // a workgroup of the finishing kernel takes a row, a thread four neighbouring columns at a time

struct Rows64FinishArgs {
  const float* parts;    // [slices][M][N]
  int slices, M, N;
  bf16_t* y;             // the product [M, N] (not NEXT)
  // NEXT: t = T(y) + res; res_out = T(t), op = T(t * nw), ssq_out [M] the rows' sums of t^2
  const bf16_t* res;     // [M, N] or null
  const bf16_t* nw;      // [N]
  bf16_t* res_out;
  bf16_t* op;            // rows ld_op apart
  float* ssq_out;
  int64_t ld_op;
};

// A workgroup per row: a thread adds the parts of four neighbouring columns, first slice first, then of the
// four columns 4,096 further on, and so on. The row's sum of squares: a thread's own columns in ascending
// order, the lanes of a wave in a fixed tree, the waves in ascending order.
template <bool NEXT>
__global__ void __launch_bounds__(R64_FINISH_THREADS) rows64_finish_kernel(const Rows64FinishArgs a) {
  __shared__ float wave_sq[R64_FINISH_THREADS / TS_WAVE];
  const int m = blockIdx.x;
  float sq = 0.f;
  for (int n = 4 * threadIdx.x; n < a.N; n += 4 * blockDim.x) {      // (N is a multiple of 64)
    const int64_t at = (int64_t)m * a.N + n;
    uint2 res = make_uint2(0, 0), nw = make_uint2(0, 0);
    if (NEXT) {
      nw = *(const uint2*)(a.nw + n);
      if (a.res) res = *(const uint2*)(a.res + at);
    }
    // four slices' parts asked for together, added first slice first
    float4 sum = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int s0 = 0; s0 < a.slices; s0 += 4) {
      float4 p[4];
#pragma unroll
      for (int j = 0; j < 4; ++j)
        p[j] = s0 + j < a.slices ? *(const float4*)(a.parts + (int64_t)(s0 + j) * a.M * a.N + at) : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (s0 + j == 0) { sum = p[0]; continue; }        // (not 0 + p: a sum of -0 stays -0)
        if (s0 + j < a.slices) { sum.x += p[j].x; sum.y += p[j].y; sum.z += p[j].z; sum.w += p[j].w; }
      }
    }
    const float s4[4] = {sum.x, sum.y, sum.z, sum.w};
    if (!NEXT) {
      *(uint2*)(a.y + at) = make_uint2(sk_round(s4[0]) | (sk_round(s4[1]) << 16), sk_round(s4[2]) | (sk_round(s4[3]) << 16));
      continue;
    }
    const uint32_t rw[2] = {res.x, res.y}, ww[2] = {nw.x, nw.y};
    float tv[4], ov[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {                           // (the low half of a word is the even column)
      const float rj = __uint_as_float((rw[j >> 1] >> (16 * (j & 1))) << 16);
      const float nj = __uint_as_float((ww[j >> 1] >> (16 * (j & 1))) << 16);
      const float t = __uint_as_float(sk_round(s4[j]) << 16) + rj;
      tv[j] = t;
      ov[j] = t * nj;
      sq = fmaf(t, t, sq);
    }
    *(uint2*)(a.res_out + at) = make_uint2(sk_round(tv[0]) | (sk_round(tv[1]) << 16), sk_round(tv[2]) | (sk_round(tv[3]) << 16));
    *(uint2*)(a.op + (int64_t)m * a.ld_op + n) = make_uint2(sk_round(ov[0]) | (sk_round(ov[1]) << 16), sk_round(ov[2]) | (sk_round(ov[3]) << 16));
  }
  if (!NEXT) return;
  sq = wave_sum(sq);
  if ((threadIdx.x & (TS_WAVE - 1)) == 0) wave_sq[threadIdx.x / TS_WAVE] = sq;
  __syncthreads();
  if (threadIdx.x == 0) {
    float total = 0.f;
#pragma unroll
    for (int w = 0; w < R64_FINISH_THREADS / TS_WAVE; ++w) total += w < (int)blockDim.x / TS_WAVE ? wave_sq[w] : 0.f;
    a.ssq_out[m] = total;
  }
}

// The same product with the reduction cut into `slices` (K / slices a multiple of 512), for a W of few rows:
// parts [slices][M][N] float is scratch that the call fills and reads. With next_nw the product is not stored:
// next_res_out [M, N], next_op [M, N] with rows ld_op apart (a multiple of 4, at least N) and ssq_out [M] (the rows'
// whole sums of squares: one part) are (next_res [M, N] or null is added first); without it y [M, N] bfloat16 is.
extern "C" int ts_gemm_rows64_sliced_bf16(void* y, void* parts, const void* x, const void* w16, int M, int N, int K, int64_t ldx,
                                          int slices, const void* next_res, const void* next_nw, void* next_res_out,
                                          void* next_op, void* ssq_out, int64_t ld_op, hipStream_t stream) {
  if (M <= 0 || N <= 0) return TS_OK;
  if (N % 64 || slices < 1 || slices > 64 || K % (512 * slices) || !parts || !r64_operands_ok(x, w16, M, N, K, ldx)) return TS_BAD_SHAPE;
  if (((uintptr_t)parts) & 15) return TS_BAD_SHAPE;
  Rows64FinishArgs f = {(const float*)parts, slices, M, N, (bf16_t*)y, (const bf16_t*)next_res, (const bf16_t*)next_nw,
                        (bf16_t*)next_res_out, (bf16_t*)next_op, (float*)ssq_out, ld_op};
  if (next_nw) {
    if (!next_res_out || !next_op || !ssq_out || (((uintptr_t)ssq_out) & 3) || ld_op < N || ld_op % 4) return TS_BAD_SHAPE;
    if ((((uintptr_t)next_res) | ((uintptr_t)next_nw) | ((uintptr_t)next_res_out) | ((uintptr_t)next_op)) & 7) return TS_BAD_SHAPE;
  } else if (!y || (((uintptr_t)y) & 7)) {
    return TS_BAD_SHAPE;
  }
  Rows64Args a = {(const bf16_t*)x, (const bf16_t*)w16, parts, M, N, K, ldx, (int64_t)N, nullptr, 0, 0.f, slices};
  const int rc = r64_launch<false, float>(a, stream);
  if (rc != TS_OK) return rc;
  const int threads = N / 4 >= R64_FINISH_THREADS ? R64_FINISH_THREADS : (N / 4 + TS_WAVE - 1) / TS_WAVE * TS_WAVE;
  if (next_nw) rows64_finish_kernel<true><<<M, threads, 0, stream>>>(f);
  else rows64_finish_kernel<false><<<M, threads, 0, stream>>>(f);
  return ts_check_launch();
}

// ---- the qkv projection in slices, finished into the rotation and the cache write

struct Rows64RopeArgs {
  const float* parts;    // [slices][M][N], columns in the order of hip.pack_weight_rope: a 16-column tile holds 8
                         // dimensions of a head's first half and, behind them, the 8 that rotate with them
  int slices, M, N, K;
  const float* ssq_in;   // a prepared norm's sums of squares [M, ssq_parts], or null
  int ssq_parts;
  float eps;
  const float* cos_sin;  // [positions, hd] 32-bit, [cos | sin] halves
  const int32_t* positions;
  const int32_t* slots;
  bf16_t* q_out;         // [M, nh * hd]
  bf16_t* k_cache;       // null: this layer owns no cache, only q is produced
  bf16_t* v_cache;
  int nh, nkv, hd, rotate, page_size;
  int64_t kp, ks, kh, vp, vs, vh, vd;   // key element: page * kp + offset * ks + head * kh + d; value: page * vp + offset * vs + head * vh + d * vd
};

// A workgroup per token: a thread adds the parts of four columns of a head's first half and of the four
// that rotate with them, first slice first, scales them by the prepared norm's rsqrt(mean square + eps),
// rounds them as the product would be stored, turns q and k by the token's position and writes q to
// q_out, k and v to the token's slot: what EPI_ROPE of gemm_skinny.hip does with its own sums.
__global__ void __launch_bounds__(R64_FINISH_THREADS) rows64_finish_rope_kernel(const Rows64RopeArgs a) {
  __shared__ float wave_sq[R64_FINISH_THREADS / TS_WAVE];
  const int m = blockIdx.x;
  float inv = 1.0f;
  if (a.ssq_in) {
    float v = 0.f;
    for (int q = threadIdx.x; q < a.ssq_parts; q += blockDim.x) v += a.ssq_in[(int64_t)m * a.ssq_parts + q];
    v = wave_sum(v);
    if ((threadIdx.x & (TS_WAVE - 1)) == 0) wave_sq[threadIdx.x / TS_WAVE] = v;
    __syncthreads();
    float total = 0.f;
    for (int w = 0; w < (int)blockDim.x / TS_WAVE; ++w) total += wave_sq[w];
    inv = __builtin_amdgcn_rsqf(total / (float)a.K + a.eps);
  }
  const int per_head = a.hd / 16, hdh = a.hd / 2;
  for (int idx = threadIdx.x; idx < a.N / 8; idx += blockDim.x) {
    const int jb = idx >> 1, nl = (idx & 1) * 4;            // the tile, and which four of its first eight columns
    const int64_t at = (int64_t)m * a.N + 16 * jb + nl;
    float4 s4 = make_float4(0.f, 0.f, 0.f, 0.f), u4 = s4;
    for (int s0 = 0; s0 < a.slices; s0 += 4) {
      float4 p[4], pu[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const bool in = s0 + j < a.slices;
        const float* src = a.parts + (int64_t)(s0 + j) * a.M * a.N + at;
        p[j] = in ? *(const float4*)src : make_float4(0.f, 0.f, 0.f, 0.f);
        pu[j] = in ? *(const float4*)(src + 8) : make_float4(0.f, 0.f, 0.f, 0.f);
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (s0 + j == 0) { s4 = p[0]; u4 = pu[0]; continue; }
        if (s0 + j < a.slices) {
          s4.x += p[j].x; s4.y += p[j].y; s4.z += p[j].z; s4.w += p[j].w;
          u4.x += pu[j].x; u4.y += pu[j].y; u4.z += pu[j].z; u4.w += pu[j].w;
        }
      }
    }
    const float s[4] = {s4.x * inv, s4.y * inv, s4.z * inv, s4.w * inv}, u[4] = {u4.x * inv, u4.y * inv, u4.z * inv, u4.w * inv};
    const int head = jb / per_head, d0 = 8 * (jb % per_head) + nl;      // d0 .. d0 + 3 of the head's first half
    float y1[4], y2[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {                         // as the product would be stored
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
  }
}

// The qkv projection of an attention layer for up to 64 rows of x with the reduction in `slices`
// (K / slices a multiple of 512): w16 is hip.pack_weight_rope of W [(nh + 2 nkv) * hd, K], parts
// [slices][M][N] float scratch. q_out [M, nh * hd] gets the rotated queries, the rotated keys and the
// values go to the slots `slots[m]` of the pages (slot -1 stores nothing; k_cache null: only q).
// ssq_in [M, ssq_parts] and eps: the prepared norm's scale per row (null: none). hd a multiple of 32,
// (nh + 2 nkv) * hd a multiple of 64, 8-byte aligned key strides.
extern "C" int ts_gemm_rows64_sliced_rope_bf16(void* q_out, void* parts, const void* x, const void* w16, int M, int K,
                                               int64_t ldx, int slices, const void* ssq_in, int ssq_parts, float eps,
                                               const float* cos_sin, const int32_t* positions, const int32_t* slots,
                                               void* k_cache, void* v_cache, int nh, int nkv, int hd, int rotate,
                                               int page_size, int64_t kp, int64_t ks, int64_t kh, int64_t vp, int64_t vs,
                                               int64_t vh, int64_t vd, hipStream_t stream) {
  if (M <= 0) return TS_OK;
  if (nh <= 0 || nkv < 0 || hd <= 0 || hd % 32 || page_size <= 0) return TS_BAD_SHAPE;
  const int N = (nh + 2 * nkv) * hd;
  if (N % 64 || slices < 1 || slices > 64 || K % (512 * slices) || !parts || !q_out || !r64_operands_ok(x, w16, M, N, K, ldx)) return TS_BAD_SHAPE;
  if ((((uintptr_t)parts) & 15) || (((uintptr_t)q_out) & 7)) return TS_BAD_SHAPE;
  if (ssq_in && (ssq_parts <= 0 || (((uintptr_t)ssq_in) & 3))) return TS_BAD_SHAPE;
  if (rotate && (!cos_sin || !positions)) return TS_BAD_SHAPE;
  if (k_cache && (!v_cache || !slots || (kp % 4) || (ks % 4) || (kh % 4) || (((uintptr_t)k_cache) & 7))) return TS_BAD_SHAPE;
  Rows64Args a = {(const bf16_t*)x, (const bf16_t*)w16, parts, M, N, K, ldx, (int64_t)N, nullptr, 0, 0.f, slices};
  const int rc = r64_launch<false, float>(a, stream);
  if (rc != TS_OK) return rc;
  Rows64RopeArgs f = {(const float*)parts, slices, M, N, K, (const float*)ssq_in, ssq_parts, eps, cos_sin, positions, slots,
                      (bf16_t*)q_out, (bf16_t*)k_cache, (bf16_t*)v_cache, nh, nkv, hd, rotate, page_size,
                      kp, ks, kh, vp, vs, vh, vd};
  const int threads = N / 8 >= R64_FINISH_THREADS ? R64_FINISH_THREADS : (N / 8 + TS_WAVE - 1) / TS_WAVE * TS_WAVE;
  rows64_finish_rope_kernel<<<M, threads, 0, stream>>>(f);
  return ts_check_launch();
}
