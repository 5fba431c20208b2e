// y[M, N] = e(f(x)[M, K] · W[N, K]^T) in bfloat16 for 17 to 64 rows of x and a wide W (the gate|up
// projection of a decode step of a few dozen requests), where time should go to reading W once.
//
// With so many rows the weight-streaming kernel of gemm_skinny.hip reads x from the second-level cache
// once per 32 rows of W, which is twice the bytes of W itself. Here a workgroup owns 64 rows of W and
// splits the work between two kinds of wave:
//   four compute waves, one 16-row tile of W each over the whole of K: the tile streams from memory
//   straight into MFMA operands, 16 steps of 32 k under way at any time (a step's register is asked for
//   again as soon as it has been used), and the four 16-row blocks of x come out of LDS;
//   four staging waves, which bring x into LDS in chunks of 256 k, in the order the lanes read it, one
//   chunk ahead of the compute waves (two buffers, a barrier per chunk). Their loads are few and hit the
//   cache; in waves of their own they do not queue behind the loads of W (a wave's loads come back in
//   the order it asked).
// The gate can ride along as in gemm_skinny.hip:
//   GLU   W = [gate rows | up rows]: waves 0 and 1 take two gate tiles, waves 2 and 3 the up tiles
//         N / 2 rows below them, and y [M, N / 2] = silu(gate) * up
// (The norm on the way in, which every workgroup would have to repeat for all of x, was tried in the
// staging waves and costs more than the norm kernel it saves: 37 µs against 21 + 7 at 64 rows.)
// W comes as the 16-row packed copy ([N / 16 tiles][K / 32 steps][64 lanes][8]); K is a multiple of
// 1,024. A row of x meets W's k in ascending order in one accumulator, whatever the other rows are.
#include <type_traits>
#include "skinny_ops.h"

#define R64_CHUNK_STEPS 8         // 32-wide k steps per chunk of x in LDS
#define R64_RING 16               // steps of W a compute wave has under way (two chunks): with 32 the chip had 32 MB under way and
                                  // every load, x's among them, came back some 5 us later (the gate|up product of 64 rows 20.7 us, 19.7 with 16)
#define R64_STAGE_STEPS (R64_CHUNK_STEPS / 4)   // steps of a chunk that one staging wave brings

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
};

template <bool GLU, typename OUT>
__global__ void __launch_bounds__(512) gemm_rows64_kernel(const Rows64Args a) {
  // x as the B operands of the matrix instruction: [buffer][step][block of 16 rows][lane], lane r + 16 g
  // holding k = 8 g .. 8 g + 7 of row r
  __shared__ uint4 xs[2][R64_CHUNK_STEPS][4][TS_WAVE];
  __shared__ float row_scale[64];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / TS_WAVE), lane = threadIdx.x & (TS_WAVE - 1);
  const int r = lane & 15, g = lane >> 4;
  const int nsteps = a.K / SK_KSTEP, nchunks = nsteps / R64_CHUNK_STEPS;   // (a multiple of 4)

  if (wave >= 4) {
    // ---- staging waves: wave sw brings steps 2 sw and 2 sw + 1 of every chunk, all four blocks of
    // rows. It asks for the next chunk before it puts this one into LDS, so that a chunk costs the
    // compute waves a barrier and not a trip to the cache.
    const int sw = wave - 4;
    bool ok[4];
    int64_t xoff[4];
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      ok[b] = 16 * b + r < a.M;                          // rows past M read row 0 and count as zeros
      xoff[b] = (int64_t)(ok[b] ? 16 * b + r : 0) * a.ldx + 8 * g;
    }
    auto ask = [&](int c, uint4 (&t)[R64_STAGE_STEPS][4]) {
      const int k0 = (c * R64_CHUNK_STEPS + R64_STAGE_STEPS * sw) * SK_KSTEP;   // first k of this wave's steps
#pragma unroll
      for (int s = 0; s < R64_STAGE_STEPS; ++s)
#pragma unroll
        for (int b = 0; b < 4; ++b) t[s][b] = *(const uint4*)(a.x + xoff[b] + k0 + s * SK_KSTEP);
    };
    auto put = [&](int c, const uint4 (&t)[R64_STAGE_STEPS][4]) {
#pragma unroll
      for (int s = 0; s < R64_STAGE_STEPS; ++s)
#pragma unroll
        for (int b = 0; b < 4; ++b) xs[c & 1][R64_STAGE_STEPS * sw + s][b][lane] = ok[b] ? t[s][b] : make_uint4(0, 0, 0, 0);
    };
    uint4 A[R64_STAGE_STEPS][4], B[R64_STAGE_STEPS][4];
    ask(0, A);
    // the rows' scales, rows 16 sw .. 16 sw + 15 in this wave: a lane every 64th part (all sixteen rows' loads
    // under way together), then the lanes in a fixed tree
    if (a.ssq_in) {
      float sums[16];
#pragma unroll
      for (int i = 0; i < 16; ++i) sums[i] = 0.f;
      for (int q = lane; q < a.ssq_parts; q += TS_WAVE) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int m = 16 * sw + i;
          sums[i] += m < a.M ? a.ssq_in[(int64_t)m * a.ssq_parts + q] : 0.f;
        }
      }
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const float total = wave_sum(sums[i]);
        if (lane == 0) row_scale[16 * sw + i] = 1.0f / sqrtf(total / (float)a.K + a.eps);
      }
    }
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
  const bf16_t* wp = a.w16 + ((int64_t)tile * nsteps * 64 + lane) * 8;      // step s at wp + 512 s
  uint4 wr[R64_RING];
  // (in this order and no other: the ring is used oldest first, and a wait is for the oldest load only if the
  // compiler sees the first loads come in the order of their use)
#pragma unroll
  for (int s = 0; s < R64_RING; ++s) {
    wr[s] = *(const uint4*)(wp + (int64_t)s * 512);
    __builtin_amdgcn_sched_barrier(0);
  }
  float4_t acc[4];
#pragma unroll
  for (int b = 0; b < 4; ++b) acc[b] = (float4_t){0.f, 0.f, 0.f, 0.f};
  __syncthreads();              // chunk 0 is there
  // a turn of the ring at a time, each register asked for again once it has been used; the last turn asks for nothing
  auto ring = [&](int base, auto more) {
#pragma unroll
    for (int h = 0; h < R64_RING / R64_CHUNK_STEPS; ++h) {
      // a chunk in four pairs of steps: the next pair's operands leave LDS while this pair's products
      // run (left to itself the compiler reads two operands, waits, multiplies, and so on)
      constexpr int PAIRS = R64_CHUNK_STEPS / 2;
      uint4 xb[2][2][4];
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int b = 0; b < 4; ++b) xb[0][i][b] = xs[(base / R64_CHUNK_STEPS + h) & 1][i][b][lane];
#pragma unroll
      for (int q = 0; q < PAIRS; ++q) {
        if (q + 1 < PAIRS) {
#pragma unroll
          for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int b = 0; b < 4; ++b) xb[(q + 1) & 1][i][b] = xs[(base / R64_CHUNK_STEPS + h) & 1][2 * (q + 1) + i][b][lane];
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          const int sl = R64_CHUNK_STEPS * h + 2 * q + i;
#pragma unroll
          for (int b = 0; b < 4; ++b) acc[b] = sk_mfma(wr[sl], xb[q & 1][i][b], acc[b]);
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
  float4_t* ex = (float4_t*)&xs[0][0][0][0];             // [2 up waves][4 blocks][lane]; every read of x is behind the last barrier
  if (GLU) {
    if (wave >= 2) {
#pragma unroll
      for (int b = 0; b < 4; ++b) ex[((wave - 2) * 4 + b) * TS_WAVE + lane] = acc[b];
    }
    __syncthreads();
    if (wave >= 2) return;
  }
  OUT* y = (OUT*)a.y;
  const int n0 = GLU ? (2 * blockIdx.x + wave) * 16 + 4 * g : tile * 16 + 4 * g;
#pragma unroll
  for (int b = 0; b < 4; ++b) {
    const int m = 16 * b + r;
    if (m >= a.M) continue;
    float4_t u = {0.f, 0.f, 0.f, 0.f};
    if (GLU) u = ex[(wave * 4 + b) * TS_WAVE + lane];
    if (a.ssq_in) {                                  // (the same for every thread)
      const float scale = row_scale[m];
      acc[b] *= scale;
      u *= scale;
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) Num<OUT>::st(y + (int64_t)m * a.ldy + n0 + j, GLU ? sk_silu(acc[b][j]) * u[j] : acc[b][j]);
  }
}

template <bool GLU, typename OUT>
static int r64_launch(const Rows64Args& a, hipStream_t stream) {
  gemm_rows64_kernel<GLU, OUT><<<a.N / 64, 512, 0, stream>>>(a);   // 64 rows of W per workgroup
  return ts_check_launch();
}

// x [M <= 64, K] (row stride ldx), w16: W [N, K] as its 16-row packed copy, y [M, N] or, with glu, [M, N / 2]
// (row stride ldy; out_f32: 32-bit sums instead of bfloat16). N a multiple of 64 (128 with glu), K of 1,024.
// ssq_in [M, ssq_parts] and eps: the prepared norm's scale per row (null: none).
extern "C" int ts_gemm_rows64_bf16(void* y, const void* x, const void* w16, int M, int N, int K, int64_t ldx, int64_t ldy,
                                   int glu, int out_f32, const void* ssq_in, int ssq_parts, float eps, hipStream_t stream) {
  if (M <= 0 || N <= 0) return TS_OK;
  if (M > 64 || N % (glu ? 128 : 64) || K <= 0 || K % 1024 || ldx < K || (ldx % 8) || !y || !x || !w16) return TS_BAD_SHAPE;
  if (ldy < (glu ? N / 2 : N) || (((uintptr_t)y) & (out_f32 ? 3 : 1))) return TS_BAD_SHAPE;
  if ((((uintptr_t)x) | ((uintptr_t)w16)) & 15) return TS_BAD_SHAPE;
  if (glu && out_f32) return TS_BAD_SHAPE;
  if (ssq_in && (ssq_parts <= 0 || (((uintptr_t)ssq_in) & 3))) return TS_BAD_SHAPE;
  Rows64Args a = {(const bf16_t*)x, (const bf16_t*)w16, y, M, N, K, ldx, ldy, (const float*)ssq_in, ssq_parts, eps};
  if (glu) return r64_launch<true, bf16_t>(a, stream);
  if (out_f32) return r64_launch<false, float>(a, stream);
  return r64_launch<false, bf16_t>(a, stream);
}
