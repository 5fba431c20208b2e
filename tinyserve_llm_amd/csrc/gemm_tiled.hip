// y[M, N] = x[M, K] · W[N, K]^T in bfloat16 with 32-bit accumulation for many rows of x, on the
// matrix cores with both operands tiled through LDS: this repository's own product beside the
// vendor library's (gemm_library.hip), which is the faster of the two (see the figures below) and
// the one the engine uses unless it is told otherwise.
//
// A workgroup of WM x WN waves computes a BM x BN tile of y, 64 of K at a time. Each k-step's
// slices of x and W are fetched by all threads as 16-byte pieces in the order the matrix
// instruction wants its operands (lane (r, g) of fragment f: row 16 (f / 2) + r, elements
// 32 (f % 2) + 8 g .. + 7), so that a wave's store into LDS and its later operand loads are
// contiguous kilobytes, free of bank conflicts. Two k-steps are in flight: while the waves
// multiply the step in one LDS buffer, the next step waits in registers to be written into the
// other buffer, and the loads of the step after it are on their way. The product is formed as
// y^T = W · x^T (W rows as the instruction's rows), which leaves a lane four consecutive columns
// of one row of y: an 8-byte store.
// GLU: W holds N / 2 gate rows, then N / 2 up rows; a workgroup takes BN / 2 of each, a wave holds
// a gate value and its up value in the same lane, and y[M, N / 2] = silu(gate) · up, each rounded
// to bfloat16 first as the separate kernels do.
// Measured (2,048 rows; tile 256 x 128, 8 waves): 682 TFLOP/s for N = 16,384, K = 2,048 where the
// library reaches 1,350; 128 x 128 tiles 420 to 560 where it reaches 800 to 1,290. A 128 x 128
// tile asks the vector memory path for 64 bytes per cycle of matrix instructions, all a compute
// unit has, so this design cannot pass about half the peak; the library's 256 x 256 tiles can.
#include "attention_mfma.h"

typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));   // (a plain vector: arrays of it stay in registers)

static __device__ __forceinline__ float4_t mfma32v(u32x4_t a, u32x4_t b, float4_t acc) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), acc, 0, 0, 0);
}

template <int BM, int BN, int WM, int WN, bool GLU, bool OUT32>
__global__ __launch_bounds__(WM * WN * TS_WAVE) void gemm_tiled_kernel(
    void* __restrict__ yv, const bf16_t* __restrict__ x, const bf16_t* __restrict__ w, int M, int N, int K,
    int64_t ldx, int64_t ldw, int64_t ldy, int row_tiles, int col_tiles, int per_die) {
  constexpr int THREADS = WM * WN * TS_WAVE;
  constexpr int FX = BM / 16 * 2, FW = BN / 16 * 2;       // fragments (a kilobyte each) of a k-step of 64
  constexpr int TM = BM / WM / 16, TN = BN / WN / 16;     // 16 x 16 tiles of a wave
  constexpr int LX = FX * 64 / THREADS, LW = FW * 64 / THREADS;
  static_assert(FX * 64 % THREADS == 0 && FW * 64 % THREADS == 0, "every thread fetches the same number of pieces");
  static_assert(!GLU || WN == 1, "a gate value and its up value must meet in one wave");
  static_assert(!(GLU && OUT32), "the gated result is bfloat16");
  bf16_t* __restrict__ y = (bf16_t*)yv;
  __shared__ u32x4_t lds[2][(FX + FW) * 64];
  // consecutive workgroups go to different dies: a die takes a contiguous run of tiles, column tile
  // by column tile, so that the tiles sharing a slice of W run on the die whose L2 holds it
  const int die = blockIdx.x % 8, turn = blockIdx.x / 8;
  const int item = die * per_die + turn;
  if (turn >= per_die || item >= row_tiles * col_tiles) return;
  const int m0 = (item % row_tiles) * BM, n0 = (item / row_tiles) * BN;
  const int t = threadIdx.x, lane = t % TS_WAVE, r = lane % 16, g = lane / 16;
  const int wave = wave_index(), wm = wave % WM, wn = wave / WM;

  const bf16_t* xp[LX];
  const bf16_t* wp[LW];
#pragma unroll
  for (int i = 0; i < LX; ++i) {
    const int f = (t + THREADS * i) / 64;
    xp[i] = x + (int64_t)min(m0 + (f / 2) * 16 + r, M - 1) * ldx + (f % 2) * 32 + 8 * g;
  }
#pragma unroll
  for (int i = 0; i < LW; ++i) {
    const int f = (t + THREADS * i) / 64;
    int col = (f / 2) * 16 + r;
    col = GLU ? n0 / 2 + col % (BN / 2) + (col >= BN / 2 ? N / 2 : 0) : n0 + col;
    wp[i] = w + (int64_t)min(col, N - 1) * ldw + (f % 2) * 32 + 8 * g;
  }
  u32x4_t sx0[LX], sw0[LW], sx1[LX], sw1[LW];
  float4_t acc[TN][TM];
#pragma unroll
  for (int j = 0; j < TN; ++j)
#pragma unroll
    for (int i = 0; i < TM; ++i) acc[j][i] = (float4_t){0.f, 0.f, 0.f, 0.f};

#define TS_FETCH(S, k0)                                                                                   \
  do {                                                                                                    \
    _Pragma("unroll") for (int i = 0; i < LX; ++i) sx##S[i] = *(const u32x4_t*)(xp[i] + (k0));            \
    _Pragma("unroll") for (int i = 0; i < LW; ++i) sw##S[i] = *(const u32x4_t*)(wp[i] + (k0));            \
  } while (0)
#define TS_STASH(S)                                                                                       \
  do {                                                                                                    \
    _Pragma("unroll") for (int i = 0; i < LX; ++i) lds[S][t + THREADS * i] = sx##S[i];                    \
    _Pragma("unroll") for (int i = 0; i < LW; ++i) lds[S][FX * 64 + t + THREADS * i] = sw##S[i];          \
  } while (0)
#define TS_MULTIPLY(S)                                                                                    \
  _Pragma("unroll") for (int h = 0; h < 2; ++h) {                                                         \
    u32x4_t fx[TM], fw[TN];                                                                               \
    _Pragma("unroll") for (int i = 0; i < TM; ++i) fx[i] = lds[S][((wm * TM + i) * 2 + h) * 64 + lane];   \
    _Pragma("unroll") for (int j = 0; j < TN; ++j) fw[j] = lds[S][FX * 64 + ((wn * TN + j) * 2 + h) * 64 + lane]; \
    _Pragma("unroll") for (int j = 0; j < TN; ++j)                                                        \
      _Pragma("unroll") for (int i = 0; i < TM; ++i) acc[j][i] = mfma32v(fw[j], fx[i], acc[j][i]);        \
  }
  // k-step s is fetched into register set s % 2, written into LDS buffer s % 2 one step before it
  // is multiplied, and its registers are free for step s + 2 from then on
  const int steps = K / 64;
  TS_FETCH(0, 0);
  if (steps == 1) {
    TS_STASH(0);
    __syncthreads();
    TS_MULTIPLY(0)
  } else {
    TS_FETCH(1, 64);
    TS_STASH(0);
    __syncthreads();
    int s = 0;
    for (; s + 3 < steps; s += 2) {
      TS_FETCH(0, 64 * (s + 2));
      TS_MULTIPLY(0)
      TS_STASH(1);
      __syncthreads();
      TS_FETCH(1, 64 * (s + 3));
      TS_MULTIPLY(1)
      TS_STASH(0);
      __syncthreads();
    }
    // two or three steps are left: step s in buffer 0, step s + 1 in register set 1
    if (steps - s == 3) {
      TS_FETCH(0, 64 * (s + 2));
      TS_MULTIPLY(0)
      TS_STASH(1);
      __syncthreads();
      TS_MULTIPLY(1)
      TS_STASH(0);
      __syncthreads();
      TS_MULTIPLY(0)
    } else {
      TS_MULTIPLY(0)
      TS_STASH(1);
      __syncthreads();
      TS_MULTIPLY(1)
    }
  }
#undef TS_FETCH
#undef TS_STASH
#undef TS_MULTIPLY

  // lane (r, g) of tile (j, i): row m0 + 16 (wm TM + i) + r of y, columns .. + 4 g .. + 3
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int m = m0 + (wm * TM + i) * 16 + r;
    if (m >= M) continue;
    if constexpr (GLU) {
#pragma unroll
      for (int j = 0; j < TN / 2; ++j) {
        const int n = n0 / 2 + j * 16 + 4 * g;
        if (n >= N / 2) continue;
        float o[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float gate = bf2f(f2bf(acc[j][i][e])), up = bf2f(f2bf(acc[j + TN / 2][i][e]));
          o[e] = gate / (1.f + __expf(-gate)) * up;
        }
        *(uint2*)(y + (int64_t)m * ldy + n) = make_uint2(pack_bf16(o[0], o[1]), pack_bf16(o[2], o[3]));
      }
    } else {
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const int n = n0 + (wn * TN + j) * 16 + 4 * g;
        if (n >= N) continue;
        const float4_t a = acc[j][i];
        if constexpr (OUT32) *(float4_t*)((float*)yv + (int64_t)m * ldy + n) = a;      // the 32-bit sums as they are
        else *(uint2*)(y + (int64_t)m * ldy + n) = make_uint2(pack_bf16(a[0], a[1]), pack_bf16(a[2], a[3]));
      }
    }
  }
}

template <int BM, int BN, int WM, int WN, bool GLU, bool OUT32 = false>
static int launch_tiled(void* y, const void* x, const void* w, int M, int N, int K, int64_t ldx, int64_t ldw,
                        int64_t ldy, hipStream_t stream) {
  const int row_tiles = (M + BM - 1) / BM, col_tiles = (N + BN - 1) / BN;
  const int per_die = (row_tiles * col_tiles + 7) / 8;
  gemm_tiled_kernel<BM, BN, WM, WN, GLU, OUT32><<<8 * per_die, WM * WN * TS_WAVE, 0, stream>>>(
      y, (const bf16_t*)x, (const bf16_t*)w, M, N, K, ldx, ldw, ldy, row_tiles, col_tiles, per_die);
  return ts_check_launch();
}

// x, w bfloat16, 16-byte aligned, rows ldx, ldw, ldy elements apart (multiples of 8; ldy of 4).
// K a multiple of 64. glu == 0: y [M, N], N a multiple of 4, bfloat16, or with out_f32 the 32-bit
// sums themselves (y float32, 16-byte aligned). glu != 0: w holds N / 2 gate rows, then N / 2 up
// rows, y [M, N / 2] = silu(gate) · up in bfloat16, N a multiple of 8.
extern "C" int ts_gemm_tiled_bf16(void* y, const void* x, const void* w, int M, int N, int K, int64_t ldx,
                                  int64_t ldw, int64_t ldy, int glu, int out_f32, hipStream_t stream) {
  if (M <= 0 || N <= 0) return TS_OK;
  if (K <= 0 || K % 64 || N % (glu ? 8 : 4) || ldx < K || ldw < K || ldy < (glu ? N / 2 : N)) return TS_BAD_SHAPE;
  if (ldx % 8 || ldw % 8 || ldy % 4 || !y || !x || !w) return TS_BAD_SHAPE;
  if ((((uintptr_t)x) | ((uintptr_t)w)) & 15 || ((uintptr_t)y) & (out_f32 ? 15 : 7) || (glu && out_f32)) return TS_BAD_SHAPE;
  // large tiles where they still give every compute unit two workgroups
  const int64_t big = (int64_t)((M + 255) / 256) * ((N + 127) / 128);
  if (glu) {
    if (big >= 512) return launch_tiled<256, 128, 4, 1, true>(y, x, w, M, N, K, ldx, ldw, ldy, stream);
    return launch_tiled<128, 128, 4, 1, true>(y, x, w, M, N, K, ldx, ldw, ldy, stream);
  }
  if (out_f32) {
    if (big >= 512) return launch_tiled<256, 128, 4, 2, false, true>(y, x, w, M, N, K, ldx, ldw, ldy, stream);
    return launch_tiled<128, 128, 2, 2, false, true>(y, x, w, M, N, K, ldx, ldw, ldy, stream);
  }
  if (big >= 512) return launch_tiled<256, 128, 4, 2, false>(y, x, w, M, N, K, ldx, ldw, ldy, stream);
  return launch_tiled<128, 128, 2, 2, false>(y, x, w, M, N, K, ldx, ldw, ldy, stream);
}
