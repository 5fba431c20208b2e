// y[M, N] = x[M, K] · W[N, K]^T for bfloat16 with few rows of x (decoding: M up to 64), where time
// goes to reading W once from HBM. A workgroup of four waves owns 16 or 32 rows of W; the waves
// split K among them, stream their slice of those rows with 16-byte loads straight into MFMA
// operands (v_mfma_f32_16x16x16_bf16: W rows are the A matrix, x^T the B matrix), and the four
// partial tiles are summed in LDS in a fixed order. x is read through the caches (it is tiny and
// shared by every workgroup). Accumulation is 32-bit; the result is rounded once.
#include "common.h"

typedef short short4_t __attribute__((ext_vector_type(4)));
typedef float float4_t __attribute__((ext_vector_type(4)));

#define SK_WAVES 4
#define SK_KSTEP 32   // k covered by one pair of MFMAs: lane group g holds k = 8 g .. 8 g + 7

// RT: 16-row tiles of W per workgroup (1 or 2); CB: 16-row blocks of x (1..4)
template <int RT, int CB, typename OUT>
__global__ void __launch_bounds__(SK_WAVES * TS_WAVE)
gemm_skinny_kernel(OUT* __restrict__ y, const bf16_t* __restrict__ x, const bf16_t* __restrict__ w, int M, int N,
                   int K, int64_t ldx, int64_t ldw, int64_t ldy) {
  __shared__ float part[SK_WAVES][RT][CB][16 * 16];
  const int wave = threadIdx.x / TS_WAVE, lane = threadIdx.x & (TS_WAVE - 1);
  const int r = lane & 15, g = lane >> 4;
  const int n0 = blockIdx.x * 16 * RT;
  const int kslice = K / SK_WAVES;              // a multiple of SK_KSTEP (checked on the host)
  const int kbeg = wave * kslice;

  float4_t acc[RT][CB];
#pragma unroll
  for (int a = 0; a < RT; ++a)
#pragma unroll
    for (int b = 0; b < CB; ++b) acc[a][b] = (float4_t){0.f, 0.f, 0.f, 0.f};

  const bf16_t* wrow[RT];
#pragma unroll
  for (int a = 0; a < RT; ++a) {
    int n = n0 + a * 16 + r;
    if (n >= N) n = N - 1;                       // rows past the end are computed and not stored
    wrow[a] = w + (int64_t)n * ldw + kbeg + 8 * g;
  }
  const bf16_t* xrow[CB];
  bool xok[CB];
#pragma unroll
  for (int b = 0; b < CB; ++b) {
    const int m = b * 16 + r;
    xok[b] = m < M;
    xrow[b] = x + (int64_t)(xok[b] ? m : 0) * ldx + kbeg + 8 * g;
  }

#pragma unroll 4
  for (int k = 0; k < kslice; k += SK_KSTEP) {
    uint4 wa[RT], xb[CB];
#pragma unroll
    for (int a = 0; a < RT; ++a) wa[a] = *(const uint4*)(wrow[a] + k);
#pragma unroll
    for (int b = 0; b < CB; ++b) xb[b] = xok[b] ? *(const uint4*)(xrow[b] + k) : make_uint4(0, 0, 0, 0);
#pragma unroll
    for (int a = 0; a < RT; ++a) {
      const short4_t a0 = __builtin_bit_cast(short4_t, make_uint2(wa[a].x, wa[a].y));
      const short4_t a1 = __builtin_bit_cast(short4_t, make_uint2(wa[a].z, wa[a].w));
#pragma unroll
      for (int b = 0; b < CB; ++b) {
        const short4_t b0 = __builtin_bit_cast(short4_t, make_uint2(xb[b].x, xb[b].y));
        const short4_t b1 = __builtin_bit_cast(short4_t, make_uint2(xb[b].z, xb[b].w));
        acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a0, b0, acc[a][b], 0, 0, 0);
        acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a1, b1, acc[a][b], 0, 0, 0);
      }
    }
  }
  // acc[a][b][j] = sum over this wave's k of W[n0 + 16 a + 4 g + j, k] * x[16 b + r, k]
#pragma unroll
  for (int a = 0; a < RT; ++a)
#pragma unroll
    for (int b = 0; b < CB; ++b)
#pragma unroll
      for (int j = 0; j < 4; ++j) part[wave][a][b][r * 16 + 4 * g + j] = acc[a][b][j];
  __syncthreads();
  // part[.][a][b][m_local * 16 + n_local]: each thread sums 4 consecutive n of one m, all waves in order
  for (int idx = threadIdx.x; idx < RT * CB * 64; idx += SK_WAVES * TS_WAVE) {
    const int tile = idx >> 6, e = idx & 63;
    const int a = tile / CB, b = tile - a * CB;
    const int ml = e >> 2, nl = (e & 3) * 4;
    const int m = b * 16 + ml, n = n0 + a * 16 + nl;
    if (m >= M) continue;
    float s[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      float t = 0.f;
#pragma unroll
      for (int wv = 0; wv < SK_WAVES; ++wv) t += part[wv][a][b][ml * 16 + nl + j];
      s[j] = t;
    }
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (n + j < N) Num<OUT>::st(y + (int64_t)m * ldy + n + j, s[j]);
  }
}

template <typename OUT>
static int launch_skinny(void* y, const void* x, const void* w, int M, int N, int K, int64_t ldx, int64_t ldw,
                         int64_t ldy, hipStream_t stream) {
  const int cb = (M + 15) / 16;
  // two row tiles per workgroup once that still leaves a few workgroups per compute unit
  const int rt = (N >= 16 * 2 * 1024) ? 2 : 1;
  dim3 grid((N + 16 * rt - 1) / (16 * rt)), block(SK_WAVES * TS_WAVE);
#define SK_LAUNCH(RT, CB)                                                                                      \
  gemm_skinny_kernel<RT, CB, OUT><<<grid, block, 0, stream>>>((OUT*)y, (const bf16_t*)x, (const bf16_t*)w, M, N, \
                                                              K, ldx, ldw, ldy)
  if (rt == 1) {
    switch (cb) {
      case 1: SK_LAUNCH(1, 1); break;
      case 2: SK_LAUNCH(1, 2); break;
      case 3: SK_LAUNCH(1, 3); break;
      default: SK_LAUNCH(1, 4); break;
    }
  } else {
    switch (cb) {
      case 1: SK_LAUNCH(2, 1); break;
      case 2: SK_LAUNCH(2, 2); break;
      case 3: SK_LAUNCH(2, 3); break;
      default: SK_LAUNCH(2, 4); break;
    }
  }
#undef SK_LAUNCH
  return ts_check_launch();
}

// out_dtype: 1 bfloat16, 0 float. Requires M <= 64, K a multiple of 128, 16-byte aligned rows.
extern "C" int ts_gemm_skinny_bf16(void* y, const void* x, const void* w, int M, int N, int K, int64_t ldx,
                                   int64_t ldw, int64_t ldy, int out_dtype, hipStream_t stream) {
  if (M <= 0 || N <= 0) return TS_OK;
  if (M > 64 || K <= 0 || K % (SK_WAVES * SK_KSTEP) || ldx % 8 || ldw % 8 || ldx < K || ldw < K || ldy < N)
    return TS_BAD_SHAPE;
  if (((uintptr_t)x | (uintptr_t)w) & 15) return TS_BAD_SHAPE;
  if (out_dtype == 1) return launch_skinny<bf16_t>(y, x, w, M, N, K, ldx, ldw, ldy, stream);
  if (out_dtype == 0) return launch_skinny<float>(y, x, w, M, N, K, ldx, ldw, ldy, stream);
  return TS_BAD_DTYPE;
}
