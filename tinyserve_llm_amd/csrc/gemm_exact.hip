// C[M, N] = A[M, K] · W[N, K]^T with 32-bit fused multiply-adds in ascending k for every output
// element, whatever M, N or the tile an element falls in: a row's result never depends on the other
// rows of the batch. This is the matrix product of the true 32-bit path (inputs float) and a plain
// stand-in for bfloat16 inputs (products exact in 32-bit, output rounded once). LDS-tiled 64x64x16,
// 256 threads, a 4x4 register tile per thread.
#include "common.h"

#define GE_BM 64
#define GE_BN 64
#define GE_BK 16

template <typename TA, typename TW, typename TC>
__global__ void __launch_bounds__(256)
gemm_exact_kernel(TC* __restrict__ C, const TA* __restrict__ A, const TW* __restrict__ W, int M, int N, int K,
                  int64_t lda, int64_t ldw, int64_t ldc) {
  __shared__ float As[GE_BK][GE_BM + 4];
  __shared__ float Ws[GE_BK][GE_BN + 4];
  const int tid = threadIdx.x;
  const int m0 = blockIdx.y * GE_BM, n0 = blockIdx.x * GE_BN;
  const int tx = tid & 15, ty = tid >> 4;  // thread's 4 columns start at tx*4, 4 rows at ty*4
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

  // loading: thread -> (row = tid / 4, 4 consecutive k starting at (tid % 4) * 4)
  const int lr = tid >> 2, lk = (tid & 3) * 4;
  for (int k0 = 0; k0 < K; k0 += GE_BK) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int k = k0 + lk + i;
      float a = 0.f, w = 0.f;
      if (k < K) {
        if (m0 + lr < M) a = Num<TA>::ld(A + (int64_t)(m0 + lr) * lda + k);
        if (n0 + lr < N) w = Num<TW>::ld(W + (int64_t)(n0 + lr) * ldw + k);
      }
      As[lk + i][lr] = a;
      Ws[lk + i][lr] = w;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < GE_BK; ++k) {
      float a[4], w[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[k][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) w[j] = Ws[k][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n < N) Num<TC>::st(C + (int64_t)m * ldc + n, acc[i][j]);
    }
  }
}

// The same sums for few rows of A (decode steps): a 64-row tile would be mostly empty and a narrow W would
// make a few dozen workgroups. Here a workgroup owns 16 rows of W, a thread one element of C, and the
// element's sum runs over k in the same ascending order with the same fused multiply-adds, so it is
// the same 32 bits as the tiled kernel gives.
#define GR_BN 16
#define GR_BM 16
#define GR_BK 64

template <typename TA, typename TW, typename TC>
__global__ void __launch_bounds__(256)
gemm_exact_rows_kernel(TC* __restrict__ C, const TA* __restrict__ A, const TW* __restrict__ W, int M, int N, int K,
                       int64_t lda, int64_t ldw, int64_t ldc) {
  __shared__ float As[GR_BM][GR_BK + 4];
  __shared__ float Ws[GR_BN][GR_BK + 4];
  const int tid = threadIdx.x;
  const int n0 = blockIdx.x * GR_BN, m0 = blockIdx.y * GR_BM;
  const int tx = tid & 15, ty = tid >> 4;     // this thread's element: row m0 + ty of A, row n0 + tx of W
  const int lr = tid >> 4, lk = (tid & 15) * 4;   // loading: row lr of the tile, 4 consecutive k from lk
  float acc = 0.f;
  for (int k0 = 0; k0 < K; k0 += GR_BK) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int k = k0 + lk + i;
      As[lr][lk + i] = (k < K && m0 + lr < M) ? Num<TA>::ld(A + (int64_t)(m0 + lr) * lda + k) : 0.f;
      Ws[lr][lk + i] = (k < K && n0 + lr < N) ? Num<TW>::ld(W + (int64_t)(n0 + lr) * ldw + k) : 0.f;
    }
    __syncthreads();
    // (the sum stops at K: no products of the tile's padding are added)
    const int kn = K - k0 < GR_BK ? K - k0 : GR_BK;
    for (int k = 0; k < kn; ++k) acc = fmaf(As[ty][k], Ws[tx][k], acc);
    __syncthreads();
  }
  const int m = m0 + ty, n = n0 + tx;
  if (m < M && n < N) Num<TC>::st(C + (int64_t)m * ldc + n, acc);
}

// in_dtype: storage of A and W; out_dtype: storage of C (0 float, 1 bfloat16).
extern "C" int ts_gemm_exact(void* C, const void* A, const void* W, int M, int N, int K, int64_t lda, int64_t ldw,
                             int64_t ldc, int in_dtype, int out_dtype, hipStream_t stream) {
  if (M <= 0 || N <= 0) return TS_OK;
  if (K <= 0 || lda < K || ldw < K || ldc < N) return TS_BAD_SHAPE;
  dim3 grid((N + GE_BN - 1) / GE_BN, (M + GE_BM - 1) / GE_BM), block(256);
  if (grid.y > 65535) return TS_BAD_SHAPE;
  if (M <= 2 * GR_BM) {                     // few rows: an element a thread
    dim3 rgrid((N + GR_BN - 1) / GR_BN, (M + GR_BM - 1) / GR_BM);
    if (in_dtype == 0 && out_dtype == 0)
      gemm_exact_rows_kernel<float, float, float><<<rgrid, block, 0, stream>>>((float*)C, (const float*)A, (const float*)W,
                                                                               M, N, K, lda, ldw, ldc);
    else if (in_dtype == 1 && out_dtype == 1)
      gemm_exact_rows_kernel<bf16_t, bf16_t, bf16_t><<<rgrid, block, 0, stream>>>((bf16_t*)C, (const bf16_t*)A,
                                                                                  (const bf16_t*)W, M, N, K, lda, ldw, ldc);
    else if (in_dtype == 1 && out_dtype == 0)
      gemm_exact_rows_kernel<bf16_t, bf16_t, float><<<rgrid, block, 0, stream>>>((float*)C, (const bf16_t*)A,
                                                                                 (const bf16_t*)W, M, N, K, lda, ldw, ldc);
    else
      return TS_BAD_DTYPE;
    return ts_check_launch();
  }
  if (in_dtype == 0 && out_dtype == 0)
    gemm_exact_kernel<float, float, float><<<grid, block, 0, stream>>>((float*)C, (const float*)A, (const float*)W, M,
                                                                       N, K, lda, ldw, ldc);
  else if (in_dtype == 1 && out_dtype == 1)
    gemm_exact_kernel<bf16_t, bf16_t, bf16_t><<<grid, block, 0, stream>>>((bf16_t*)C, (const bf16_t*)A,
                                                                          (const bf16_t*)W, M, N, K, lda, ldw, ldc);
  else if (in_dtype == 1 && out_dtype == 0)
    gemm_exact_kernel<bf16_t, bf16_t, float><<<grid, block, 0, stream>>>((float*)C, (const bf16_t*)A,
                                                                         (const bf16_t*)W, M, N, K, lda, ldw, ldc);
  else
    return TS_BAD_DTYPE;
  return ts_check_launch();
}
