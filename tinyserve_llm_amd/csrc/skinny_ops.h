// Small pieces of the weight-streaming kernels (gemm_skinny.hip): the matrix
// instruction on 16-byte operands, conversions between bfloat16 pairs and floats, the gate.
#pragma once
#include "common.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));

#define SK_KSTEP 32      // k covered by one MFMA: lane group g holds k = 8 g .. 8 g + 7
#define MODE_PLAIN 0
#define MODE_NORM 1
#define MODE_PREP 2
#define EPI_NONE 0
#define EPI_GLU 1
#define EPI_ROPE 2
#define EPI_NEXT 3

// acc + A · B over 32 k: lane (r, g) gives k = 8 g .. 8 g + 7 of row r of A and of column r of B
static __device__ __forceinline__ float4_t sk_mfma(const uint4& a, const uint4& b, float4_t acc) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), acc, 0, 0, 0);
}

static __device__ __forceinline__ void sk_unpack(const uint4& v, float* f) {
  const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    f[2 * i] = __uint_as_float(w[i] << 16);
    f[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
  }
}
// round to nearest even; the values here are finite sums and products of finite activations
static __device__ __forceinline__ uint32_t sk_round(float f) {
  const uint32_t u = __float_as_uint(f);
  return (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
}
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float float2_t __attribute__((ext_vector_type(2)));
// eight floats to eight bfloat16, round to nearest even, by the hardware's packed conversion
static __device__ __forceinline__ uint4 sk_pack(const float* f) {
  uint32_t w[4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
    w[i] = __builtin_bit_cast(uint32_t, __builtin_convertvector((float2_t){f[2 * i], f[2 * i + 1]}, bf16x2_t));
  return make_uint4(w[0], w[1], w[2], w[3]);
}
// Rows of x fetched in long pieces (a load takes 256 bytes or more of a row, not 64 bytes of each of 16 rows) reach the
// order the matrix instruction wants through LDS. Where in a block's [64] places of 16 bytes the piece of row r (of
// 16), step s, k = 8 g .. 8 g + 7 lies: the 16 pieces that neighbouring lanes of such a load write (one row, 4 steps
// x 4 g) land in 16 different places, and the 64 lanes of a reading wave (16 rows x 4 g of one step) read 64
// different places, so neither meets in a bank.
static __device__ __forceinline__ int sk_place(int r, int s, int g) { return (r ^ ((g + 4 * s) & 15)) + 16 * g; }

static __device__ __forceinline__ float sk_silu(float g) {
  return g * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.44269504088896340736f * g));
}

