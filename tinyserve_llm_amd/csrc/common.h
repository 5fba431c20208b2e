// Shared device helpers for the gfx950 kernels: storage types, conversions, wave reductions.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define TS_WAVE 64

typedef uint16_t bf16_t;  // bfloat16 stored as its 16 raw bits

__device__ __forceinline__ float bf2f(bf16_t h) { return __uint_as_float(((uint32_t)h) << 16); }

// round to nearest even; NaN stays NaN
__device__ __forceinline__ bf16_t f2bf(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (bf16_t)((u >> 16) | 0x40u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (bf16_t)(u >> 16);
}

template <typename T> struct Num;
template <> struct Num<float> {
  static __device__ __forceinline__ float ld(const float* p) { return *p; }
  static __device__ __forceinline__ void st(float* p, float v) { *p = v; }
  static __device__ __forceinline__ float round(float v) { return v; }
};
template <> struct Num<bf16_t> {
  static __device__ __forceinline__ float ld(const bf16_t* p) { return bf2f(*p); }
  static __device__ __forceinline__ void st(bf16_t* p, float v) { *p = f2bf(v); }
  static __device__ __forceinline__ float round(float v) { return bf2f(f2bf(v)); }
};

// A kernel's arguments lie in memory that no cache holds when the kernel starts, and the compiler fetches them
// as the code comes to need them: a long argument block is then waited for two or three times, a trip to
// memory each, before the first load of the operands can go out. This asks for one word of each 64 bytes of
// the block at the very start, so that all of it arrives in one trip and every later fetch finds it in the
// scalar cache.
template <int BYTES>
__device__ __forceinline__ void ts_fetch_arguments() {
  typedef const uint32_t __attribute__((address_space(4))) * args_t;
  const args_t block = (args_t)__builtin_amdgcn_kernarg_segment_ptr();
  uint32_t seen = 0;
#pragma unroll
  for (int at = 0; at < BYTES; at += 64) seen |= block[at / 4];
  asm volatile("" ::"s"(seen));
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = TS_WAVE / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, TS_WAVE);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = TS_WAVE / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, TS_WAVE));
  return v;
}

// Orders shared-memory writes of a wavefront before the reads of its other lanes.
__device__ __forceinline__ void wave_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Error codes returned by the extern "C" launchers (0 = launched).
#define TS_OK 0
#define TS_BAD_DTYPE 1
#define TS_BAD_SHAPE 2
#define TS_LAUNCH_FAILED 3
#define TS_TOO_LARGE 4

static inline int ts_check_launch() {
  return hipGetLastError() == hipSuccess ? TS_OK : TS_LAUNCH_FAILED;
}
