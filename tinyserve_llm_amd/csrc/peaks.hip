// Two kernels that do nothing useful as fast as they can, to measure on the box what the published
// peaks promise: one reads an array once (memory bandwidth), one issues matrix instructions on
// registers (bfloat16 matrix rate). bench.py --peaks times them.
#include "skinny_ops.h"

// every workgroup reads its contiguous share in 16-byte pieces, eight loads in flight per lane
__global__ void __launch_bounds__(256) peak_read_kernel(const uint4* __restrict__ p, size_t pieces, uint32_t* __restrict__ sink) {
  const size_t per_group = (pieces + gridDim.x - 1) / gridDim.x;
  const size_t begin = (size_t)blockIdx.x * per_group, end = begin + per_group < pieces ? begin + per_group : pieces;
  uint32_t acc = 0;
  size_t i = begin + threadIdx.x;
  for (; i + 7 * 256 < end; i += 8 * 256) {
    uint4 v[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = p[i + (size_t)j * 256];
#pragma unroll
    for (int j = 0; j < 8; ++j) acc ^= v[j].x ^ v[j].y ^ v[j].z ^ v[j].w;
  }
  for (; i < end; i += 256) { const uint4 v = p[i]; acc ^= v.x ^ v.y ^ v.z ^ v.w; }
  if (acc == 0x9e3779b9u) sink[blockIdx.x] = acc;     // (never, in practice: the loads must not be optimised away)
}

// four independent chains of v_mfma_f32_16x16x32_bf16 per wave
__global__ void __launch_bounds__(256) peak_mfma_kernel(float* __restrict__ sink, int iters) {
  const uint32_t one = 0x3f803f80u;                   // two bfloat16 ones
  const uint4 a = make_uint4(one, one, one, one), b = make_uint4(one + threadIdx.x % 2, one, one, one);
  float4_t acc[4];
#pragma unroll
  for (int c = 0; c < 4; ++c) acc[c] = (float4_t){0.f, 0.f, 0.f, 0.f};
  for (int i = 0; i < iters; ++i) {
#pragma unroll
    for (int c = 0; c < 4; ++c) acc[c] = sk_mfma(a, b, acc[c]);
  }
  float s = 0.f;
#pragma unroll
  for (int c = 0; c < 4; ++c) s += acc[c][0] + acc[c][1] + acc[c][2] + acc[c][3];
  if (s == -1.0f) sink[blockIdx.x] = s;               // (never)
}

// Reads `bytes` (a multiple of 16) at p once with `workgroups` workgroups.
extern "C" int ts_peak_read(const void* p, size_t bytes, void* sink, int workgroups, hipStream_t stream) {
  if (!p || !sink || bytes % 16 || workgroups <= 0 || ((uintptr_t)p & 15)) return TS_BAD_SHAPE;
  peak_read_kernel<<<workgroups, 256, 0, stream>>>((const uint4*)p, bytes / 16, (uint32_t*)sink);
  return ts_check_launch();
}

// workgroups x 4 waves x iters x 4 matrix instructions of 2 x 16 x 16 x 32 operations each.
extern "C" int ts_peak_mfma(void* sink, int iters, int workgroups, hipStream_t stream) {
  if (!sink || iters <= 0 || workgroups <= 0) return TS_BAD_SHAPE;
  peak_mfma_kernel<<<workgroups, 256, 0, stream>>>((float*)sink, iters);
  return ts_check_launch();
}
