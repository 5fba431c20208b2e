// Token choice from 32-bit logits (64 workgroups share a row, a second kernel picks among their
// bests): the highest logit at temperature 0, else a
// draw from softmax(logits / temperature) by the exponential race
//     argmax_i  softmax_i / E_i   =   argmax_i  logit_i / t - log(E_i),   E_i ~ Exp(1), E_i >= 1e-10
// (tinyserve_llm/engine/sampler.py:13-23). The noise of element i of a row comes from a counter
// hash of (seed, the row's key, i), where the key names request, sample and output position: a
// draw does not depend on the row's place in the batch. Ties go to the lowest index.
#include "common.h"

#define SAMPLE_THREADS 256
#define SAMPLE_SLICES 64       // workgroups that share a row

__device__ __forceinline__ uint64_t mix64(uint64_t x) {
  x ^= x >> 30; x *= 0xBF58476D1CE4E5B9ull;
  x ^= x >> 27; x *= 0x94D049BB133111EBull;
  x ^= x >> 31;
  return x;
}

__device__ __forceinline__ float exp1_noise(uint64_t seed, uint64_t key, uint32_t i) {
  const uint64_t x = mix64(mix64(seed ^ (key * 0x9E3779B97F4A7C15ull)) + (uint64_t)i * 0xD1342543DE82EF95ull);
  const float u = (float)((x >> 40) + 1) * (1.0f / 16777216.0f);  // (0, 1]
  const float e = -logf(u);
  return e < 1e-10f ? 1e-10f : e;
}

__device__ __forceinline__ bool better(float v, int i, float bv, int bi) { return v > bv || (v == bv && i < bi); }

// Stage 1: workgroup (slice, row) finds the best of its slice of the vocabulary.
__global__ void __launch_bounds__(SAMPLE_THREADS)
sample_slice_kernel(float* __restrict__ best_v, int32_t* __restrict__ best_i, const float* __restrict__ logits,
                    const int32_t* __restrict__ row_of, const float* __restrict__ temps, const int64_t* __restrict__ keys,
                    uint64_t seed, int vocab, int64_t ld) {
  __shared__ float sv[SAMPLE_THREADS / TS_WAVE];
  __shared__ int si[SAMPLE_THREADS / TS_WAVE];
  const int r = blockIdx.y, slice = blockIdx.x;
  const float* row = logits + (int64_t)(row_of ? row_of[r] : r) * ld;   // several draws may read one row
  const float t = temps[r];
  const uint64_t key = (uint64_t)keys[r];
  const int per = (vocab + SAMPLE_SLICES - 1) / SAMPLE_SLICES;
  const int beg = slice * per, end = beg + per < vocab ? beg + per : vocab;
  float bv = -INFINITY;
  int bi = 0x7fffffff;
  for (int i = beg + threadIdx.x; i < end; i += SAMPLE_THREADS) {
    float v = row[i];
    if (t > 0.f) v = v / t - logf(exp1_noise(seed, key, (uint32_t)i));
    if (better(v, i, bv, bi)) { bv = v; bi = i; }
  }
#pragma unroll
  for (int off = TS_WAVE / 2; off > 0; off >>= 1) {
    const float ov = __shfl_xor(bv, off, TS_WAVE);
    const int oi = __shfl_xor(bi, off, TS_WAVE);
    if (better(ov, oi, bv, bi)) { bv = ov; bi = oi; }
  }
  if ((threadIdx.x & (TS_WAVE - 1)) == 0) { sv[threadIdx.x / TS_WAVE] = bv; si[threadIdx.x / TS_WAVE] = bi; }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < SAMPLE_THREADS / TS_WAVE; ++w)
      if (better(sv[w], si[w], bv, bi)) { bv = sv[w]; bi = si[w]; }
    best_v[r * SAMPLE_SLICES + slice] = bv;
    best_i[r * SAMPLE_SLICES + slice] = bi;
  }
}

// Stage 2: one wave per row picks among the slices' bests.
__global__ void __launch_bounds__(TS_WAVE)
sample_pick_kernel(int32_t* __restrict__ out, const float* __restrict__ best_v, const int32_t* __restrict__ best_i) {
  const int r = blockIdx.x, lane = threadIdx.x;
  float bv = lane < SAMPLE_SLICES ? best_v[r * SAMPLE_SLICES + lane] : -INFINITY;
  int bi = lane < SAMPLE_SLICES ? best_i[r * SAMPLE_SLICES + lane] : 0x7fffffff;
#pragma unroll
  for (int off = TS_WAVE / 2; off > 0; off >>= 1) {
    const float ov = __shfl_xor(bv, off, TS_WAVE);
    const int oi = __shfl_xor(bi, off, TS_WAVE);
    if (better(ov, oi, bv, bi)) { bv = ov; bi = oi; }
  }
  if (lane == 0) out[r] = bi == 0x7fffffff ? 0 : bi;
}

// work_v, work_i: [rows, SAMPLE_SLICES] float / int32 workspaces. row_of: null, or for each of the `rows`
// draws the row of `logits` it reads (checked by the caller against the rows that `logits` has).
static int sample_launch(int32_t* out, float* work_v, int32_t* work_i, const float* logits, const int32_t* row_of,
                         const float* temps, const int64_t* keys, uint64_t seed, int rows, int vocab, int64_t ld,
                         hipStream_t stream) {
  if (rows <= 0) return TS_OK;
  if (vocab <= 0 || ld < vocab || rows > 65535) return TS_BAD_SHAPE;
  static_assert(SAMPLE_SLICES <= TS_WAVE, "one wave picks among the slices");
  sample_slice_kernel<<<dim3(SAMPLE_SLICES, rows), SAMPLE_THREADS, 0, stream>>>(work_v, work_i, logits, row_of, temps,
                                                                              keys, seed, vocab, ld);
  int rc = ts_check_launch();
  if (rc) return rc;
  sample_pick_kernel<<<rows, TS_WAVE, 0, stream>>>(out, work_v, work_i);
  return ts_check_launch();
}

extern "C" int ts_sample(int32_t* out, float* work_v, int32_t* work_i, const float* logits, const float* temps,
                         const int64_t* keys, uint64_t seed, int rows, int vocab, int64_t ld, hipStream_t stream) {
  return sample_launch(out, work_v, work_i, logits, nullptr, temps, keys, seed, rows, vocab, ld, stream);
}

// The same for `rows` draws of which draw r reads row row_of[r] of `logits` (n samples of one prompt
// read the one row that its last position gave).
extern "C" int ts_sample_rows(int32_t* out, float* work_v, int32_t* work_i, const float* logits, const int32_t* row_of,
                              const float* temps, const int64_t* keys, uint64_t seed, int rows, int vocab, int64_t ld,
                              hipStream_t stream) {
  if (!row_of) return TS_BAD_SHAPE;
  return sample_launch(out, work_v, work_i, logits, row_of, temps, keys, seed, rows, vocab, ld, stream);
}

// ids[i] = prev[src[i]] where src[i] >= 0: the tokens a step drew become the next step's input
// without passing through the host (src names, per entry of the next step, the row of the step
// before whose token it feeds; -1 keeps the id the host packed).
__global__ void feed_tokens_kernel(int32_t* __restrict__ ids, const int32_t* __restrict__ prev,
                                   const int32_t* __restrict__ src, int n, int prev_n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int s = src[i];
  if (s >= 0 && s < prev_n) ids[i] = prev[s];
}

extern "C" int ts_feed_tokens(int32_t* ids, const int32_t* prev, const int32_t* src, int n, int prev_n,
                              hipStream_t stream) {
  if (n <= 0) return TS_OK;
  if (!ids || !prev || !src || prev_n <= 0) return TS_BAD_SHAPE;
  feed_tokens_kernel<<<(n + 255) / 256, 256, 0, stream>>>(ids, prev, src, n, prev_n);
  return ts_check_launch();
}

// ---- the draw without any allocation ---------------------------------------------------------------
// `ts_sample_static` is `ts_sample` with the two workspaces taken from a fixed array in device
// memory instead of from the caller (declared in sample_static.h, which says whom it is for).
// The array's name is only a handle on the host: the address that kernels and copies may use is
// asked for once per device, with that device current, and kept.
#include <mutex>
#include "sample_static.h"

#define SAMPLE_STATIC_BYTES ((size_t)TS_SAMPLE_STATIC_MAX_ROWS * SAMPLE_SLICES * (sizeof(float) + sizeof(int32_t)))
#define SAMPLE_STATIC_MAX_DEVICES 64

static __device__ __align__(256) unsigned char sample_scratch[SAMPLE_STATIC_BYTES];

static std::mutex sample_scratch_lock;
static void* sample_scratch_ptr[SAMPLE_STATIC_MAX_DEVICES];   // per device: where its copy of the array lies

// The current device's copy of the array, or nullptr if the runtime will not name it.
static void* sample_scratch_here() {
  int device = -1;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= SAMPLE_STATIC_MAX_DEVICES) return nullptr;
  std::lock_guard<std::mutex> hold(sample_scratch_lock);
  if (sample_scratch_ptr[device] == nullptr) {
    void* ptr = nullptr;
    if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(sample_scratch)) != hipSuccess) return nullptr;
    sample_scratch_ptr[device] = ptr;
  }
  return sample_scratch_ptr[device];
}

extern "C" int ts_sample_static(int32_t* out, const float* logits, const float* temps, const int64_t* keys,
                                uint64_t seed, int rows, int vocab, int64_t ld, hipStream_t stream) {
  if (rows <= 0) return TS_OK;
  if (rows > TS_SAMPLE_STATIC_MAX_ROWS) return TS_TOO_LARGE;
  if (!out || !logits || !temps || !keys) return TS_BAD_SHAPE;
  unsigned char* base = (unsigned char*)sample_scratch_here();
  if (base == nullptr) return TS_LAUNCH_FAILED;
  // every (row, slice) place that the second kernel reads is written by the first kernel of the same
  // call, so nothing of the last call's contents has to be cleared
  float* work_v = (float*)base;
  int32_t* work_i = (int32_t*)(base + (size_t)TS_SAMPLE_STATIC_MAX_ROWS * SAMPLE_SLICES * sizeof(float));
  return ts_sample(out, work_v, work_i, logits, temps, keys, seed, rows, vocab, ld, stream);
}
