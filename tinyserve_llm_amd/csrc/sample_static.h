// The one entry point of the kernel library that allocates nothing.
//
// It has no counterpart in tejkas/tinyserve-llm. It is for callers that cannot allocate device
// memory at the moment of the call: code that is being recorded into a HIP graph, serving loops that
// must not touch the allocator, and harnesses that forbid hipMalloc. The caller still brings inputs
// and outputs; what `ts_sample` takes as two workspaces lies here in a fixed array in device memory
// (512 KB, held by every GPU the library runs on until the process ends).
//
//   * At most TS_SAMPLE_STATIC_MAX_ROWS rows a call; more is refused with TS_TOO_LARGE and nothing
//     is launched.
//   * The device that `stream`, `out` and the inputs belong to must be the current one.
//   * Every call on a GPU uses that GPU's one array: calls that overlap on one GPU (two streams, two
//     threads) race and may return each other's tokens. Calls on one stream are ordered and safe.
//   * No hipMalloc, hipFree or allocating library routine is called.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define TS_SAMPLE_STATIC_MAX_ROWS 1024

// out[r] = the token drawn for row r of float32 `logits` [rows, vocab] (row stride `ld`): the
// highest logit where temps[r] is 0, else the exponential race with the noise of (seed, keys[r]).
// Returns 0, or an error code of common.h.
extern "C" int ts_sample_static(int32_t* out, const float* logits, const float* temps, const int64_t* keys,
                                uint64_t seed, int rows, int vocab, int64_t ld, hipStream_t stream);
