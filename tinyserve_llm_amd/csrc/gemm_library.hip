// y[M, N] = x[M, K] · W[N, K]^T in bfloat16 with 32-bit accumulation (y bfloat16, or the 32-bit sums
// themselves) for many rows of x, through the
// vendor's matrix library (hipBLASLt), called directly: the descriptors and the algorithm the
// library's heuristic picks for a shape are made once and kept, so that a call costs little more
// than the launch (a framework's general matmul asks the heuristic again at every call, which is
// most of its 20 µs on the host, and that is what bounds steps of a few hundred tokens).
// For products with few rows (decode steps of 33 to 256 requests) the heuristic's first candidate is
// often not the fastest (measured at 64 rows with weights read from memory, the layer sizes of a 1B
// Llama: qkv 12.0 µs against 8.9 for the best candidate, o 11.8 against 8.8, down 23.2 against
// 15.5), so a caller may ask for such a shape to be tuned: every candidate is timed on the call's
// own operands, with the caches swept in between as they are when a step reads each weight once,
// and the fastest is kept.
// For products with many rows the heuristic's choice depends on the row count in a way the work does
// not: at the layer sizes of an 8B Llama, 2,048 rows take 761 µs for a layer's four products and
// 2,063 rows (a prompt portion beside fifteen decoding requests) 865 µs, the down projection alone
// 209 and 357; 4,096 rows 1,167 µs and 4,127 rows 1,711. So a shape of more than 256 rows that is
// no multiple of 256 also tries the algorithms the heuristic picks for the multiples of 256 below
// and above it, where the library supports them for the shape, and keeps the fastest of the three
// (timed once, at the shape's first call outside a capture, on that call's operands).
// Row-major y = x · W^T is, in the library's column-major terms, y^T = W^T-as-stored transposed
// times x^T-as-stored: A = W with op T (K x N, leading dimension ldw), B = x with op N (K x M,
// leading dimension ldx), D = y (N x M, leading dimension ldy).
#include <hipblaslt/hipblaslt.h>
#include <hipblaslt/hipblaslt-ext.hpp>

#include <map>
#include <mutex>
#include <tuple>

#include "common.h"

namespace {

constexpr size_t LT_WORKSPACE_BYTES = 128u << 20;  // what the library may use per device, allocated once
constexpr int LT_MAX_DEVICES = 16;
constexpr size_t LT_MAX_PLANS = 8192;              // per device; a serving process meets many row counts
constexpr int LT_CANDIDATES = 16;                  // asked of the heuristic for a plan,
constexpr int LT_TUNE_CANDIDATES = 48;             // and when a shape is tuned
constexpr int LT_TUNE_MIN_ROWS = 9;                // shapes with fewer rows keep the heuristic's choice (little to gain),
constexpr int LT_TUNE_MAX_ROWS = 256;              // and so do shapes with more (the first candidate was the fastest)
constexpr int LT_TUNE_RUNS = 2;                    // timed runs per candidate; the faster counts
constexpr int LT_GRAPH_MAX_ROWS = 1024;            // the most rows of a step that may be recorded into a graph
constexpr int LT_BORROW_ROWS = 256;                // shapes beyond the tuned ones borrow from the multiples of this many rows

struct LtPlan {
  hipblasLtMatmulDesc_t desc = nullptr;
  hipblasLtMatrixLayout_t a = nullptr, b = nullptr, d = nullptr;
  hipblasLtMatmulAlgo_t algo;
  size_t workspace = 0;
  bool tuned = false;
  bool chosen = false;       // picked among borrowed algorithms by timing
  // algorithms picked for neighbouring row counts that also serve this shape, until one of them
  // or `algo` has been chosen by timing
  int borrowed = 0;
  hipblasLtMatmulAlgo_t other[2];
  size_t other_workspace[2] = {0, 0};
};

struct LtDevice {
  hipblasLtHandle_t handle = nullptr;
  void* workspace = nullptr;
  std::map<std::tuple<int, int, int, int64_t, int64_t, int64_t, int>, LtPlan> plans;   // (..., 32-bit output or not)
};

std::mutex lt_mutex;
LtDevice lt_devices[LT_MAX_DEVICES];
// Whether candidates may be timed at all. Off: every shape keeps the heuristic's first candidate,
// so that two processes round a product the same way (candidates differ in the order of their sums).
bool lt_timing = true;

// The first of the library's candidates for these layouts that fits the workspace (they come best
// first, whatever workspace they want). Shapes that a recorded decode step may hold take a candidate
// without workspace if there is one: an algorithm that clears its workspace would put a memory-set
// node into the graph.
bool lt_first(LtDevice& dev, hipblasLtMatmulDesc_t desc, hipblasLtMatrixLayout_t a, hipblasLtMatrixLayout_t b,
              hipblasLtMatrixLayout_t d, int M, hipblasLtMatmulAlgo_t* algo, size_t* workspace) {
  hipblasLtMatmulPreference_t pref = nullptr;
  if (hipblasLtMatmulPreferenceCreate(&pref) != HIPBLAS_STATUS_SUCCESS) return false;
  const uint64_t limit = LT_WORKSPACE_BYTES;
  bool ok = hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &limit, sizeof(limit)) == HIPBLAS_STATUS_SUCCESS;
  hipblasLtMatmulHeuristicResult_t found[LT_CANDIDATES];
  int count = 0, pick = -1;
  ok = ok && hipblasLtMatmulAlgoGetHeuristic(dev.handle, desc, a, b, d, d, pref, LT_CANDIDATES, found, &count) == HIPBLAS_STATUS_SUCCESS;
  for (int i = 0; ok && M <= LT_GRAPH_MAX_ROWS && i < count && pick < 0; ++i)
    if (found[i].state == HIPBLAS_STATUS_SUCCESS && found[i].workspaceSize == 0) pick = i;
  for (int i = 0; ok && i < count && pick < 0; ++i)
    if (found[i].state == HIPBLAS_STATUS_SUCCESS && found[i].workspaceSize <= LT_WORKSPACE_BYTES) pick = i;
  hipblasLtMatmulPreferenceDestroy(pref);
  if (!ok || pick < 0) return false;
  *algo = found[pick].algo;
  *workspace = found[pick].workspaceSize;
  return true;
}

// What the heuristic picks for `rows` rows of the plan's shape, if the library supports it for the
// plan's own row count too (within the workspace, and without one where the shape may be recorded).
void lt_borrow(LtDevice& dev, LtPlan& plan, int M, int N, int K, int64_t ldx, int64_t ldy, int rows, hipDataType out) {
  hipblasLtMatrixLayout_t b = nullptr, d = nullptr;
  hipblasLtMatmulAlgo_t algo;
  size_t workspace = 0;
  const float one = 1.0f, zero = 0.0f;
  if (hipblasLtMatrixLayoutCreate(&b, HIP_R_16BF, K, rows, ldx) == HIPBLAS_STATUS_SUCCESS &&
      hipblasLtMatrixLayoutCreate(&d, out, N, rows, ldy) == HIPBLAS_STATUS_SUCCESS &&
      lt_first(dev, plan.desc, plan.a, b, d, M, &algo, &workspace) &&
      hipblaslt_ext::matmulIsAlgoSupported(dev.handle, plan.desc, &one, plan.a, plan.b, &zero, plan.d, plan.d, algo,
                                           workspace) == HIPBLAS_STATUS_SUCCESS &&
      workspace <= LT_WORKSPACE_BYTES && (M > LT_GRAPH_MAX_ROWS || workspace == 0)) {
    plan.other[plan.borrowed] = algo;
    plan.other_workspace[plan.borrowed] = workspace;
    ++plan.borrowed;
  }
  if (b) hipblasLtMatrixLayoutDestroy(b);
  if (d) hipblasLtMatrixLayoutDestroy(d);
}

// The plan for a shape on the current device; made (and the library asked for its best algorithm)
// the first time the shape is met. Returns null if the library has nothing for it.
LtPlan* lt_plan(LtDevice& dev, int M, int N, int K, int64_t ldx, int64_t ldw, int64_t ldy, int out_f32) {
  const auto key = std::make_tuple(M, N, K, ldx, ldw, ldy, out_f32);
  const hipDataType out = out_f32 ? HIP_R_32F : HIP_R_16BF;
  auto it = dev.plans.find(key);
  if (it != dev.plans.end()) return it->second.desc ? &it->second : nullptr;
  if (dev.plans.size() >= LT_MAX_PLANS) {   // start over rather than grow without bound
    for (auto& kv : dev.plans) {
      if (!kv.second.desc) continue;
      hipblasLtMatrixLayoutDestroy(kv.second.a);
      hipblasLtMatrixLayoutDestroy(kv.second.b);
      hipblasLtMatrixLayoutDestroy(kv.second.d);
      hipblasLtMatmulDescDestroy(kv.second.desc);
    }
    dev.plans.clear();
  }
  LtPlan plan;
  bool ok = hipblasLtMatmulDescCreate(&plan.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F) == HIPBLAS_STATUS_SUCCESS;
  const hipblasOperation_t ta = HIPBLAS_OP_T, tb = HIPBLAS_OP_N;
  ok = ok && hipblasLtMatmulDescSetAttribute(plan.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &ta, sizeof(ta)) == HIPBLAS_STATUS_SUCCESS;
  ok = ok && hipblasLtMatmulDescSetAttribute(plan.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &tb, sizeof(tb)) == HIPBLAS_STATUS_SUCCESS;
  ok = ok && hipblasLtMatrixLayoutCreate(&plan.a, HIP_R_16BF, K, N, ldw) == HIPBLAS_STATUS_SUCCESS;
  ok = ok && hipblasLtMatrixLayoutCreate(&plan.b, HIP_R_16BF, K, M, ldx) == HIPBLAS_STATUS_SUCCESS;
  ok = ok && hipblasLtMatrixLayoutCreate(&plan.d, out, N, M, ldy) == HIPBLAS_STATUS_SUCCESS;
  ok = ok && lt_first(dev, plan.desc, plan.a, plan.b, plan.d, M, &plan.algo, &plan.workspace);
  if (ok) {
    if (M > LT_TUNE_MAX_ROWS && M % LT_BORROW_ROWS) {
      lt_borrow(dev, plan, M, N, K, ldx, ldy, M / LT_BORROW_ROWS * LT_BORROW_ROWS, out);
      lt_borrow(dev, plan, M, N, K, ldx, ldy, (M / LT_BORROW_ROWS + 1) * LT_BORROW_ROWS, out);
    }
  } else {
    if (plan.a) hipblasLtMatrixLayoutDestroy(plan.a);
    if (plan.b) hipblasLtMatrixLayoutDestroy(plan.b);
    if (plan.d) hipblasLtMatrixLayoutDestroy(plan.d);
    if (plan.desc) hipblasLtMatmulDescDestroy(plan.desc);
    plan = LtPlan();                        // remembered as "nothing for this shape"
  }
  auto& kept = dev.plans[key];
  kept = plan;
  return kept.desc ? &kept : nullptr;
}

// Times the library's candidates for the plan's shape on the operands of this call and keeps the
// fastest. Before every timed run `flush_bytes` at `flush` are overwritten, which empties the caches
// of the weights. Synchronizes with the stream; never called while it is being captured.
void lt_tune(LtDevice& dev, LtPlan& plan, void* y, const void* x, const void* w, void* flush, size_t flush_bytes,
             hipStream_t stream) {
  plan.tuned = true;
  hipblasLtMatmulPreference_t pref = nullptr;
  if (hipblasLtMatmulPreferenceCreate(&pref) != HIPBLAS_STATUS_SUCCESS) return;
  const uint64_t limit = LT_WORKSPACE_BYTES;
  hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &limit, sizeof(limit));
  hipblasLtMatmulHeuristicResult_t found[LT_TUNE_CANDIDATES];
  int count = 0;
  const bool listed = hipblasLtMatmulAlgoGetHeuristic(dev.handle, plan.desc, plan.a, plan.b, plan.d, plan.d, pref,
                                                      LT_TUNE_CANDIDATES, found, &count) == HIPBLAS_STATUS_SUCCESS;
  hipblasLtMatmulPreferenceDestroy(pref);
  hipEvent_t begin = nullptr, end = nullptr;
  if (!listed || hipEventCreate(&begin) != hipSuccess || hipEventCreate(&end) != hipSuccess) {
    if (begin) hipEventDestroy(begin);
    return;
  }
  const float one = 1.0f, zero = 0.0f;
  float best = -1.0f;
  for (int i = 0; i < count; ++i) {
    if (found[i].state != HIPBLAS_STATUS_SUCCESS || found[i].workspaceSize != 0) continue;   // see lt_plan
    float fastest = -1.0f;
    for (int run = 0; run <= LT_TUNE_RUNS; ++run) {         // the first run is not timed
      if (flush && flush_bytes && hipMemsetAsync(flush, run, flush_bytes, stream) != hipSuccess) break;
      hipEventRecord(begin, stream);
      if (hipblasLtMatmul(dev.handle, plan.desc, &one, w, plan.a, x, plan.b, &zero, y, plan.d, y, plan.d, &found[i].algo,
                          dev.workspace, LT_WORKSPACE_BYTES, stream) != HIPBLAS_STATUS_SUCCESS) { fastest = -1.0f; break; }
      hipEventRecord(end, stream);
      if (hipEventSynchronize(end) != hipSuccess) { fastest = -1.0f; break; }
      float ms = 0.0f;
      if (run && hipEventElapsedTime(&ms, begin, end) == hipSuccess && (fastest < 0.0f || ms < fastest)) fastest = ms;
    }
    if (fastest >= 0.0f && (best < 0.0f || fastest < best)) {
      best = fastest;
      plan.algo = found[i].algo;
      plan.workspace = found[i].workspaceSize;
    }
  }
  hipEventDestroy(begin);
  hipEventDestroy(end);
}

// Times the plan's own algorithm and the borrowed ones on the operands of this call (caches as
// they are: products of this many rows are bound by arithmetic) and keeps the fastest.
// Synchronizes with the stream; never called while it is being captured.
void lt_choose(LtDevice& dev, LtPlan& plan, void* y, const void* x, const void* w, hipStream_t stream) {
  const int candidates = plan.borrowed + 1;
  plan.borrowed = 0;
  plan.chosen = true;
  hipEvent_t begin = nullptr, end = nullptr;
  if (hipEventCreate(&begin) != hipSuccess || hipEventCreate(&end) != hipSuccess) {
    if (begin) hipEventDestroy(begin);
    return;
  }
  const float one = 1.0f, zero = 0.0f;
  float best = -1.0f;
  int pick = 0;
  for (int i = 0; i < candidates; ++i) {
    hipblasLtMatmulAlgo_t* algo = i ? &plan.other[i - 1] : &plan.algo;
    float fastest = -1.0f;
    for (int run = 0; run <= LT_TUNE_RUNS; ++run) {         // the first run is not timed
      hipEventRecord(begin, stream);
      if (hipblasLtMatmul(dev.handle, plan.desc, &one, w, plan.a, x, plan.b, &zero, y, plan.d, y, plan.d, algo,
                          dev.workspace, LT_WORKSPACE_BYTES, stream) != HIPBLAS_STATUS_SUCCESS) { fastest = -1.0f; break; }
      hipEventRecord(end, stream);
      if (hipEventSynchronize(end) != hipSuccess) { fastest = -1.0f; break; }
      float ms = 0.0f;
      if (run && hipEventElapsedTime(&ms, begin, end) == hipSuccess && (fastest < 0.0f || ms < fastest)) fastest = ms;
    }
    if (fastest >= 0.0f && (best < 0.0f || fastest < best)) {
      best = fastest;
      pick = i;
    }
  }
  if (pick) {
    plan.algo = plan.other[pick - 1];
    plan.workspace = plan.other_workspace[pick - 1];
  }
  hipEventDestroy(begin);
  hipEventDestroy(end);
}

}  // namespace

// The current device's handle and workspace; made at the first call on the device.
static LtDevice* lt_device() {
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= LT_MAX_DEVICES) return nullptr;
  LtDevice& dev = lt_devices[device];
  if (!dev.handle) {
    if (hipblasLtCreate(&dev.handle) != HIPBLAS_STATUS_SUCCESS) { dev.handle = nullptr; return nullptr; }
    if (hipMalloc(&dev.workspace, LT_WORKSPACE_BYTES) != hipSuccess) {
      hipblasLtDestroy(dev.handle);
      dev.handle = nullptr;
      return nullptr;
    }
  }
  return &dev;
}

// Makes the current device's library handle and workspace (128 MB, kept until the process ends).
// The products below do it themselves at their first call; a caller that will record them into a
// graph calls this beforehand, since memory cannot be allocated while a stream is captured.
extern "C" int ts_gemm_library_init() {
  std::lock_guard<std::mutex> guard(lt_mutex);
  return lt_device() ? TS_OK : TS_LAUNCH_FAILED;
}

// Switches the timing of candidates on or off for the process (see lt_timing); returns what it was.
extern "C" int ts_gemm_library_timing(int on) {
  std::lock_guard<std::mutex> guard(lt_mutex);
  const int was = lt_timing;
  lt_timing = on != 0;
  return was;
}

// The algorithm kept for every shape met so far on the current device, as rows of six numbers:
// M, N, K, 32-bit output or not, how it was chosen (0 the heuristic's first candidate, 1 the fastest
// of the timed candidates, 2 still to be chosen among borrowed ones) and the library's index of the
// solution. Writes at most `capacity` rows; returns how many shapes there are.
extern "C" int ts_gemm_library_choices(int64_t* rows, int capacity) {
  std::lock_guard<std::mutex> guard(lt_mutex);
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= LT_MAX_DEVICES) return 0;
  int n = 0;
  for (auto& kv : lt_devices[device].plans) {
    if (!kv.second.desc) continue;
    if (n < capacity && rows) {
      int64_t* r = rows + 6 * n;
      r[0] = std::get<0>(kv.first);
      r[1] = std::get<1>(kv.first);
      r[2] = std::get<2>(kv.first);
      r[3] = std::get<6>(kv.first);
      r[4] = kv.second.borrowed ? 2 : (kv.second.tuned || kv.second.chosen ? 1 : 0);
      r[5] = hipblaslt_ext::getIndexFromAlgo(kv.second.algo);
    }
    ++n;
  }
  return n;
}

// x, w bfloat16; y bfloat16, or float32 if out_f32 (the 32-bit sums as they are, not rounded to
// bfloat16 on the way); rows of x, w and y are ldx, ldw, ldy elements apart (each at least the row's
// length). The stream may be one that is being captured into a graph (after ts_gemm_library_init).
// tune != 0: a shape of 9 to 256 rows that has not been tuned yet is tuned first (see above),
// unless the stream is being captured; `flush` is device memory of `flush_bytes` that may be
// overwritten (more than the caches hold), or null to time with warm caches.
extern "C" int ts_gemm_library_bf16(void* y, const void* x, const void* w, int M, int N, int K, int64_t ldx,
                                    int64_t ldw, int64_t ldy, int out_f32, int tune, void* flush, size_t flush_bytes,
                                    hipStream_t stream) {
  if (M <= 0 || N <= 0) return TS_OK;
  if (K <= 0 || ldx < K || ldw < K || ldy < N || !y || !x || !w) return TS_BAD_SHAPE;
  std::lock_guard<std::mutex> guard(lt_mutex);
  LtDevice* dev = lt_device();
  if (!dev) return TS_LAUNCH_FAILED;
  LtPlan* plan = lt_plan(*dev, M, N, K, ldx, ldw, ldy, out_f32 != 0);
  if (!plan) return TS_BAD_SHAPE;
  if (lt_timing && tune && !plan->tuned && M >= LT_TUNE_MIN_ROWS && M <= LT_TUNE_MAX_ROWS) {
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &capturing) == hipSuccess && capturing == hipStreamCaptureStatusNone)
      lt_tune(*dev, *plan, y, x, w, flush, flush_bytes, stream);
  }
  if (lt_timing && plan->borrowed) {
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &capturing) == hipSuccess && capturing == hipStreamCaptureStatusNone)
      lt_choose(*dev, *plan, y, x, w, stream);
  }
  const float one = 1.0f, zero = 0.0f;
  const hipblasStatus_t st = hipblasLtMatmul(dev->handle, plan->desc, &one, w, plan->a, x, plan->b, &zero, y, plan->d, y,
                                             plan->d, &plan->algo, dev->workspace, LT_WORKSPACE_BYTES, stream);
  return st == HIPBLAS_STATUS_SUCCESS ? TS_OK : TS_LAUNCH_FAILED;
}
