// Plain bfloat16 matrix products with many rows through the GEMM library (hipBLASLt),
// called directly: the reference sends every projection to its vendor's library too
// (/root/reference/src/matmul/root.zig:292-313 calls cuBLAS).
//
//   y [M, N] = x [M, K] . w [N, K]^T          bfloat16 in, 32-bit sums, bfloat16 or
//                                              32-bit out
//   y [P, M, N] (32-bit) with K cut into P ranges, as one batched product: partial
//                                              sums that the consumer adds up
//   y [M, N] (32-bit) += x . w^T               the product added to what y holds (the
//                                              residual stream), the library's beta = 1
//
// No device code here.  What a call costs on the host matters for steps of a few
// hundred tokens, which issue some sixty of these products: the descriptors and the
// algorithm the library's heuristic names for a shape are made once per (device,
// M, N, K, output type, P) and kept, so a later call is one hipblasLtMatmul, or, for
// operands seen before, one launch of a prepared instance (see InstanceKey).
// The same shape therefore always runs the same kernel, recorded in a graph or not.
//
// Which algorithm: the heuristic's first answer is not always the fastest on this GPU
// (measured, bfloat16 out, weights from memory: 2,048 rows on [2048, 8192] weights 88 us with
// the first answer, 76 with the eighteenth; on [2048, 2048] 29 against 25; 64 rows on
// [3072, 2048] 15.4 against 9.0, on [6144, 2048] 13.5 against 11.0), so with `tune` the first
// call of a shape times the first TUNE_CANDIDATES answers on the call's own operands and
// keeps the fastest.  In a model every weight comes from memory: the timed runs take turns
// over copies of the weight, so that a run's weights do not lie in a cache (timed warm, the
// ranking is another one: a decode step of 64 rows got slower), and they are issued behind a
// copy that keeps the GPU busy meanwhile, so that they run back to back and the kernels are
// timed, not the host's calls.  Shapes whose row counts fall into the same block (of
// TUNE_BUCKET rows from TUNE_BUCKET rows on, between two powers of two below) share the
// choice where the heuristic names a block's winner for them too, and at most TUNE_PER_BLOCK
// row counts of a block are timed themselves, so a server that sees every batch size and
// portion length times some dozens of shapes, 10 to 60 ms each, not thousands.  (Naming the winner to the library by its index
// for a new row count of a block, instead of looking for it among the heuristic's answers
// for that row count, cost 300 ms at its first use.)  Which answer wins can differ from run
// to run when two are close: callers that want the same bits run after run pass tune = 0
// and get the first answer.  ZIG_AI_GEMM_TUNE_LOG=1 prints a line for every shape timed.
#include <hip/hip_runtime.h>
#include <hipblaslt/hipblaslt-ext.hpp>
#include <hipblaslt/hipblaslt.h>

#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <map>
#include <memory>
#include <mutex>
#include <string>
#include <tuple>
#include <vector>

#include "common.h"

#define ZA_API extern "C" __attribute__((visibility("default")))

namespace {

struct Plan {
  hipblasLtMatmulDesc_t op = nullptr;
  hipblasLtMatrixLayout_t a = nullptr, b = nullptr, c = nullptr;
  hipblasLtMatmulAlgo_t algo;
  size_t workspace = 0;
  bool usable = false;
  bool settled = true;   // false: the candidates are still to be timed
  std::vector<hipblasLtMatmulHeuristicResult_t> candidates;
};

constexpr int OUT_BF16 = 0, OUT_F32 = 1, OUT_ADDED = 2;   // what y is: see the head of this file

constexpr int TUNE_MIN_ROWS = 17;      // (up to 16 rows this package's own kernels run)
constexpr size_t TUNE_MIN_WEIGHT = (size_t)1 << 19;   // elements: a megabyte of bfloat16; below, nothing to gain
constexpr int TUNE_BUCKET = 256;
constexpr int TUNE_CANDIDATES = 24;
constexpr size_t TUNE_PER_BLOCK = 4;     // row counts of one block that are timed themselves
constexpr size_t TUNE_COPY_BYTES = (size_t)512 << 20;    // room for copies of a weight

bool tune_log() {
  static const bool on = [] {
    const char* v = std::getenv("ZIG_AI_GEMM_TUNE_LOG");
    return v && v[0] == '1';
  }();
  return on;
}

int tune_block(int M) {
  if (M >= TUNE_BUCKET) return 16 + (M + TUNE_BUCKET - 1) / TUNE_BUCKET;
  int block = 0;
  while ((1 << block) < M) ++block;
  return block;
}

using Key = std::tuple<int, int, int, int, int, int, int>;   // device, M, N, K, output type, P, tune
// device, block of rows, N, K, output type, P -> the library's indices of the algorithms that won
using TunedKey = std::tuple<int, int, int, int, int, int>;

// A product on given operands, with its kernel arguments made: issuing it again is one
// launch (some 6 us less on the host than hipblasLtMatmul, which derives the arguments
// at every call; making an instance costs some 12 us more than one such call).  Steps of
// the same shape get the same addresses from the tensor library's allocator, so the
// products of a loop over equal steps (portions of a long prompt, decode batches that
// are not replayed from a graph) are found again.  An instance is made when a shape and
// its operands are seen for the second time (an entry without one marks the first); a
// table that has grown to max_instances() is emptied, after the device has finished what
// was issued.
using InstanceKey = std::tuple<Key, const void*, const void*, void*, void*>;   // shape, x, w, y, workspace
// (ZIG_AI_GEMM_INSTANCES overrides the size of the table; 0 switches the instances off)
size_t max_instances() {
  static const size_t limit = [] {
    const char* v = std::getenv("ZIG_AI_GEMM_INSTANCES");
    return v ? (size_t)std::strtoul(v, nullptr, 10) : (size_t)8192;
  }();
  return limit;
}

std::mutex g_lock;
std::map<int, hipblasLtHandle_t> g_handles;
std::map<Key, Plan> g_plans;
std::map<TunedKey, std::vector<int>> g_tuned;   // a block's winners, the first timed first
std::map<InstanceKey, std::unique_ptr<hipblaslt_ext::Gemm>> g_instances;
const float kOne = 1.0f, kZero = 0.0f;
thread_local std::string g_error;

int fail(int code, const std::string& what) {
  g_error = what;
  return code;
}

bool ok(hipblasStatus_t s, const char* what, std::string* why) {
  if (s == HIPBLAS_STATUS_SUCCESS) return true;
  *why = std::string(what) + " failed with hipBLAS status " + std::to_string((int)s);
  return false;
}

// Column-major terms: y^T (N x M, leading dimension N) = w (stored K x N, transposed)
// times x^T (stored K x M).  A range p of K starts p * K/P elements into a row of
// either operand; its result is the p-th [M, N] block of y.
bool make_plan(hipblasLtHandle_t handle, int M, int N, int K, int out_kind, int P,
               size_t workspace_bytes, bool tune, Plan* plan, std::string* why) {
  const int kp = K / P;
  const hipDataType out_type = out_kind != OUT_BF16 ? HIP_R_32F : HIP_R_16BF;
  if (!ok(hipblasLtMatmulDescCreate(&plan->op, HIPBLAS_COMPUTE_32F, HIP_R_32F), "MatmulDescCreate", why))
    return false;
  const int32_t ta = HIPBLAS_OP_T, tb = HIPBLAS_OP_N;
  if (!ok(hipblasLtMatmulDescSetAttribute(plan->op, HIPBLASLT_MATMUL_DESC_TRANSA, &ta, sizeof(ta)),
          "set TRANSA", why) ||
      !ok(hipblasLtMatmulDescSetAttribute(plan->op, HIPBLASLT_MATMUL_DESC_TRANSB, &tb, sizeof(tb)),
          "set TRANSB", why))
    return false;
  if (!ok(hipblasLtMatrixLayoutCreate(&plan->a, HIP_R_16BF, kp, N, K), "layout of w", why) ||
      !ok(hipblasLtMatrixLayoutCreate(&plan->b, HIP_R_16BF, kp, M, K), "layout of x", why) ||
      !ok(hipblasLtMatrixLayoutCreate(&plan->c, out_type, N, M, N), "layout of y", why))
    return false;
  if (P > 1) {
    const int32_t count = P;
    const int64_t in_stride = kp, out_stride = (int64_t)M * N;
    hipblasLtMatrixLayout_t layouts[3] = {plan->a, plan->b, plan->c};
    for (int i = 0; i < 3; ++i) {
      const int64_t stride = i < 2 ? in_stride : out_stride;
      if (!ok(hipblasLtMatrixLayoutSetAttribute(layouts[i], HIPBLASLT_MATRIX_LAYOUT_BATCH_COUNT, &count,
                                                sizeof(count)), "set batch count", why) ||
          !ok(hipblasLtMatrixLayoutSetAttribute(layouts[i], HIPBLASLT_MATRIX_LAYOUT_STRIDED_BATCH_OFFSET,
                                                &stride, sizeof(stride)), "set batch stride", why))
        return false;
    }
  }
  hipblasLtMatmulPreference_t pref = nullptr;
  if (!ok(hipblasLtMatmulPreferenceCreate(&pref), "PreferenceCreate", why)) return false;
  const uint64_t limit = workspace_bytes;
  static const int tune_candidates = [] {    // (ZIG_AI_GEMM_TUNE_CANDIDATES: for comparisons)
    const char* v = std::getenv("ZIG_AI_GEMM_TUNE_CANDIDATES");
    const int n = v ? std::atoi(v) : 0;
    return n > 0 && n <= 512 ? n : TUNE_CANDIDATES;
  }();
  const int wanted = tune ? tune_candidates : 1;
  std::vector<hipblasLtMatmulHeuristicResult_t> found(wanted);
  int n_found = 0;
  bool good = ok(hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES,
                                                       &limit, sizeof(limit)), "set workspace limit", why) &&
              ok(hipblasLtMatmulAlgoGetHeuristic(handle, plan->op, plan->a, plan->b, plan->c, plan->c, pref,
                                                 wanted, found.data(), &n_found), "AlgoGetHeuristic", why);
  hipblasLtMatmulPreferenceDestroy(pref);
  if (!good) return false;
  if (n_found < 1 || found[0].state != HIPBLAS_STATUS_SUCCESS || found[0].workspaceSize > workspace_bytes) {
    *why = "the library names no algorithm for this shape";
    return true;   // a plan that is not usable: the caller takes another kernel
  }
  plan->algo = found[0].algo;
  plan->workspace = found[0].workspaceSize;
  plan->usable = true;
  if (tune) {
    for (int i = 0; i < n_found; ++i)
      if (found[i].state == HIPBLAS_STATUS_SUCCESS && found[i].workspaceSize <= workspace_bytes)
        plan->candidates.push_back(found[i]);
    plan->settled = plan->candidates.size() < 2;
  }
  return true;
}

// Times the plan's candidates on the call's operands (y is overwritten by every one of
// them, and by the product proper afterwards) and returns the fastest: one run to load
// the kernel, then TUNE_RUNS timed ones.  In a model a product's weights come from
// memory, so the timed runs take turns over copies of the weight made for the occasion
// (as many as fit TUNE_COPY_BYTES, at most TUNE_COPIES; the weight itself is one of the
// turns): a run's weights were last touched several runs ago and have left the caches.
// (Clearing a large buffer before every run instead left its write-backs in the timed
// run's way and ranked the candidates differently from a loop over many weights.)  The
// stream is waited for; this happens once per block of row counts.  A candidate that
// fails is out.
// The timed runs of a candidate are issued behind a copy that keeps the GPU busy for as
// long as the host needs to issue them (some 8 us a call): they then run back to back, and
// what is timed is the kernels, not the host (a product of a few microseconds, timed as
// fast as the host could issue it, looked the same with every candidate: [1024, 1024] at
// 24 to 64 rows 8.1 to 8.9 us for twenty of twenty-four, where the kernels take 5.6 to 11).
constexpr int TUNE_RUNS = 8;
constexpr int TUNE_COPIES = 7;
constexpr size_t TUNE_BACKLOG_BYTES = (size_t)128 << 20;   // copied twice: some 100 us
int fastest_candidate(hipblasLtHandle_t handle, const Plan& plan, const void* x, const void* w,
                      size_t weight_bytes, void* y, size_t added_bytes, void* workspace,
                      size_t workspace_bytes, hipStream_t stream) {
  // a product that is added to y is timed on a y of its own (`added_bytes` of it, zero at
  // first): the caller's holds what the product proper is to be added to
  const float* beta = added_bytes ? &kOne : &kZero;
  struct Release {
    void* p;
    ~Release() { if (p) (void)hipFree(p); }
  };
  void* own_y = nullptr;
  if (added_bytes) {
    if (hipMalloc(&own_y, added_bytes) != hipSuccess ||
        hipMemsetAsync(own_y, 0, added_bytes, stream) != hipSuccess) {
      (void)hipGetLastError();
      if (own_y) (void)hipFree(own_y);
      return 0;                   // no room: the first answer
    }
    y = own_y;
  }
  Release release_y{own_y};
  int copies = (int)(TUNE_COPY_BYTES / weight_bytes);
  if (copies > TUNE_COPIES) copies = TUNE_COPIES;
  char* room = nullptr;
  if (copies > 0 && hipMalloc((void**)&room, (size_t)copies * weight_bytes) != hipSuccess) {
    (void)hipGetLastError();
    copies = 0;                   // no room: every run on the weight itself
  }
  Release release{room};
  for (int c = 0; c < copies; ++c)
    if (hipMemcpyAsync(room + (size_t)c * weight_bytes, w, weight_bytes, hipMemcpyDeviceToDevice,
                       stream) != hipSuccess) {
      (void)hipGetLastError();
      copies = c;
      break;
    }
  hipEvent_t t0 = nullptr, t1 = nullptr;
  if (hipEventCreate(&t0) != hipSuccess || hipEventCreate(&t1) != hipSuccess) {
    if (t0) (void)hipEventDestroy(t0);
    (void)hipGetLastError();
    (void)hipStreamSynchronize(stream);
    return 0;
  }
  char* backlog = nullptr;
  static const bool host_paced = [] {       // (ZIG_AI_GEMM_TUNE_HOST_PACED=1: for comparisons)
    const char* v = std::getenv("ZIG_AI_GEMM_TUNE_HOST_PACED");
    return v && v[0] == '1';
  }();
  if (host_paced) {
  } else if (hipMalloc((void**)&backlog, 2 * TUNE_BACKLOG_BYTES) != hipSuccess) {
    (void)hipGetLastError();
    backlog = nullptr;            // no room: the runs are timed as the host issues them
  }
  Release release_backlog{backlog};
  auto keep_busy = [&]() {
    if (!backlog) return;
    (void)hipMemcpyAsync(backlog + TUNE_BACKLOG_BYTES, backlog, TUNE_BACKLOG_BYTES,
                         hipMemcpyDeviceToDevice, stream);
    (void)hipMemcpyAsync(backlog, backlog + TUNE_BACKLOG_BYTES, TUNE_BACKLOG_BYTES,
                         hipMemcpyDeviceToDevice, stream);
  };
  int turn = 0;
  auto next_weight = [&]() -> const void* {
    const int c = turn++ % (copies + 1);
    return c == copies ? w : (const void*)(room + (size_t)c * weight_bytes);
  };
  int best = 0;
  float best_ms = -1.f;
  {
    // (the clocks come up under the first runs: the first candidate is not to pay for that)
    hipblasLtMatmulAlgo_t algo = plan.candidates[0].algo;
    for (int r = 0; r < 4; ++r)
      (void)hipblasLtMatmul(handle, plan.op, &kOne, next_weight(), plan.a, x, plan.b, beta, y, plan.c,
                            y, plan.c, &algo, workspace, workspace_bytes, stream);
  }
  for (size_t i = 0; i < plan.candidates.size(); ++i) {
    hipblasLtMatmulAlgo_t algo = plan.candidates[i].algo;
    auto run = [&]() {
      return hipblasLtMatmul(handle, plan.op, &kOne, next_weight(), plan.a, x, plan.b, beta, y,
                             plan.c, y, plan.c, &algo, workspace, workspace_bytes,
                             stream) == HIPBLAS_STATUS_SUCCESS;
    };
    float ms = 0.f;
    bool fine = run();
    keep_busy();
    fine = fine && hipEventRecord(t0, stream) == hipSuccess;
    for (int r = 0; r < TUNE_RUNS && fine; ++r) fine = run();
    fine = fine && hipEventRecord(t1, stream) == hipSuccess && hipEventSynchronize(t1) == hipSuccess &&
           hipEventElapsedTime(&ms, t0, t1) == hipSuccess;
    if (!fine) {
      (void)hipGetLastError();
      continue;
    }
    ms /= TUNE_RUNS;
    if (tune_log())
      fprintf(stderr, "[zig_ai_amd]   answer %zu (the library's index %d): %.1f us\n", i,
              hipblaslt_ext::getIndexFromAlgo(algo), ms * 1e3f);
    if (best_ms < 0.f || ms < best_ms) {
      best_ms = ms;
      best = (int)i;
    }
  }
  (void)hipEventDestroy(t0);
  (void)hipEventDestroy(t1);
  return best;
}

}  // namespace

ZA_API const char* za_lt_last_error() { return g_error.c_str(); }

// Returns 0, ZA_ERR_ARG, ZA_ERR_UNSUPPORTED (the library has no algorithm for the
// shape: nothing was launched) or a positive hipBLAS status.
// `tune`: see the head of this file.
// `out_kind`: 0 bfloat16, 1 32-bit, 2 32-bit added to what y holds (P = 1).
ZA_API int za_lt_matmul(const void* x, const void* w, void* y, int M, int N, int K, int out_kind,
                        int P, int tune, void* workspace, size_t workspace_bytes,
                        hipStream_t stream) {
  if (!x || !w || !y || M < 1 || N < 1 || K < 1 || P < 1 || K % P || out_kind < OUT_BF16 ||
      out_kind > OUT_ADDED || (P > 1 && out_kind != OUT_F32))
    return fail(ZA_ERR_ARG, "za_lt_matmul: bad argument");
  const float* beta = out_kind == OUT_ADDED ? &kOne : &kZero;
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess) return fail(ZA_ERR_ARG, "za_lt_matmul: no current device");
  Plan plan;
  hipblasLtHandle_t handle = nullptr;
  {
    std::lock_guard<std::mutex> guard(g_lock);
    auto h = g_handles.find(device);
    if (h == g_handles.end()) {
      hipblasLtHandle_t made = nullptr;
      const hipblasStatus_t s = hipblasLtCreate(&made);
      if (s != HIPBLAS_STATUS_SUCCESS) return fail((int)s, "hipblasLtCreate failed");
      h = g_handles.emplace(device, made).first;
    }
    handle = h->second;
    const bool tuning = tune && M >= TUNE_MIN_ROWS && (size_t)N * K >= TUNE_MIN_WEIGHT;
    const Key key(device, M, N, K, out_kind, P, tuning ? 1 : 0);
    auto it = g_plans.find(key);
    if (it == g_plans.end()) {
      Plan made;
      std::string why;
      if (!make_plan(handle, M, N, K, out_kind, P, workspace_bytes, tuning, &made, &why))
        return fail(ZA_ERR_ARG, "za_lt_matmul: " + why);
      it = g_plans.emplace(key, made).first;
    }
    Plan& kept = it->second;
    if (kept.usable && !kept.settled) {
      const TunedKey block(device, tune_block(M), N, K, out_kind, P);
      auto choose = [&](size_t i) {
        kept.algo = kept.candidates[i].algo;
        kept.workspace = kept.candidates[i].workspaceSize;
      };
      hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
      const bool recording = hipStreamIsCapturing(stream, &capturing) != hipSuccess ||
                             capturing != hipStreamCaptureStatusNone;
      // Neighbouring row counts that have been timed: the winner of one of them, the one
      // timed last first, if it is among this shape's answers.  The heuristic does not
      // give every row count of a block the same answers (64 rows on [1024, 1024] lack
      // what wins at 48 rows, and the first answer takes twice as long): a row count
      // without any of the block's winners is timed itself, up to TUNE_PER_BLOCK a block;
      // beyond that the first answer stays.
      std::vector<int>& winners = g_tuned[block];
      bool found = false;
      for (size_t wi = winners.size(); wi-- > 0 && !found;)
        for (size_t i = 0; i < kept.candidates.size() && !found; ++i)
          if (hipblaslt_ext::getIndexFromAlgo(kept.candidates[i].algo) == winners[wi]) {
            choose(i);
            found = true;
          }
      if (!found && !recording && winners.size() < TUNE_PER_BLOCK) {
        const auto began = std::chrono::steady_clock::now();
        const int best = fastest_candidate(handle, kept, x, w, (size_t)N * K * sizeof(uint16_t), y,
                                           out_kind == OUT_ADDED ? (size_t)M * N * sizeof(float) : 0,
                                           workspace, workspace_bytes, stream);
        choose((size_t)best);
        if (tune_log())
          fprintf(stderr, "[zig_ai_amd] timed %zu candidates for M=%d N=%d K=%d P=%d %s: answer %d in %.1f ms\n",
                  kept.candidates.size(), M, N, K, P,
                  out_kind == OUT_ADDED ? "added to f32" : out_kind == OUT_F32 ? "f32" : "bf16", best,
                  std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - began).count());
        winners.push_back(hipblaslt_ext::getIndexFromAlgo(kept.algo));
      }
      // (a shape first met while a stream is recorded keeps the first answer for good:
      // the same shape always runs the same kernel)
      kept.settled = true;
      kept.candidates.clear();
      kept.candidates.shrink_to_fit();
    }
    plan = kept;
  }
  if (!plan.usable || plan.workspace > workspace_bytes)
    return fail(ZA_ERR_UNSUPPORTED, "za_lt_matmul: the library names no algorithm for this shape");
  hipblaslt_ext::Gemm* instance = nullptr;
  {
    std::lock_guard<std::mutex> guard(g_lock);
    const InstanceKey ikey(Key(device, M, N, K, out_kind, P,
                               tune && M >= TUNE_MIN_ROWS && (size_t)N * K >= TUNE_MIN_WEIGHT ? 1 : 0),
                           x, w, y, workspace);
    auto it = g_instances.find(ikey);
    if (it == g_instances.end()) {
      if (g_instances.size() >= max_instances()) {
        // Instances may own memory that products already issued still read: the table is
        // emptied only once the device has finished them, and never while a stream is
        // being recorded (then it simply stays full until the next call outside).
        hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(stream, &capturing) == hipSuccess &&
            capturing == hipStreamCaptureStatusNone && hipDeviceSynchronize() == hipSuccess)
          g_instances.clear();
      }
      if (g_instances.size() < max_instances()) g_instances.emplace(ikey, nullptr);   // seen once
    } else {
      if (!it->second) {
        std::unique_ptr<hipblaslt_ext::Gemm> made(new hipblaslt_ext::Gemm(
            handle, plan.op, &kOne, w, plan.a, x, plan.b, beta, y, plan.c, y, plan.c));
        hipblasLtMatmulAlgo_t algo = plan.algo;
        if (made->initialize(algo, workspace) == HIPBLAS_STATUS_SUCCESS) it->second = std::move(made);
      }
      instance = it->second.get();                 // null: the plain call below
    }
  }
  const hipblasStatus_t s =
      instance ? instance->run(stream)
               : hipblasLtMatmul(handle, plan.op, &kOne, w, plan.a, x, plan.b, beta, y, plan.c, y,
                                 plan.c, &plan.algo, workspace, workspace_bytes, stream);
  if (s != HIPBLAS_STATUS_SUCCESS)
    return fail((int)s > 0 ? (int)s : ZA_ERR_ARG,
                "the library's product failed with hipBLAS status " + std::to_string((int)s));
  return 0;
}
