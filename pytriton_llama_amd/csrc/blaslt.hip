// The library matrix product for the many rows of a prompt: y = x W^T through hipBLASLt,
// called directly (the reference runs its projections through cuBLAS by way of nn.Linear,
// lite_llama/models/llama.py:37-40,61,120,221).
//
// Why not through torch: its linear() asks the library for an algorithm on every call and
// takes about 20 us on the host, more than most of the kernels it launches; a prompt portion
// then runs at the speed of the host. Here the descriptors and the algorithm of a shape are
// made once and kept, and a call is a table look-up and hipblasLtMatmul (3 to 4 us).
//
// The algorithm: the library proposes several for a shape, best first by its own estimate, and a
// shape runs the first unless the caller asks for timing. The estimate is right for the 2,048
// rows of a prompt at the 1B widths (timed in place, no later proposal beats the first) and off
// for some shapes of large decoding batches (64 rows, depth 8,192, 2,048 columns: the seventh
// proposal takes 12.7 us, the first 17.5). Timing a shape costs about two hundred runs of its
// product and a wait for the stream, which only a shape that comes back thousands of times
// repays: the steps that are recorded as graphs. So the recorder switches the timing on for its
// warm-up pass (ptl_blaslt_set_tuning), where the first call of a shape not yet timed runs the
// proposals on the caller's own operands and keeps the fastest; everywhere else, and always while
// the stream is being captured, nothing is timed. All proposals are asked for when the plan is
// made: asked again later, the library answers from what it gave the first time.
// PTL_BLASLT_LOG=1 in the environment prints what the timing found, PTL_BLASLT_NO_TUNING=1 keeps
// the library's first proposal everywhere.
#include "common.h"
#include <hipblaslt/hipblaslt.h>
#include <cstdio>
#include <cstdlib>
#include <map>
#include <mutex>
#include <tuple>
#include <vector>

namespace {

constexpr size_t WORKSPACE_BYTES = 64u << 20;
// Plans kept at most. Steps replayed as graphs meet a few dozen shapes; steps launched kernel by
// kernel bring a new M with every prompt length, so the table is emptied when it is full (the
// library is only read at call time: a plan may go once its call has returned).
constexpr size_t MAX_PLANS = 1024;
constexpr int TUNE_PROPOSALS = 12;
constexpr int TUNE_REPEATS = 8;
constexpr float TUNE_MARGIN = 0.95f;
constexpr size_t MAX_TUNED = 256;

struct Plan {
  hipblasLtMatmulDesc_t desc = nullptr;
  hipblasLtMatrixLayout_t a = nullptr, b = nullptr, c = nullptr;
  std::vector<hipblasLtMatmulHeuristicResult_t> proposals;   // the library's, in its order
  int chosen = 0;                                 // the one that is run
  bool tuned = false;                             // timed, or given up: not tried again
};

// (M, N, K, ldx, ldy, output type)
using Key = std::tuple<int, int, int, long, long, int>;

struct State {
  hipblasLtHandle_t handle = nullptr;
  void* workspace = nullptr;
  std::map<Key, Plan> plans;
  size_t tuned = 0;
  bool tuning = false;
  hipEvent_t t0 = nullptr, t1 = nullptr;
  std::mutex lock;
};

State& state() {
  static State s;
  return s;
}

bool ok(hipblasStatus_t st) { return st == HIPBLAS_STATUS_SUCCESS; }

void drop_plan(Plan& p) {
  if (p.a) hipblasLtMatrixLayoutDestroy(p.a);
  if (p.b) hipblasLtMatrixLayoutDestroy(p.b);
  if (p.c) hipblasLtMatrixLayoutDestroy(p.c);
  if (p.desc) hipblasLtMatmulDescDestroy(p.desc);
  p = Plan();
}

hipblasStatus_t run_algo(State& s, const Plan& p, const hipblasLtMatmulAlgo_t& algo, void* y, const void* x,
                         const void* w, hipStream_t stream) {
  const float one = 1.0f, zero = 0.0f;
  return hipblasLtMatmul(s.handle, p.desc, &one, w, p.a, x, p.b, &zero, y, p.c, y, p.c, &algo, s.workspace,
                         WORKSPACE_BYTES, stream);
}

bool propose(State& s, Plan& p) {
  hipblasLtMatmulPreference_t pref = nullptr;
  if (!ok(hipblasLtMatmulPreferenceCreate(&pref))) return false;
  const uint64_t ws = WORKSPACE_BYTES;
  hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &ws, sizeof(ws));
  hipblasLtMatmulHeuristicResult_t found[TUNE_PROPOSALS];
  int n = 0;
  const hipblasStatus_t st = hipblasLtMatmulAlgoGetHeuristic(s.handle, p.desc, p.a, p.b, p.c, p.c, pref,
                                                             TUNE_PROPOSALS, found, &n);
  hipblasLtMatmulPreferenceDestroy(pref);
  if (!ok(st)) return false;
  for (int i = 0; i < n; ++i)
    if (found[i].workspaceSize <= WORKSPACE_BYTES) p.proposals.push_back(found[i]);
  return !p.proposals.empty();
}

// Times the proposals on the caller's operands (y is overwritten with the same product each time)
// and chooses the fastest. Any failure leaves the choice that p has.
void tune_plan(State& s, Plan& p, const Key& key, void* y, const void* x, const void* w, hipStream_t stream) {
  hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &capturing) != hipSuccess) {
    (void)hipGetLastError();
    return;
  }
  if (capturing != hipStreamCaptureStatusNone) return;            // nothing that waits: a later call may
  p.tuned = true;
  const int found = (int)p.proposals.size();
  if (found < 2 || s.tuned >= MAX_TUNED) return;
  ++s.tuned;
  const auto& proposals = p.proposals;
  if (!s.t0 && (hipEventCreate(&s.t0) != hipSuccess || hipEventCreate(&s.t1) != hipSuccess)) {
    (void)hipGetLastError();
    s.t0 = s.t1 = nullptr;
    return;
  }
  static const bool log = getenv("PTL_BLASLT_LOG") != nullptr;
  float times[TUNE_PROPOSALS];
  for (int i = 0; i < found; ++i) times[i] = -1.f;
  // two passes over the proposals, the lower time of each counts: the clocks rise during the first
  for (int pass = 0; pass < 2; ++pass) {
    for (int i = 0; i < found; ++i) {
      if (pass == 1 && times[i] < 0.f) continue;
      if (!ok(run_algo(s, p, proposals[i].algo, y, x, w, stream))) continue;    // (also warms it up)
      if (hipEventRecord(s.t0, stream) != hipSuccess) return;
      bool fine = true;
      for (int r = 0; r < TUNE_REPEATS && fine; ++r) fine = ok(run_algo(s, p, proposals[i].algo, y, x, w, stream));
      if (hipEventRecord(s.t1, stream) != hipSuccess || hipEventSynchronize(s.t1) != hipSuccess) return;
      float ms = 0.f;
      if (!fine || hipEventElapsedTime(&ms, s.t0, s.t1) != hipSuccess) continue;
      if (times[i] < 0.f || ms < times[i]) times[i] = ms;
    }
  }
  // the library's first stays unless another is clearly faster (the operands are warm in the
  // caches here and cold in a step: a few per cent say nothing)
  float best = times[0] >= 0.f ? times[0] * TUNE_MARGIN : -1.f;
  int best_i = 0;
  for (int i = 1; i < found; ++i)
    if (times[i] >= 0.f && (best < 0.f || times[i] < best)) { best = times[i]; best_i = i; }
  if (log) {
    fprintf(stderr, "[blaslt] %d rows, %d columns, depth %d:", std::get<0>(key), std::get<1>(key), std::get<2>(key));
    for (int i = 0; i < found; ++i) fprintf(stderr, " %.1f", times[i] * 1e3f / TUNE_REPEATS);
    fprintf(stderr, " us -> proposal %d\n", best_i);
  }
  if (best >= 0.f) p.chosen = best_i;
}

int make_plan(State& s, Plan& p, int M, int N, int K, long ldx, long ldy, int out_dtype) {
  // Column-major view: y^T [N, M] = W [N, K] x^T [K, M]. W lies as a K x N column-major
  // matrix (leading dimension K) and is transposed; x as K x M (leading dimension ldx).
  const hipDataType out_type = out_dtype == PTL_DTYPE_F32 ? HIP_R_32F : HIP_R_16BF;
  const hipblasOperation_t tr = HIPBLAS_OP_T, no = HIPBLAS_OP_N;
  if (!ok(hipblasLtMatmulDescCreate(&p.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F)) ||
      !ok(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &tr, sizeof(tr))) ||
      !ok(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &no, sizeof(no))) ||
      !ok(hipblasLtMatrixLayoutCreate(&p.a, HIP_R_16BF, K, N, K)) ||
      !ok(hipblasLtMatrixLayoutCreate(&p.b, HIP_R_16BF, K, M, ldx)) ||
      !ok(hipblasLtMatrixLayoutCreate(&p.c, out_type, N, M, ldy)))
    return PTL_ERR_LAUNCH;
  return propose(s, p) ? PTL_OK : PTL_ERR_ARG;
}

hipblasStatus_t run(State& s, const Plan& p, void* y, const void* x, const void* w, hipStream_t stream) {
  return run_algo(s, p, p.proposals[p.chosen].algo, y, x, w, stream);
}

}  // namespace

// on != 0: from now on the first call of a shape that was not timed yet times the library's
// proposals for it (at most TUNE_PROPOSALS) and keeps the fastest; 0: shapes keep what they have
// and new ones run the library's first proposal. For the warm-up pass before a graph is recorded.
extern "C" void ptl_blaslt_set_tuning(int on) {
  State& s = state();
  std::lock_guard<std::mutex> guard(s.lock);
  s.tuning = on != 0 && getenv("PTL_BLASLT_NO_TUNING") == nullptr;
}

// y [M, N] (row stride ldy; bfloat16 or float32) = x [M, K] (bfloat16, row stride ldx) W^T,
// W [N, K] bfloat16 with dense rows. Rows of x and W 16-byte aligned.
extern "C" int ptl_blaslt_gemm_bf16(void* y, const void* x, const void* w, int M, int N, int K,
                                    long ldx, long ldy, int out_dtype, hipStream_t stream) {
  if (M <= 0 || N <= 0) return PTL_OK;
  if (K <= 0 || ldx < K || ldy < N || (out_dtype != PTL_DTYPE_F32 && out_dtype != PTL_DTYPE_BF16))
    return PTL_ERR_ARG;
  State& s = state();
  std::lock_guard<std::mutex> guard(s.lock);
  if (s.handle == nullptr) {
    // the one allocation of these libraries: the library's workspace, at the first call.
    // Handle and workspace are kept together or not at all, so a call after a failure tries again
    hipblasLtHandle_t handle = nullptr;
    void* workspace = nullptr;
    if (!ok(hipblasLtCreate(&handle))) return PTL_ERR_LAUNCH;
    if (hipMalloc(&workspace, WORKSPACE_BYTES) != hipSuccess) {
      (void)hipGetLastError();
      hipblasLtDestroy(handle);
      return PTL_ERR_LAUNCH;
    }
    s.handle = handle;
    s.workspace = workspace;
  }
  const Key key(M, N, K, ldx, ldy, out_dtype);
  auto it = s.plans.find(key);
  if (it == s.plans.end()) {
    if (s.plans.size() >= MAX_PLANS) {
      for (auto& kv : s.plans) drop_plan(kv.second);
      s.plans.clear();
    }
    Plan p;
    const int rc = make_plan(s, p, M, N, K, ldx, ldy, out_dtype);
    if (rc != PTL_OK) {
      drop_plan(p);
      return rc;
    }
    it = s.plans.emplace(key, p).first;
  }
  Plan& plan = it->second;
  if (s.tuning && !plan.tuned) tune_plan(s, plan, key, y, x, w, stream);
  return ok(run(s, plan, y, x, w, stream)) ? PTL_OK : PTL_ERR_LAUNCH;
}
