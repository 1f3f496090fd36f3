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
// call runs the first unless it asks for the timed choice (use_timed). The estimate is right for
// the 2,048 rows of a prompt at the 1B widths (timed in place, no later proposal beats the first)
// and off for some shapes of large decoding batches (64 rows, depth 8,192, 2,048 columns: the
// seventh proposal takes 12.7 us, the first 17.5). Timing a shape costs about two hundred runs of
// its product and a wait for the stream, which only a shape that comes back thousands of times
// repays: the steps that are recorded as graphs. So only the recorder asks for the timed choice
// (in its warm-up pass, where the first such call of a shape runs the proposals on the caller's
// own operands, and in the recording itself, where nothing is timed and the kept choice runs);
// every other call runs the library's first proposal, before and after a recording alike.
// Another proposal than the first is kept only if it is clearly faster and if its result on the
// caller's operands agrees with the first proposal's (within the rounding of the output type:
// proposals add in different orders, so bfloat16 results may differ by an ulp); one that
// disagrees is never run again. Which proposal wins a timing can change from process to process,
// and with it the last bit of a recorded step's results: a caller that wants the same bits in
// every process never asks for the timed choice. All proposals are asked for when the plan is
// made: asked again later, the library answers from what it gave the first time.
// PTL_BLASLT_LOG=1 in the environment prints what the timing found, PTL_BLASLT_NO_TUNING=1 keeps
// the library's first proposal everywhere.
#include "common.h"
#include <hipblaslt/hipblaslt.h>
#include <algorithm>
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
// Shapes timed at most (each stays in the table for good). 48 portion buckets of five products
// and the decode buckets make about 260 for one runner.
constexpr size_t MAX_TIMED = 768;

struct Plan {
  hipblasLtMatmulDesc_t desc = nullptr;
  hipblasLtMatrixLayout_t a = nullptr, b = nullptr, c = nullptr;
  std::vector<hipblasLtMatmulHeuristicResult_t> proposals;   // the library's, in its order
  int timed_choice = 0;                           // what a call that asks for the timed choice runs
  bool timed = false;                             // timed, or given up: not tried again
};

// (M, N, K, ldx, ldy, output type)
using Key = std::tuple<int, int, int, long, long, int>;

struct State {
  hipblasLtHandle_t handle = nullptr;
  void* workspace = nullptr;
  std::map<Key, Plan> plans;
  size_t timed = 0;
  bool said_full = false;
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

// check[0]: the largest |ref| as float bits; check[1]: elements of got that differ from ref by more
// than 2^-6 of the larger of the two plus 2^-10 of the largest |ref| (two right proposals differ
// by the rounding of the output type and by the order of their float32 sums; a wrong one, which
// drops or misplaces a tile, differs by about the largest value)
template <typename T>
__global__ void largest_kernel(const T* ref, int M, int N, long ld, unsigned* check) {
  float m = 0.f;
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < (size_t)M * N;
       i += (size_t)gridDim.x * blockDim.x)
    m = fmaxf(m, fabsf(to_float<T>(ref[(i / N) * ld + i % N])));
  m = wave_max(m);
  if ((threadIdx.x & 63) == 0) atomicMax(check, __float_as_uint(m));
}

template <typename T>
__global__ void disagree_kernel(const T* got, const T* ref, int M, int N, long ld, unsigned* check) {
  const float floor_ = __uint_as_float(check[0]) * (1.0f / 1024.0f);
  unsigned bad = 0;
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < (size_t)M * N;
       i += (size_t)gridDim.x * blockDim.x) {
    const size_t at = (i / N) * ld + i % N;
    const float a = to_float<T>(got[at]), b = to_float<T>(ref[at]);
    const bool fine = fabsf(a - b) <= fmaxf(fabsf(a), fabsf(b)) * (1.0f / 64.0f) + floor_;
    bad += fine ? 0u : 1u;                 // (a NaN compares false: counted)
  }
  if (bad) atomicAdd(check + 1, bad);
}

// Whether proposal ``i`` gives, on the caller's operands, what ``ref`` holds (the first
// proposal's result, laid out as y). check: two words of device memory behind ref.
bool agrees(State& s, const Plan& p, int i, const Key& key, void* y, const void* ref, unsigned* check,
            const void* x, const void* w, hipStream_t stream) {
  const int M = std::get<0>(key), N = std::get<1>(key);
  const long ld = std::get<4>(key);
  const bool f32 = std::get<5>(key) == PTL_DTYPE_F32;
  if (!ok(run_algo(s, p, p.proposals[i].algo, y, x, w, stream))) return false;
  const unsigned zero[2] = {0u, 0u};
  if (hipMemcpyAsync(check, zero, sizeof(zero), hipMemcpyHostToDevice, stream) != hipSuccess) return false;
  const int blocks = (int)std::min<size_t>(1024, ((size_t)M * N + 255) / 256);
  if (f32) {
    largest_kernel<float><<<blocks, 256, 0, stream>>>((const float*)ref, M, N, ld, check);
    disagree_kernel<float><<<blocks, 256, 0, stream>>>((const float*)y, (const float*)ref, M, N, ld, check);
  } else {
    largest_kernel<bf16_t><<<blocks, 256, 0, stream>>>((const bf16_t*)ref, M, N, ld, check);
    disagree_kernel<bf16_t><<<blocks, 256, 0, stream>>>((const bf16_t*)y, (const bf16_t*)ref, M, N, ld, check);
  }
  unsigned out[2] = {0u, 1u};
  if (hipMemcpyAsync(out, check, sizeof(out), hipMemcpyDeviceToHost, stream) != hipSuccess ||
      hipStreamSynchronize(stream) != hipSuccess)
    return false;
  return out[1] == 0u;
}

// Times the proposals on the caller's operands (y is overwritten with the same product each time)
// and keeps the fastest whose result agrees with the first proposal's. Any failure leaves the
// first proposal. Not while the stream is captured: a later call may.
void time_plan(State& s, Plan& p, const Key& key, void* y, const void* x, const void* w, hipStream_t stream) {
  hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &capturing) != hipSuccess) {
    (void)hipGetLastError();
    return;
  }
  if (capturing != hipStreamCaptureStatusNone) return;
  static const bool log = getenv("PTL_BLASLT_LOG") != nullptr;
  p.timed = true;
  const int found = (int)p.proposals.size();
  if (found < 2) return;
  if (s.timed >= MAX_TIMED) {
    if (!s.said_full) fprintf(stderr, "[blaslt] %zu shapes have been timed; further shapes run the library's "
                                      "first proposal\n", s.timed);
    s.said_full = true;
    return;
  }
  ++s.timed;
  const auto& proposals = p.proposals;
  if (!s.t0 && (hipEventCreate(&s.t0) != hipSuccess || hipEventCreate(&s.t1) != hipSuccess)) {
    (void)hipGetLastError();
    s.t0 = s.t1 = nullptr;
    return;
  }
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
  if (log) {
    fprintf(stderr, "[blaslt] %d rows, %d columns, depth %d:", std::get<0>(key), std::get<1>(key), std::get<2>(key));
    for (int i = 0; i < found; ++i) fprintf(stderr, " %.1f", times[i] * 1e3f / TUNE_REPEATS);
    fprintf(stderr, " us\n");
  }
  if (times[0] < 0.f) return;
  // the library's first stays unless another is clearly faster (the operands are warm in the
  // caches here and cold in a step: a few per cent say nothing) and gives the same product
  const int M = std::get<0>(key);
  const long ld = std::get<4>(key);
  const size_t bytes = (size_t)M * ld * (std::get<5>(key) == PTL_DTYPE_F32 ? 4 : 2);
  char* ref = nullptr;
  for (;;) {
    int best_i = 0;
    float best = times[0] * TUNE_MARGIN;
    for (int i = 1; i < found; ++i)
      if (times[i] >= 0.f && times[i] < best) { best = times[i]; best_i = i; }
    if (best_i == 0) break;
    if (ref == nullptr) {
      // the first proposal's result, kept beside y for the comparison (the one allocation of a
      // timing, given back below; nothing here runs while a graph is recorded)
      if (hipMalloc((void**)&ref, bytes + 16) != hipSuccess) {
        (void)hipGetLastError();
        ref = nullptr;
        break;
      }
      if (!ok(run_algo(s, p, proposals[0].algo, y, x, w, stream)) ||
          hipMemcpyAsync(ref, y, bytes, hipMemcpyDeviceToDevice, stream) != hipSuccess)
        break;
    }
    if (agrees(s, p, best_i, key, y, ref, (unsigned*)(ref + ((bytes + 7) & ~(size_t)7)), x, w, stream)) {
      p.timed_choice = best_i;
      if (log) fprintf(stderr, "[blaslt]   -> proposal %d\n", best_i);
      break;
    }
    fprintf(stderr, "[blaslt] %d rows, %d columns, depth %d: proposal %d disagrees with the first and is "
                    "left out\n", M, std::get<1>(key), std::get<2>(key), best_i);
    times[best_i] = -1.f;
  }
  if (ref != nullptr) {
    (void)hipStreamSynchronize(stream);
    (void)hipFree(ref);
  }
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

}  // namespace

// y [M, N] (row stride ldy; bfloat16 or float32) = x [M, K] (bfloat16, row stride ldx) W^T,
// W [N, K] bfloat16 with dense rows. Rows of x and W 16-byte aligned.
// use_timed != 0: run the proposal that a timing of this shape kept, and time the shape now if
// it has not been (unless the stream is being captured); 0: the library's first proposal.
extern "C" int ptl_blaslt_gemm_bf16(void* y, const void* x, const void* w, int M, int N, int K,
                                    long ldx, long ldy, int out_dtype, int use_timed, hipStream_t stream) {
  if (M <= 0 || N <= 0) return PTL_OK;
  if (K <= 0 || ldx < K || ldy < N || (out_dtype != PTL_DTYPE_F32 && out_dtype != PTL_DTYPE_BF16))
    return PTL_ERR_ARG;
  static const bool never_timed = getenv("PTL_BLASLT_NO_TUNING") != nullptr;
  if (never_timed) use_timed = 0;
  State& s = state();
  std::lock_guard<std::mutex> guard(s.lock);
  if (s.handle == nullptr) {
    // the one lasting allocation of these libraries: the library's workspace, at the first call.
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
      // shapes that were timed stay (recorded graphs run their choice, and so must a later
      // recording of the same shape); the others are made again when they come back
      for (auto at = s.plans.begin(); at != s.plans.end();) {
        if (at->second.timed) { ++at; continue; }
        drop_plan(at->second);
        at = s.plans.erase(at);
      }
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
  if (use_timed && !plan.timed) time_plan(s, plan, key, y, x, w, stream);
  const int which = use_timed ? plan.timed_choice : 0;
  return ok(run_algo(s, plan, plan.proposals[which].algo, y, x, w, stream)) ? PTL_OK : PTL_ERR_LAUNCH;
}

// How many shapes have been timed, and the proposal kept for one (-1: no plan for it, or not
// timed). For tests and logs.
extern "C" int ptl_blaslt_timed_shapes() {
  State& s = state();
  std::lock_guard<std::mutex> guard(s.lock);
  return (int)s.timed;
}

extern "C" int ptl_blaslt_timed_choice(int M, int N, int K, long ldx, long ldy, int out_dtype) {
  State& s = state();
  std::lock_guard<std::mutex> guard(s.lock);
  auto it = s.plans.find(Key(M, N, K, ldx, ldy, out_dtype));
  return it == s.plans.end() || !it->second.timed ? -1 : it->second.timed_choice;
}
