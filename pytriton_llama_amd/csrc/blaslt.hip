// The library matrix product for the many rows of a prompt: y = x W^T through hipBLASLt,
// called directly (the reference runs its projections through cuBLAS by way of nn.Linear,
// lite_llama/models/llama.py:37-40,61,120,221).
//
// Why not through torch: its linear() asks the library for an algorithm on every call and
// takes about 20 us on the host, more than most of the kernels it launches; a prompt portion
// then runs at the speed of the host. Here the descriptors and the algorithm of a shape are
// made once and kept, and a call is a table look-up and hipblasLtMatmul (3 to 4 us).
//
// The algorithm is the library's first proposal for the shape (timing its first eight proposals
// for 2,048-row products found nothing faster).
#include "common.h"
#include <hipblaslt/hipblaslt.h>
#include <map>
#include <mutex>
#include <tuple>

namespace {

constexpr size_t WORKSPACE_BYTES = 64u << 20;
// Plans kept at most. Steps replayed as graphs meet a few dozen shapes; steps launched kernel by
// kernel bring a new M with every prompt length, so the table is emptied when it is full (the
// library is only read at call time: a plan may go once its call has returned).
constexpr size_t MAX_PLANS = 1024;

struct Plan {
  hipblasLtMatmulDesc_t desc = nullptr;
  hipblasLtMatrixLayout_t a = nullptr, b = nullptr, c = nullptr;
  hipblasLtMatmulHeuristicResult_t proposal;      // the library's first for this shape
};

// (M, N, K, ldx, ldy, output type)
using Key = std::tuple<int, int, int, long, long, int>;

struct State {
  hipblasLtHandle_t handle = nullptr;
  void* workspace = nullptr;
  std::map<Key, Plan> plans;
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
  hipblasLtMatmulPreference_t pref = nullptr;
  if (!ok(hipblasLtMatmulPreferenceCreate(&pref))) return PTL_ERR_LAUNCH;
  const uint64_t ws = WORKSPACE_BYTES;
  hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &ws, sizeof(ws));
  int found = 0;
  const hipblasStatus_t st = hipblasLtMatmulAlgoGetHeuristic(s.handle, p.desc, p.a, p.b, p.c, p.c, pref, 1,
                                                             &p.proposal, &found);
  hipblasLtMatmulPreferenceDestroy(pref);
  return ok(st) && found > 0 ? PTL_OK : PTL_ERR_ARG;
}

hipblasStatus_t run(State& s, const Plan& p, void* y, const void* x, const void* w, hipStream_t stream) {
  const float one = 1.0f, zero = 0.0f;
  return hipblasLtMatmul(s.handle, p.desc, &one, w, p.a, x, p.b, &zero, y, p.c, y, p.c, &p.proposal.algo,
                         s.workspace, WORKSPACE_BYTES, stream);
}

}  // namespace

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
  return ok(run(s, it->second, y, x, w, stream)) ? PTL_OK : PTL_ERR_LAUNCH;
}
