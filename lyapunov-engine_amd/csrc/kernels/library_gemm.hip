// Large bfloat16 matrix products through the vendor's library (hipBLASLt), called
// directly: out [M, N] = a [M, K] * w [N, K]^T, the projection of a whole prompt
// or portion.  The reference leaves these products to cuBLAS behind nn.Linear
// (python/lyapunov_engine/models/llama.py:45-48, 112-117, 177).
//
// The library's own call costs a few microseconds on the host once the product's
// description and the chosen algorithm are kept; building them anew for every
// call (what a general tensor library does) costs four times that, which is what
// a prompt of a few hundred tokens spends most of its time on.  So: one plan per
// (shape, strides, output type), made at the first call and reused.
#include <hip/hip_runtime.h>
#include <hipblaslt/hipblaslt.h>

#include <map>
#include <tuple>

#include "common.h"

namespace lyp {
namespace {

struct Plan {
  hipblasLtMatmulDesc_t desc = nullptr;
  hipblasLtMatrixLayout_t lw = nullptr, la = nullptr, lo = nullptr;
  hipblasLtMatmulAlgo_t algo;
  size_t workspace = 0;
};

using Key = std::tuple<int, int, int, int, int, int, int, int>;  // device, M, N, K, lda, ldw, ldo, out type

struct State {
  std::map<int, hipblasLtHandle_t> handles;  // per device
  std::map<Key, Plan> plans;
};

State& state() {
  static State s;
  return s;
}

#define LYP_BLAS(call, what)                                                       \
  do {                                                                             \
    const hipblasStatus_t st_ = (call);                                            \
    if (st_ != HIPBLAS_STATUS_SUCCESS) {                                           \
      lyp::set_error("library gemm: %s failed with status %d", what, static_cast<int>(st_)); \
      return -1;                                                                   \
    }                                                                              \
  } while (0)

int make_plan(hipblasLtHandle_t handle, Plan& p, int M, int N, int K, int lda, int ldw, int ldo, int out_type,
              size_t workspace_bytes) {
  // Row-major out = a w^T is, in the library's column-major terms, out^T [N, M] = w^T-stored [K, N] transposed
  // times a-stored [K, M].
  const hipDataType in_t = HIP_R_16BF, out_t = out_type == kF32 ? HIP_R_32F : HIP_R_16BF;
  LYP_BLAS(hipblasLtMatmulDescCreate(&p.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F), "MatmulDescCreate");
  const hipblasOperation_t ta = HIPBLAS_OP_T, tb = HIPBLAS_OP_N;
  LYP_BLAS(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &ta, sizeof(ta)), "set TRANSA");
  LYP_BLAS(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &tb, sizeof(tb)), "set TRANSB");
  LYP_BLAS(hipblasLtMatrixLayoutCreate(&p.lw, in_t, K, N, ldw), "layout of the weights");
  LYP_BLAS(hipblasLtMatrixLayoutCreate(&p.la, in_t, K, M, lda), "layout of the activations");
  LYP_BLAS(hipblasLtMatrixLayoutCreate(&p.lo, out_t, N, M, ldo), "layout of the output");
  hipblasLtMatmulPreference_t pref = nullptr;
  LYP_BLAS(hipblasLtMatmulPreferenceCreate(&pref), "PreferenceCreate");
  uint64_t ws = workspace_bytes;
  hipblasStatus_t st =
      hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &ws, sizeof(ws));
  hipblasLtMatmulHeuristicResult_t found[1];
  int n_found = 0;
  if (st == HIPBLAS_STATUS_SUCCESS)
    st = hipblasLtMatmulAlgoGetHeuristic(handle, p.desc, p.lw, p.la, p.lo, p.lo, pref, 1, found, &n_found);
  hipblasLtMatmulPreferenceDestroy(pref);
  LYP_BLAS(st, "AlgoGetHeuristic");
  if (n_found < 1) {
    lyp::set_error("library gemm: the library has no algorithm for %d x %d x %d", M, N, K);
    return -1;
  }
  p.algo = found[0].algo;
  p.workspace = found[0].workspaceSize;
  return 0;
}

}  // namespace
}  // namespace lyp

using namespace lyp;

extern "C" {

// out [M, N] (bfloat16, or float when out_dtype is kF32) = a [M, K] * w [N, K]^T, both bfloat16 with
// rows lda and ldw apart; `workspace` is device memory the library may use (workspace_bytes of it).
int lyp_library_gemm_nt(const void* a, const void* w, void* out, int out_dtype, int M, int N, int K, int lda, int ldw,
                        int ldo, void* workspace, long long workspace_bytes, hipStream_t stream) {
  LYP_REQUIRE(M > 0 && N > 0 && K > 0 && lda >= K && ldw >= K && ldo >= N, "library gemm: %d x %d x %d, strides %d %d %d",
              M, N, K, lda, ldw, ldo);
  LYP_REQUIRE(out_dtype == kF32 || out_dtype == kBF16, "library gemm: output type %d", out_dtype);
  LYP_REQUIRE(a && w && out, "library gemm: null operand");
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess) {
    set_error("library gemm: no current device");
    return -1;
  }
  State& s = state();
  auto h = s.handles.find(device);
  if (h == s.handles.end()) {
    hipblasLtHandle_t handle = nullptr;
    LYP_BLAS(hipblasLtCreate(&handle), "hipblasLtCreate");
    h = s.handles.emplace(device, handle).first;
  }
  const Key key{device, M, N, K, lda, ldw, ldo, out_dtype};
  auto it = s.plans.find(key);
  if (it == s.plans.end()) {
    Plan p;
    if (make_plan(h->second, p, M, N, K, lda, ldw, ldo, out_dtype, static_cast<size_t>(workspace_bytes)) != 0) return -1;
    it = s.plans.emplace(key, p).first;
  }
  const Plan& p = it->second;
  LYP_REQUIRE(p.workspace <= static_cast<size_t>(workspace_bytes) && (p.workspace == 0 || workspace),
              "library gemm: the chosen algorithm wants %zu bytes of workspace, %lld are given", p.workspace,
              workspace_bytes);
  const float alpha = 1.0f, beta = 0.0f;
  LYP_BLAS(hipblasLtMatmul(h->second, p.desc, &alpha, w, p.lw, a, p.la, &beta, out, p.lo, out, p.lo, &p.algo, workspace,
                           p.workspace, stream),
           "hipblasLtMatmul");
  return 0;
}

// Number of plans kept (for tests).
int lyp_library_gemm_plans() { return static_cast<int>(state().plans.size()); }

}  // extern "C"
