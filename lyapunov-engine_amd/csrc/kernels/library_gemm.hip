// Large bfloat16 matrix products through the vendor's library (hipBLASLt), called
// directly: out [M, N] = a [M, K] * w [N, K]^T, the projection of a whole prompt
// or portion.  The reference leaves these products to cuBLAS behind nn.Linear
// (python/lyapunov_engine/models/llama.py:45-48, 112-117, 177).
//
// The library's own call costs a few microseconds on the host once the product's
// description and the chosen algorithm are kept; building them anew for every
// call (what a general tensor library does) costs twice that, which is what
// a prompt of a few hundred tokens spends most of its time on.  So: one plan per
// (shape, strides, output type), made at the first call and reused.
//
// The library's heuristic orders its algorithms by a model of the machine.  While
// tuning is switched on (lyp_library_gemm_tuning, meant for an engine's warm-up and
// for the run before a graph is captured), a shape's first call measures instead:
// every solution the library has for these types that takes the shape (about two
// thousand of twenty thousand) is run once, as a screen; the fastest few of the
// screen and the heuristic's first few are then run on the call's own operands
// under the conditions of a model step, and the fastest is kept.  Against the
// heuristic's first choice that gave, on the 1B shape: at 128 rows q/k/v 19.7 ->
// 14.5 us and o 15.4 -> 11.6 us; at 8,192 rows gate/up 352 -> 324 us and down 157
// -> 144 us; at 2,048 rows the heuristic's first choice is within 3 % of the best.
// A plan, once made, is never changed: the same shape gives the same sums for as
// long as the process lives.  A choice made by measurement is handed on: a shape
// that first shows up while tuning is off takes the choice measured for the same
// matrix at the nearest number of rows.  LYAPUNOV_AMD_GEMM_LOG=1 prints every
// measured choice.
#include <hip/hip_runtime.h>
#include <hipblaslt/hipblaslt.h>
#include <hipblaslt/hipblaslt-ext.hpp>

#include <algorithm>
#include <cstdlib>
#include <map>
#include <tuple>
#include <vector>

#include "common.h"

namespace lyp {
namespace {

struct Plan {
  hipblasLtMatmulDesc_t desc = nullptr;
  hipblasLtMatrixLayout_t lw = nullptr, la = nullptr, lo = nullptr;
  hipblasLtMatmulAlgo_t algo;
  size_t workspace = 0;
};

// device, M, N, K, lda, ldw, ldo, out type, made for a graph (without a workspace)
using Key = std::tuple<int, int, int, int, int, int, int, int, int>;

// device, N, K, out type, made for a graph: the products a measured choice may be handed on to
using Family = std::tuple<int, int, int, int, int>;

struct State {
  std::map<int, hipblasLtHandle_t> handles;  // per device
  std::map<Key, Plan> plans;
  // Algorithms chosen by measurement, by number of rows, per family of products.  A shape that
  // first shows up while tuning is off (a prompt portion of some odd length in the middle of
  // serving) takes the choice measured for the nearest number of rows, if the library accepts it
  // there, rather than the heuristic's.
  std::map<Family, std::map<int, hipblasLtMatmulAlgo_t>> measured;
};

State& state() {
  static State s;
  return s;
}

int g_tuning_candidates = 0;   // > 1: a new plan is chosen by measurement among this many candidates
bool g_tuning_no_workspace = false;  // a new plan's algorithm is one that needs no workspace
constexpr int kMostCandidates = 32;
constexpr float kTuningMargin = 0.95f;  // what a candidate's time has to stay under, relative to the heuristic's first choice
bool g_tuning_all = true;      // screen all of the library's solutions, not only the heuristic's first few


#define LYP_BLAS(call, what)                                                       \
  do {                                                                             \
    const hipblasStatus_t st_ = (call);                                            \
    if (st_ != HIPBLAS_STATUS_SUCCESS) {                                           \
      lyp::set_error("library gemm: %s failed with status %d", what, static_cast<int>(st_)); \
      return -1;                                                                   \
    }                                                                              \
  } while (0)

// ---- a candidate's result against the heuristic's first choice
// A solution the library lists for a shape is not thereby right for it: before a measured
// candidate may win, its output on the call's own operands is held against the output of the
// heuristic's first choice.  Two sums of the same products in another order differ by rounding:
// a few units in the last place of the output type, relative to the larger of the two values,
// and for values that cancel, relative to the matrix's largest value.
__global__ void max_abs_kernel(const void* x, int is_f32, int M, int N, int ld, unsigned* out) {
  float m = 0.f;
  const size_t total = static_cast<size_t>(M) * N;
  for (size_t i = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x; i < total;
       i += static_cast<size_t>(gridDim.x) * blockDim.x) {
    const size_t at = (i / N) * ld + i % N;
    const float v = is_f32 ? static_cast<const float*>(x)[at] : to_f32(static_cast<const bf16_t*>(x)[at]);
    m = fmaxf(m, fabsf(v));   // a NaN is not counted here; the comparison below counts it
  }
  atomicMax(out, __float_as_uint(m));   // non-negative floats order as their bits do
}

__global__ void count_off_kernel(const void* got, const void* ref, int is_f32, int M, int N, int ld,
                                 const unsigned* ref_max, unsigned* off) {
  const float scale = __uint_as_float(*ref_max);
  const float rel = is_f32 ? 1e-4f : 1.6e-2f;   // bf16: two units in the last place (8 bits)
  const float floor_ = (is_f32 ? 1e-5f : 2e-3f) * scale;
  unsigned n = 0;
  const size_t total = static_cast<size_t>(M) * N;
  for (size_t i = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x; i < total;
       i += static_cast<size_t>(gridDim.x) * blockDim.x) {
    const size_t at = (i / N) * ld + i % N;
    const float a = is_f32 ? static_cast<const float*>(got)[at] : to_f32(static_cast<const bf16_t*>(got)[at]);
    const float b = is_f32 ? static_cast<const float*>(ref)[at] : to_f32(static_cast<const bf16_t*>(ref)[at]);
    const float d = fabsf(a - b);
    if (!(d <= rel * fmaxf(fabsf(a), fabsf(b)) + floor_)) ++n;   // also when either is a NaN
  }
  if (n) atomicAdd(off, n);
}

// How many values of `got` are off `ref` (both [M, N], rows ld apart) by more than rounding; -1 if
// the check itself failed.  `scratch`: two unsigned values on the device.  Waits for the stream.
long long values_off(const void* got, const void* ref, int is_f32, int M, int N, int ld, unsigned* scratch,
                     hipStream_t stream) {
  unsigned host[2] = {0, 0};
  if (hipMemcpyAsync(scratch, host, sizeof(host), hipMemcpyHostToDevice, stream) != hipSuccess) return -1;
  const int blocks = 256;
  max_abs_kernel<<<blocks, 256, 0, stream>>>(ref, is_f32, M, N, ld, scratch);
  count_off_kernel<<<blocks, 256, 0, stream>>>(got, ref, is_f32, M, N, ld, scratch, scratch + 1);
  if (hipMemcpyAsync(host, scratch, sizeof(host), hipMemcpyDeviceToHost, stream) != hipSuccess ||
      hipStreamSynchronize(stream) != hipSuccess)
    return -1;
  return host[1];
}

int g_rejected = 0;   // candidates turned down because their output was off (for tests and the log)

// Runs the product `times` times with candidate `c`; false if the library refuses it.
bool run_candidate(hipblasLtHandle_t handle, const Plan& p, const hipblasLtMatmulHeuristicResult_t& c, const void* a,
                   const void* w, void* out, void* workspace, hipStream_t stream, int times) {
  const float alpha = 1.0f, beta = 0.0f;
  for (int i = 0; i < times; ++i)
    if (hipblasLtMatmul(handle, p.desc, &alpha, w, p.lw, a, p.la, &beta, out, p.lo, out, p.lo, &c.algo, workspace,
                        c.workspaceSize, stream) != HIPBLAS_STATUS_SUCCESS)
      return false;
  return true;
}

// The fastest of the candidates on the operands of this call (which it runs several times: the
// output is written again and again with the same values).  Waits for the stream.  A product in
// a model step finds its weights in memory, not in a cache (a step reads more weights than the
// caches hold), and its activations just written: before every timed run the caches are filled
// with other data and the activations are read once.  Candidates ranked with everything still
// in the cache from the run before were slower in the step than the library's first choice.
int fastest_candidate(hipblasLtHandle_t handle, const Plan& p, const hipblasLtMatmulHeuristicResult_t* found, int n_found,
                      const void* a, size_t a_bytes, const void* w, void* out, int out_is_f32, int M, int N, int ldo,
                      void* workspace, size_t workspace_bytes, hipStream_t stream, float* first_ms, float* chosen_ms) {
  hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &capturing) != hipSuccess || capturing != hipStreamCaptureStatusNone) return 0;
  constexpr size_t kFlushBytes = size_t{512} << 20;   // twice the memory-side cache
  const size_t out_bytes = (static_cast<size_t>(M - 1) * ldo + N) * (out_is_f32 ? 4 : 2);
  void* other = nullptr;
  if (hipMalloc(&other, kFlushBytes + ((a_bytes + 15) / 16) * 16 + ((out_bytes + 15) / 16) * 16 + 16) != hipSuccess) {
    (void)hipGetLastError();
    return 0;
  }
  // behind the flush area and the copy of the activations: the first choice's output, and two counters
  void* ref_out = static_cast<char*>(other) + kFlushBytes + ((a_bytes + 15) / 16) * 16;
  unsigned* counters = reinterpret_cast<unsigned*>(static_cast<char*>(ref_out) + ((out_bytes + 15) / 16) * 16);
  bool have_ref = false;
  hipEvent_t e0 = nullptr, e1 = nullptr;
  int best = 0;
  float best_ms = -1.f;
  if (hipEventCreate(&e0) == hipSuccess && hipEventCreate(&e1) == hipSuccess) {
    for (int c = 0; c < n_found; ++c) {
      if (found[c].workspaceSize > workspace_bytes) continue;
      if (!run_candidate(handle, p, found[c], a, w, out, workspace, stream, 1)) continue;
      if (c == 0) {
        have_ref = hipMemcpyAsync(ref_out, out, out_bytes, hipMemcpyDeviceToDevice, stream) == hipSuccess;
      } else {
        // without the first choice's output to hold it against, no other candidate is taken
        const long long off = have_ref ? values_off(out, ref_out, out_is_f32, M, N, ldo, counters, stream) : -1;
        if (off != 0) {
          ++g_rejected;
          if (getenv("LYAPUNOV_AMD_GEMM_LOG"))
            fprintf(stderr, "[lyapunov-amd] product %d x %d: candidate %d (solution %d) turned down, %lld values off the "
                    "first choice's\n", M, N, c, hipblaslt_ext::getIndexFromAlgo(const_cast<hipblasLtMatmulAlgo_t&>(found[c].algo)), off);
          continue;
        }
      }
      float fastest = -1.f;
      for (int run = 0; run < 3; ++run) {
        float ms = 0.f;
        if (hipMemsetAsync(other, run, kFlushBytes, stream) != hipSuccess ||
            hipMemcpyAsync(static_cast<char*>(other) + kFlushBytes, a, a_bytes, hipMemcpyDeviceToDevice, stream) != hipSuccess ||
            hipEventRecord(e0, stream) != hipSuccess || !run_candidate(handle, p, found[c], a, w, out, workspace, stream, 1) ||
            hipEventRecord(e1, stream) != hipSuccess || hipEventSynchronize(e1) != hipSuccess ||
            hipEventElapsedTime(&ms, e0, e1) != hipSuccess) {
          fastest = -1.f;
          break;
        }
        if (fastest < 0.f || ms < fastest) fastest = ms;
      }
      if (c == 0) *first_ms = fastest;
      // Another candidate has to be ahead of the heuristic's first choice by a clear margin: a
      // few per cent are within what two timings of the same kernel differ by, and what wins
      // such a toss here has lost by more than that inside a model step.
      const float bar = (c > 0 && *first_ms >= 0.f && best == 0) ? kTuningMargin * best_ms : best_ms;
      if (fastest >= 0.f && (best_ms < 0.f || fastest < bar)) best_ms = fastest, best = c;
    }
  }
  if (e0) (void)hipEventDestroy(e0);
  if (e1) (void)hipEventDestroy(e1);
  (void)hipStreamSynchronize(stream);
  (void)hipFree(other);
  // whatever candidate ran last, the output now holds the product; the caller runs the chosen one once more
  *chosen_ms = best_ms;
  return best_ms < 0.f ? 0 : best;
}

// Appends to `found` the `keep` fastest of all the library's solutions for these types that take
// this product (and fit the workspace), by one warm run each on the call's operands; the careful
// measurement of the few is the caller's.  Does nothing while the stream is being captured.
void screen_all(hipblasLtHandle_t handle, const Plan& p, hipDataType in_t, hipDataType out_t, hipblasOperation_t ta,
                hipblasOperation_t tb, const void* a, const void* w, void* out, void* workspace, size_t workspace_bytes,
                hipStream_t stream, int keep, std::vector<hipblasLtMatmulHeuristicResult_t>& found) {
  hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &capturing) != hipSuccess || capturing != hipStreamCaptureStatusNone) return;
  std::vector<hipblasLtMatmulHeuristicResult_t> all;
  if (hipblaslt_ext::getAllAlgos(handle, hipblaslt_ext::GemmType::HIPBLASLT_GEMM, ta, tb, in_t, in_t, out_t, out_t,
                                 HIPBLAS_COMPUTE_32F, all) != HIPBLAS_STATUS_SUCCESS)
    return;
  hipEvent_t e0 = nullptr, e1 = nullptr;
  if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) {
    if (e0) (void)hipEventDestroy(e0);
    return;
  }
  const float alpha = 1.0f, beta = 0.0f;
  std::vector<std::pair<float, size_t>> timed;
  for (size_t i = 0; i < all.size(); ++i) {
    size_t need = 0;
    if (hipblaslt_ext::matmulIsAlgoSupported(handle, p.desc, &alpha, p.lw, p.la, &beta, p.lo, p.lo, all[i].algo, need) !=
            HIPBLAS_STATUS_SUCCESS ||
        need > workspace_bytes)
      continue;
    all[i].workspaceSize = need;
    float ms = 0.f;
    if (hipEventRecord(e0, stream) != hipSuccess || !run_candidate(handle, p, all[i], a, w, out, workspace, stream, 1) ||
        hipEventRecord(e1, stream) != hipSuccess || hipEventSynchronize(e1) != hipSuccess ||
        hipEventElapsedTime(&ms, e0, e1) != hipSuccess) {
      (void)hipGetLastError();
      continue;
    }
    timed.emplace_back(ms, i);
  }
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  (void)hipStreamSynchronize(stream);
  std::sort(timed.begin(), timed.end());
  for (size_t k = 0; k < timed.size() && k < static_cast<size_t>(keep); ++k) {
    const hipblasLtMatmulHeuristicResult_t& c = all[timed[k].second];
    const int index = hipblaslt_ext::getIndexFromAlgo(const_cast<hipblasLtMatmulAlgo_t&>(c.algo));
    bool have = false;
    for (auto& f : found) have = have || hipblaslt_ext::getIndexFromAlgo(f.algo) == index;
    if (!have) found.push_back(c);
  }
}

int make_plan(hipblasLtHandle_t handle, Plan& p, int device, int M, int N, int K, int lda, int ldw, int ldo, int out_type,
              const void* a, const void* w, void* out, void* workspace, size_t workspace_bytes, hipStream_t stream) {
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
  if (g_tuning_no_workspace) workspace_bytes = 0;  // the library then offers only algorithms that need none
  const Family family{device, N, K, out_type, g_tuning_no_workspace ? 1 : 0};
  auto& measured = state().measured[family];
  if (g_tuning_candidates <= 1 && !measured.empty()) {
    // tuning is off: the choice measured for the nearest number of rows (by ratio), if it applies here
    auto best = measured.begin();
    auto ratio = [M](int m) { return m > M ? static_cast<double>(m) / M : static_cast<double>(M) / m; };
    for (auto it = measured.begin(); it != measured.end(); ++it)
      if (ratio(it->first) < ratio(best->first)) best = it;
    const float alpha = 1.0f, beta = 0.0f;
    size_t need = 0;
    if (hipblaslt_ext::matmulIsAlgoSupported(handle, p.desc, &alpha, p.lw, p.la, &beta, p.lo, p.lo, best->second, need) ==
            HIPBLAS_STATUS_SUCCESS &&
        need <= workspace_bytes) {
      p.algo = best->second;
      p.workspace = need;
      return 0;
    }
  }
  hipblasLtMatmulPreference_t pref = nullptr;
  LYP_BLAS(hipblasLtMatmulPreferenceCreate(&pref), "PreferenceCreate");
  uint64_t ws = workspace_bytes;
  hipblasStatus_t st =
      hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &ws, sizeof(ws));
  std::vector<hipblasLtMatmulHeuristicResult_t> found(kMostCandidates);
  int n_found = 0;
  const int wanted = g_tuning_candidates < 1 ? 1 : (g_tuning_candidates > kMostCandidates ? kMostCandidates : g_tuning_candidates);
  if (st == HIPBLAS_STATUS_SUCCESS)
    st = hipblasLtMatmulAlgoGetHeuristic(handle, p.desc, p.lw, p.la, p.lo, p.lo, pref, wanted, found.data(), &n_found);
  hipblasLtMatmulPreferenceDestroy(pref);
  LYP_BLAS(st, "AlgoGetHeuristic");
  if (n_found < 1) {
    lyp::set_error("library gemm: the library has no algorithm for %d x %d x %d", M, N, K);
    return -1;
  }
  found.resize(n_found);
  if (g_tuning_candidates > 1 && g_tuning_all)
    screen_all(handle, p, in_t, out_t, ta, tb, a, w, out, workspace, workspace_bytes, stream, wanted, found);
  const int n_heuristic = n_found;
  n_found = static_cast<int>(found.size());
  float first_ms = -1.f, chosen_ms = -1.f;
  const int chosen =
      n_found > 1 ? fastest_candidate(handle, p, found.data(), n_found, a, static_cast<size_t>(M - 1) * lda * 2 + static_cast<size_t>(K) * 2,
                                      w, out, out_type == kF32 ? 1 : 0, M, N, ldo, workspace, workspace_bytes, stream,
                                      &first_ms, &chosen_ms)
                  : 0;
  if (n_found > 1 && getenv("LYAPUNOV_AMD_GEMM_LOG"))
    fprintf(stderr, "[lyapunov-amd] product %d x %d x %d: %d candidates of the heuristic, %d of the screen; the heuristic's "
            "first takes %.1f us, the chosen one (number %d, solution %d) %.1f us\n", M, N, K, n_heuristic,
            n_found - n_heuristic, first_ms * 1e3f, chosen, hipblaslt_ext::getIndexFromAlgo(found[chosen].algo),
            chosen_ms * 1e3f);
  p.algo = found[chosen].algo;
  p.workspace = found[chosen].workspaceSize;
  if (g_tuning_candidates > 1 && n_found > 1) measured[M] = p.algo;
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
  const Key key{device, M, N, K, lda, ldw, ldo, out_dtype, g_tuning_no_workspace ? 1 : 0};
  auto it = s.plans.find(key);
  if (it == s.plans.end()) {
    Plan p;
    if (make_plan(h->second, p, device, M, N, K, lda, ldw, ldo, out_dtype, a, w, out, workspace,
                  static_cast<size_t>(workspace_bytes), stream) != 0) {
      if (p.lw) hipblasLtMatrixLayoutDestroy(p.lw);  // what a failed attempt had made so far
      if (p.la) hipblasLtMatrixLayoutDestroy(p.la);
      if (p.lo) hipblasLtMatrixLayoutDestroy(p.lo);
      if (p.desc) hipblasLtMatmulDescDestroy(p.desc);
      return -1;
    }
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

// candidates > 1: from now on the plan of a shape not seen before is chosen by running that many of
// the library's candidates (at most 32) on the first call's operands, which waits for the stream;
// 0 or 1: the library's first choice, without a measurement.  Returns the previous number of
// candidates (to be handed back, with no_workspace 0, when the tuning ends).
// With no_workspace the library is asked for algorithms that need no workspace: for products that
// are about to be recorded into a graph (an algorithm with a workspace may clear it with a memset
// node, and memset nodes in replayed graphs are not to be trusted on this machine).  Such plans are
// kept apart from the others, so the setting has to stay on while the graph is recorded.
int lyp_library_gemm_tuning(int candidates, int no_workspace) {
  const int before = g_tuning_candidates;
  g_tuning_candidates = candidates;
  g_tuning_no_workspace = no_workspace != 0;
  return before;
}

// Whether tuning also screens every solution the library has (the default) or only measures the
// heuristic's first few.
void lyp_library_gemm_tuning_all(int on) { g_tuning_all = on != 0; }

// Number of plans kept (for tests).
int lyp_library_gemm_plans() { return static_cast<int>(state().plans.size()); }

// Candidates that were measured and turned down because their output differed from the heuristic's
// first choice by more than rounding (for tests).
int lyp_library_gemm_rejected() { return g_rejected; }

// How the plan of a product was made: the library's solution index, or -1 if no plan of this shape is kept.
int lyp_library_gemm_solution(int M, int N, int K, int lda, int ldw, int ldo, int out_dtype, int for_graph) {
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess) return -1;
  auto it = state().plans.find(Key{device, M, N, K, lda, ldw, ldo, out_dtype, for_graph ? 1 : 0});
  if (it == state().plans.end()) return -1;
  return hipblaslt_ext::getIndexFromAlgo(it->second.algo);
}

}  // extern "C"
