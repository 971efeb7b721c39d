// Library matrix product for prompt portions of more than 64 tokens:
//   out[M, N] = x[M, K] . w[N, K]^T     bf16 in, float32 accumulation, bf16 out
// through hipBLASLt, as the reference uses nn.Linear (src/tokamak/model/layers.py:103,
// src/tokamak/model/transformer.py:67-69,85).  Host code only.
//
// Two things a generic call path does not do:
//  * the plan of a shape (descriptors, algorithm, workspace need) is made once and
//    kept, so a call costs a map lookup and one launch;
//  * the algorithm is chosen by measurement: the first time a shape class (N, K, M
//    rounded up to 128) is seen, the library's candidates for it are each run a few
//    times on the caller's operands and the fastest is kept for the class.  The
//    library's own first choice is often not the fastest (by up to 2x for some of
//    this model's shapes).  The numbers an algorithm computes do not depend on the
//    others that were tried.  (Trying every algorithm of the library instead
//    of its first candidates was measured too: it takes a second per shape class
//    and gains under 2 %, so it is not offered.)
#include <hip/hip_runtime.h>
#include <hipblaslt/hipblaslt.h>
#include <hipblaslt/hipblaslt-ext.hpp>

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <map>
#include <mutex>
#include <tuple>
#include <vector>
#include "slots.h"

#define TK_API extern "C" __attribute__((visibility("default")))

namespace {

struct Plan {
  hipblasLtMatmulDesc_t desc = nullptr;
  hipblasLtMatrixLayout_t lw = nullptr, lx = nullptr, lo = nullptr;
  hipblasLtMatmulAlgo_t algo;
};

using ShapeKey = std::tuple<int, int, int, long, long, long>;  // M, N, K, ldx, ldw, ldo
using ClassKey = std::tuple<int, int, int>;                    // ceil(M / 128), N, K

std::mutex g_lock;
hipblasLtHandle_t g_handle = nullptr;
std::map<ShapeKey, Plan> g_plans;
std::map<ClassKey, hipblasLtMatmulAlgo_t> g_class_algo;
long g_tuned = 0;

constexpr int kMaxCandidates = 32;
constexpr int kClassRows = 128;

int make_descriptors(Plan& p, int M, int N, int K, long ldx, long ldw, long ldo) {
  // column-major view: out^T [N, M] = (w^T)^T [N, K] . x^T [K, M]
  if (hipblasLtMatmulDescCreate(&p.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F) != HIPBLAS_STATUS_SUCCESS) return -10;
  hipblasOperation_t ta = HIPBLAS_OP_T, tb = HIPBLAS_OP_N;
  hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &ta, sizeof(ta));
  hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &tb, sizeof(tb));
  if (hipblasLtMatrixLayoutCreate(&p.lw, HIP_R_16BF, K, N, ldw) != HIPBLAS_STATUS_SUCCESS) return -11;
  if (hipblasLtMatrixLayoutCreate(&p.lx, HIP_R_16BF, K, M, ldx) != HIPBLAS_STATUS_SUCCESS) return -11;
  if (hipblasLtMatrixLayoutCreate(&p.lo, HIP_R_16BF, N, M, ldo) != HIPBLAS_STATUS_SUCCESS) return -11;
  return 0;
}

bool usable(const Plan& p, hipblasLtMatmulAlgo_t& algo, size_t ws_bytes) {
  const float alpha = 1.f, beta = 0.f;
  size_t need = 0;
  return hipblaslt_ext::matmulIsAlgoSupported(g_handle, p.desc, &alpha, p.lw, p.lx, &beta, p.lo, p.lo,
                                              algo, need) == HIPBLAS_STATUS_SUCCESS &&
         need <= ws_bytes;
}

hipblasStatus_t run(const Plan& p, hipblasLtMatmulAlgo_t& algo, const void* x, const void* w, void* out,
                    void* ws, size_t ws_bytes, hipStream_t stream) {
  const float alpha = 1.f, beta = 0.f;
  return hipblasLtMatmul(g_handle, p.desc, &alpha, w, p.lw, x, p.lx, &beta, out, p.lo, out, p.lo, &algo,
                         ws, ws_bytes, stream);
}

// Average milliseconds of `runs` products after one untimed one, or < 0 if it fails.
float time_algo(const Plan& p, hipblasLtMatmulAlgo_t& algo, const void* x, const void* w, void* out, void* ws,
                size_t ws_bytes, hipStream_t stream, hipEvent_t e0, hipEvent_t e1, int runs) {
  if (run(p, algo, x, w, out, ws, ws_bytes, stream) != HIPBLAS_STATUS_SUCCESS) return -1.f;
  hipEventRecord(e0, stream);
  for (int r = 0; r < runs; ++r)
    if (run(p, algo, x, w, out, ws, ws_bytes, stream) != HIPBLAS_STATUS_SUCCESS) return -1.f;
  hipEventRecord(e1, stream);
  if (hipEventSynchronize(e1) != hipSuccess) return -1.f;
  float ms = 0.f;
  hipEventElapsedTime(&ms, e0, e1);
  return ms / runs;
}

// The algorithm for a new shape class: the fastest of the library's first `tune`
// candidates, measured on the caller's operands.  false: the library has none.
bool choose_algorithm(Plan& p, int tune, const void* x, const void* w, void* out, int M, int N, void* ws,
                      size_t ws_bytes, hipStream_t stream, bool& measured) {
  hipblasLtMatmulPreference_t pref;
  if (hipblasLtMatmulPreferenceCreate(&pref) != HIPBLAS_STATUS_SUCCESS) return false;
  uint64_t cap = ws_bytes;
  hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &cap, sizeof(cap));
  const int want = tune > 1 ? (tune < kMaxCandidates ? tune : kMaxCandidates) : 1;
  std::vector<hipblasLtMatmulHeuristicResult_t> found(want);
  int got = 0;
  const hipblasStatus_t st = hipblasLtMatmulAlgoGetHeuristic(g_handle, p.desc, p.lw, p.lx, p.lo, p.lo, pref, want,
                                                             found.data(), &got);
  hipblasLtMatmulPreferenceDestroy(pref);
  if (st != HIPBLAS_STATUS_SUCCESS || got <= 0) return false;
  std::vector<hipblasLtMatmulAlgo_t> candidates;
  for (int i = 0; i < got; ++i)
    if (found[i].state == HIPBLAS_STATUS_SUCCESS && found[i].workspaceSize <= ws_bytes)
      candidates.push_back(found[i].algo);
  if (candidates.empty()) return false;
  measured = false;
  if (candidates.size() == 1) {
    p.algo = candidates[0];
    return true;
  }
  hipEvent_t e0, e1;
  hipEventCreate(&e0);
  hipEventCreate(&e1);
  float best_ms = -1.f, first_ms = -1.f;
  size_t best = 0;
  for (size_t i = 0; i < candidates.size(); ++i) {
    const float ms = time_algo(p, candidates[i], x, w, out, ws, ws_bytes, stream, e0, e1, 3);
    if (i == 0) first_ms = ms;
    if (ms > 0.f && (best_ms < 0.f || ms < best_ms)) {
      best_ms = ms;
      best = i;
    }
  }
  hipEventDestroy(e0);
  hipEventDestroy(e1);
  if (best_ms < 0.f) return false;
  if (std::getenv("TOKAMAK_AMD_LT_VERBOSE") != nullptr)
    fprintf(stderr, "[blas_lt] M=%d N=%d: took candidate %zu of %zu at %.1f us; the library's first choice %.1f us\n",
            M, N, best, candidates.size(), best_ms * 1e3f, first_ms * 1e3f);
  p.algo = candidates[best];
  measured = true;
  return true;
}

}  // namespace

// tune: how many of the library's candidates to time for a new shape class (<= 1: take
// its first choice).  Returns 0, or a negative
// code: -1 bad arguments, -2 no algorithm, -3 the product failed, -10/-11 descriptors.
TK_API int tk_lt_gemm(const void* x, const void* w, void* out, int M, int N, int K, long ldx, long ldw,
                      long ldo, void* workspace, size_t ws_bytes, int tune, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || ldx < K || ldw < K || ldo < N) return -1;
  std::lock_guard<std::mutex> guard(g_lock);
  if (g_handle == nullptr && hipblasLtCreate(&g_handle) != HIPBLAS_STATUS_SUCCESS) return -10;

  const ShapeKey key{M, N, K, ldx, ldw, ldo};
  auto it = g_plans.find(key);
  if (it == g_plans.end()) {
    Plan p;
    if (const int err = make_descriptors(p, M, N, K, ldx, ldw, ldo)) return err;
    const ClassKey cls{(M + kClassRows - 1) / kClassRows, N, K};
    auto known = g_class_algo.find(cls);
    bool have = false;
    if (known != g_class_algo.end()) {
      p.algo = known->second;
      have = usable(p, p.algo, ws_bytes);
    }
    if (!have) {
      bool measured = false;
      if (!choose_algorithm(p, tune, x, w, out, M, N, workspace, ws_bytes, stream, measured)) return -2;
      if (measured) {
        g_class_algo[cls] = p.algo;
        ++g_tuned;
      }
    }
    it = g_plans.emplace(key, p).first;
  }
  Plan& p = it->second;
  return run(p, p.algo, x, w, out, workspace, ws_bytes, stream) == HIPBLAS_STATUS_SUCCESS ? 0 : -3;
}

// How many shape classes have been tuned by measurement so far (for tests and logs).
TK_API long tk_lt_tuned_classes() {
  std::lock_guard<std::mutex> guard(g_lock);
  return g_tuned;
}

// the same entry points in slot form (slots.h), for launch lists
TK_SLOTS(tk_lt_gemm)
