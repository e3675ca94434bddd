// Library matrix products of the bfloat16 path with many rows: hipBLASLt, called directly.
//
//   C[m, n] (+)= sum_k X[m, k] W[n, k]        X [M, K], W [N, K] bfloat16 row-major; C [M, N] bfloat16 or float32
//
// (the reference's engine hands these products to a library as well: F.linear, inference_engine/model.py:172-185).
// Everything here is host code: which of the library's kernels runs a shape is decided here, once per shape, and
// kept.  By default that is the library's own first suggestion; mie_lt_tune() times the library's suggestions
// for one shape on the device and keeps the fastest (the library's order of suggestions is an estimate: at the
// shapes of a decode step of a few hundred rows the best one is often not the first).  A caller tunes the row
// counts it knows will recur (the batch sizes its decode graphs are captured at, the token budget of a step)
// and never inside a stream capture; mie_lt_gemm() itself only looks the shape up and launches, and may be
// captured.
//
// In the library's column-major terms: C^T [N, M] = op(A) B with A = W as stored (a [K, N] matrix of leading
// dimension ldw, transposed), B = X as stored (a [K, M] matrix of leading dimension ldx): a "TN" product.
#include "common.hpp"

#include <hipblaslt/hipblaslt.h>
#include <hipblaslt/hipblaslt-ext.hpp>

#include <algorithm>
#include <map>
#include <mutex>
#include <tuple>
#include <vector>

enum { LT_STORE_BF16 = 0, LT_STORE_F32 = 1, LT_ADD_F32 = 2 };      // what happens to C

namespace {

struct Plan {
  hipblasLtMatmulDesc_t desc = nullptr;
  hipblasLtMatrixLayout_t a = nullptr, b = nullptr, c = nullptr;
  hipblasLtMatmulAlgo_t algo;
  size_t workspace = 0;
  bool tuned = false;
};

typedef std::tuple<int, int, int, int, long, long, long, int> Key;      // device, M, N, K, ldx, ldw, ldc, kind

std::mutex g_lock;
std::map<Key, Plan> g_plans;
hipblasLtHandle_t g_handle[64];

#define LT_CHECK(call, what)                                                                     \
  do {                                                                                           \
    hipblasStatus_t st_ = (call);                                                                \
    if (st_ != HIPBLAS_STATUS_SUCCESS) MIE_FAIL("lt_gemm: %s failed with status %d", what, (int)st_); \
  } while (0)

int handle_for(int dev, hipblasLtHandle_t* h) {
  if (!g_handle[dev]) LT_CHECK(hipblasLtCreate(&g_handle[dev]), "hipblasLtCreate");
  *h = g_handle[dev];
  return 0;
}

// The library's suggestions for a shape, best estimate first.
int suggestions(hipblasLtHandle_t h, const Plan& p, size_t max_workspace, int wanted,
                std::vector<hipblasLtMatmulHeuristicResult_t>& out) {
  hipblasLtMatmulPreference_t pref;
  LT_CHECK(hipblasLtMatmulPreferenceCreate(&pref), "hipblasLtMatmulPreferenceCreate");
  uint64_t ws = max_workspace;
  hipblasStatus_t st = hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &ws, sizeof ws);
  out.resize(wanted);
  int got = 0;
  if (st == HIPBLAS_STATUS_SUCCESS)
    st = hipblasLtMatmulAlgoGetHeuristic(h, p.desc, p.a, p.b, p.c, p.c, pref, wanted, out.data(), &got);
  hipblasLtMatmulPreferenceDestroy(pref);
  if (st != HIPBLAS_STATUS_SUCCESS) MIE_FAIL("lt_gemm: the library has no kernel for this product (status %d)", (int)st);
  out.resize(got > 0 ? got : 0);
  if (out.empty()) MIE_FAIL("lt_gemm: the library suggested no kernel for this product");
  return 0;
}

int make_plan(hipblasLtHandle_t h, Plan& p, int M, int N, int K, long ldx, long ldw, long ldc, int kind, size_t max_workspace) {
  LT_CHECK(hipblasLtMatmulDescCreate(&p.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F), "hipblasLtMatmulDescCreate");
  const int32_t ta = HIPBLAS_OP_T, tb = HIPBLAS_OP_N;
  LT_CHECK(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &ta, sizeof ta), "set TRANSA");
  LT_CHECK(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &tb, sizeof tb), "set TRANSB");
  LT_CHECK(hipblasLtMatrixLayoutCreate(&p.a, HIP_R_16BF, K, N, ldw), "layout of W");
  LT_CHECK(hipblasLtMatrixLayoutCreate(&p.b, HIP_R_16BF, K, M, ldx), "layout of X");
  LT_CHECK(hipblasLtMatrixLayoutCreate(&p.c, kind == LT_STORE_BF16 ? HIP_R_16BF : HIP_R_32F, N, M, ldc), "layout of C");
  // the first of the library's suggestions that runs in the workspace the caller has (the library is told the
  // limit, and still may name kernels that want more)
  std::vector<hipblasLtMatmulHeuristicResult_t> s;
  if (suggestions(h, p, max_workspace, 8, s)) return -1;
  for (const auto& r : s)
    if (r.state == HIPBLAS_STATUS_SUCCESS && r.workspaceSize <= max_workspace) {
      p.algo = r.algo;
      p.workspace = r.workspaceSize;
      return 0;
    }
  MIE_FAIL("lt_gemm: every kernel the library suggests for this product wants more than %zu bytes of workspace", max_workspace);
}

int run(hipblasLtHandle_t h, const Plan& p, const hipblasLtMatmulAlgo_t& algo, const void* X, const void* W, void* C, int kind,
        void* workspace, size_t ws_bytes, hipStream_t s) {
  const float alpha = 1.f, beta = kind == LT_ADD_F32 ? 1.f : 0.f;
  LT_CHECK(hipblasLtMatmul(h, p.desc, &alpha, W, p.a, X, p.b, &beta, C, p.c, C, p.c, &algo, workspace, ws_bytes, s), "hipblasLtMatmul");
  return 0;
}

int check_operands(const char* what, const void* X, long ldx, const void* W, long ldw, const void* C, long ldc, int M, int N, int K,
                   int kind) {
  if (M <= 0 || N <= 0 || K <= 0) MIE_FAIL("%s: sizes %d x %d x %d", what, M, N, K);
  if (kind < LT_STORE_BF16 || kind > LT_ADD_F32) MIE_FAIL("%s: kind %d", what, kind);
  if (!X || !W || !C) MIE_FAIL("%s: null operand", what);
  if (ldx < K || ldw < K || ldc < N) MIE_FAIL("%s: leading dims %ld, %ld, %ld for %d x %d x %d", what, ldx, ldw, ldc, M, N, K);
  return 0;
}

int plan_for(int M, int N, int K, long ldx, long ldw, long ldc, int kind, size_t ws_bytes, hipblasLtHandle_t* h, Plan** plan) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) MIE_FAIL("lt_gemm: no current device");
  if (handle_for(dev, h)) return -1;
  const Key key(dev, M, N, K, ldx, ldw, ldc, kind);
  auto it = g_plans.find(key);
  if (it == g_plans.end()) {
    Plan p;
    if (make_plan(*h, p, M, N, K, ldx, ldw, ldc, kind, ws_bytes)) return -1;
    it = g_plans.emplace(key, p).first;
  }
  *plan = &it->second;
  return 0;
}

}  // namespace

MIE_EXPORT const char* lt_gemm_last_error() { return g_mie_error; }

// C (+)= X W^T on ``stream`` with the kernel kept for this shape (the library's first suggestion unless
// mie_lt_tune chose another).  workspace: device memory the library's kernels may use (16-byte aligned).
MIE_EXPORT int mie_lt_gemm(const void* X, long ldx, const void* W, long ldw, void* C, long ldc, int M, int N, int K, int kind,
                           void* workspace, long ws_bytes, hipStream_t stream) {
  if (check_operands("lt_gemm", X, ldx, W, ldw, C, ldc, M, N, K, kind)) return -1;
  std::lock_guard<std::mutex> hold(g_lock);
  hipblasLtHandle_t h;
  Plan* p;
  if (plan_for(M, N, K, ldx, ldw, ldc, kind, (size_t)ws_bytes, &h, &p)) return -1;
  if (p->workspace > (size_t)ws_bytes) MIE_FAIL("lt_gemm: the kernel chosen for this shape needs %zu bytes of workspace, %ld given", p->workspace, ws_bytes);
  return run(h, *p, p->algo, X, W, C, kind, workspace, (size_t)ws_bytes, stream);
}

// 1 if a kernel was chosen for this shape by timing, 0 if not (yet).
MIE_EXPORT int mie_lt_is_tuned(long ldx, long ldw, long ldc, int M, int N, int K, int kind) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 0;
  std::lock_guard<std::mutex> hold(g_lock);
  auto it = g_plans.find(Key(dev, M, N, K, ldx, ldw, ldc, kind));
  return it != g_plans.end() && it->second.tuned;
}

// Chooses this shape's kernel by timing, on ``stream`` (which must not be capturing).  candidates > 0: that many of
// the library's suggestions; candidates = 0: every kernel the library has for these operand types that takes the
// shape (hundreds).  First every candidate runs ``reps`` times back to back, operands warm; then the eight fastest
// and the library's first suggestion are timed one launch at a time with the weights cold, as a model's step finds
// them: before each launch ``cold`` (cold_bytes of device memory, more than the memory-side cache holds; may be
// null: then the warm times decide) is overwritten.  The first suggestion stays unless another is clearly faster.  C is written (and, for the adding kind, added to) over and over: give a buffer whose contents
// do not matter.  best_us / first_us: the times of the kernel kept and of the library's first suggestion.
MIE_EXPORT int mie_lt_tune(const void* X, long ldx, const void* W, long ldw, void* C, long ldc, int M, int N, int K, int kind,
                           void* workspace, long ws_bytes, int candidates, int reps, void* cold, long cold_bytes,
                           float* best_us, float* first_us, hipStream_t stream) {
  if (check_operands("lt_tune", X, ldx, W, ldw, C, ldc, M, N, K, kind)) return -1;
  if (candidates < 0 || reps < 1) MIE_FAIL("lt_tune: %d candidates, %d repetitions", candidates, reps);
  hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &capturing) != hipSuccess || capturing != hipStreamCaptureStatusNone)
    MIE_FAIL("lt_tune: the stream is being captured; kernels are chosen before a capture, not inside one");
  std::lock_guard<std::mutex> hold(g_lock);
  hipblasLtHandle_t h;
  Plan* p;
  if (plan_for(M, N, K, ldx, ldw, ldc, kind, (size_t)ws_bytes, &h, &p)) return -1;
  std::vector<hipblasLtMatmulHeuristicResult_t> s;
  if (suggestions(h, *p, (size_t)ws_bytes, candidates > 0 ? candidates : 1, s)) return -1;      // the first suggestion leads
  if (candidates == 0) {
    std::vector<hipblasLtMatmulHeuristicResult_t> all;
    const hipDataType tc = kind == LT_STORE_BF16 ? HIP_R_16BF : HIP_R_32F;
    if (hipblaslt_ext::getAllAlgos(h, hipblaslt_ext::GemmType::HIPBLASLT_GEMM, HIPBLAS_OP_T, HIPBLAS_OP_N, HIP_R_16BF, HIP_R_16BF,
                                   tc, tc, HIPBLAS_COMPUTE_32F, all) == HIPBLAS_STATUS_SUCCESS) {
      const float alpha = 1.f, beta = kind == LT_ADD_F32 ? 1.f : 0.f;
      for (auto& r : all) {
        size_t need = 0;
        if (hipblaslt_ext::matmulIsAlgoSupported(h, p->desc, &alpha, p->a, p->b, &beta, p->c, p->c, r.algo, need) != HIPBLAS_STATUS_SUCCESS)
          continue;
        r.workspaceSize = need;
        r.state = HIPBLAS_STATUS_SUCCESS;
        s.push_back(r);
      }
    }
  }
  hipEvent_t e0, e1;
  if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) MIE_FAIL("lt_tune: cannot create events");
  // what one timing of candidate i gives: microseconds a launch, or a negative number if it does not run
  auto time_of = [&](size_t i, int launches, bool cold_first) -> float {
    if (cold_first && hipMemsetAsync(cold, 0, (size_t)cold_bytes, stream) != hipSuccess) return -1.f;
    hipEventRecord(e0, stream);
    for (int r = 0; r < launches; ++r)
      if (run(h, *p, s[i].algo, X, W, C, kind, workspace, (size_t)ws_bytes, stream)) return -1.f;
    hipEventRecord(e1, stream);
    if (hipEventSynchronize(e1) != hipSuccess) return -2.f;
    float ms = 0.f;
    hipEventElapsedTime(&ms, e0, e1);
    return ms * 1000.f / launches;
  };
  std::vector<std::pair<float, size_t>> warm;
  float first = 0.f;
  int rc = 0;
  for (size_t i = 0; i < s.size(); ++i) {
    if (s[i].state != HIPBLAS_STATUS_SUCCESS || s[i].workspaceSize > (size_t)ws_bytes) continue;
    if (run(h, *p, s[i].algo, X, W, C, kind, workspace, (size_t)ws_bytes, stream)) continue;      // (loads the kernel) one that does not run is skipped
    const float us = time_of(i, reps, false);
    if (us == -2.f) { rc = -1; break; }
    if (us < 0.f) continue;
    if (i == 0) first = us;
    warm.emplace_back(us, i);
  }
  if (rc == 0 && warm.empty()) {
    snprintf(g_mie_error, sizeof g_mie_error, "lt_tune: none of the library's kernels ran");
    rc = -1;
  }
  float best = 1e30f;
  if (rc == 0) {
    std::sort(warm.begin(), warm.end());
    const bool use_cold = cold && cold_bytes > 0;
    const size_t finalists = use_cold ? (warm.size() < 8 ? warm.size() : 8) : 1;
    size_t keep = warm[0].second;
    if (use_cold) {
      bool first_in = false;
      for (size_t f = 0; f < finalists; ++f) first_in |= warm[f].second == 0;
      std::vector<size_t> order;
      for (size_t f = 0; f < finalists; ++f) order.push_back(warm[f].second);
      if (!first_in && s[0].state == HIPBLAS_STATUS_SUCCESS) order.push_back(0);       // the library's own choice always competes
      // the least of 2 x reps cold launches each (the least is what interference from outside cannot lower);
      // another kernel replaces the library's own choice only if it is clearly faster: a microsecond and 3 %
      float first_cold = -1.f;
      for (size_t i : order) {
        float least = 1e30f;
        bool ok = true;
        for (int r = 0; r < 2 * reps && ok; ++r) {
          const float us = time_of(i, 1, true);
          ok = us >= 0.f;
          if (us < least) least = us;
        }
        if (!ok) continue;
        if (i == 0) first_cold = least;
        if (least < best) { best = least; keep = i; }
      }
      if (first_cold > 0.f) {
        first = first_cold;
        if (keep != 0 && best > first_cold - (1.0f > 0.03f * first_cold ? 1.0f : 0.03f * first_cold)) {
          keep = 0;
          best = first_cold;
        }
      }
    } else {
      best = warm[0].first;
    }
    p->algo = s[keep].algo;
    p->workspace = s[keep].workspaceSize;
    p->tuned = true;
  }
  hipEventDestroy(e0);
  hipEventDestroy(e1);
  if (rc) return rc;
  if (best_us) *best_us = best;
  if (first_us) *first_us = first;
  return 0;
}
