// Dense products of bfloat16 operands through hipBLASLt's C interface:
//   out[rows, n_out] = x[rows, width] . w[n_out, width]^T,   32-bit accumulation, out bfloat16 or float32.
// (The reference uses the vendor's library for the same products, src/backends/cuda/ops/gemm.cu; its grouped and
// skinny products are kernels of its own, as here.)  Called straight from here a product costs the host about
// 10 us instead of the 19 us that the same call costs through the tensor library.  Which of the library's kernels
// forms a shape is decided at the shape's first product outside a capture: the library names its candidates in the
// order of its own guess, each of the first sixteen forms the product, timed, and the quickest is kept for the
// shape if it needs less than 0.85 of the first one's time, else the first (INFERX_GEMM_CANDIDATES=1: always the
// first, which is also what the tensor library takes).  Measured alone: 256 rows x 6,144 x 2,048: 14.7 against
// 20.4 us; 1,056 x 3,584 x 20,480: 160 against 231; 2,048 x 3,584 x 20,480: 243 against 396; most other shapes 2 to
// 10 %, which the margin leaves alone.  In the model: a mixed step of 1,056 tokens at the larger shape 46.2 against
// 47.8 ms, a portion of 256 tokens at the smaller 6.42 against 6.58.  The trial costs a new shape about 64 products
// of its own size, once.
//
// A product may use a workspace (the library's split and stream-K kernels do).  Products on different streams may
// run at the same time, so a stream gets a workspace of its own, 64 MB, at its first product whose kernel asks for
// one (most ask for none, and then nothing is allocated); that product must not be recorded into a graph (the engine
// warms a stream up with the same shapes before it captures on it).  Workspaces live until the process ends.  The
// plans (one per shape: a descriptor, three layouts, the chosen kernel) are kept for the kMaxPlans shapes used last;
// steps of many different token counts would otherwise add one per count without bound.
#include <hipblaslt/hipblaslt.h>

#include <algorithm>
#include <cstdlib>
#include <map>
#include <mutex>
#include <tuple>
#include <utility>
#include <vector>

#include "common.h"

namespace {

constexpr size_t kWorkspaceBytes = size_t(64) << 20;
constexpr size_t kMaxPlans = 1024;

constexpr int kMaxCandidates = 16;
constexpr int kDefaultCandidates = 16;
constexpr int kTuneRuns = 3;
constexpr float kKeepFirstWithin = 0.85f;

struct Choice {
  hipblasLtMatmulAlgo_t algo;
  size_t workspace;
};

struct Plan {
  bool usable = false;
  std::vector<Choice> choices;  // the library's candidates while the plan waits to be tuned (empty afterwards)
  hipblasLtMatmulDesc_t desc = nullptr;
  hipblasLtMatrixLayout_t w = nullptr, x = nullptr, out = nullptr;
  hipblasLtMatmulAlgo_t algo;
  size_t workspace = 0;
  uint64_t last_use = 0;
};

void destroy(Plan& p) {
  if (p.w) hipblasLtMatrixLayoutDestroy(p.w);
  if (p.x) hipblasLtMatrixLayoutDestroy(p.x);
  if (p.out) hipblasLtMatrixLayoutDestroy(p.out);
  if (p.desc) hipblasLtMatmulDescDestroy(p.desc);
  p = Plan();
}

struct PerDevice {
  hipblasLtHandle_t handle = nullptr;
  std::map<std::tuple<int64_t, int64_t, int64_t, int>, Plan> plans;
  std::map<hipStream_t, void*> workspaces;
  uint64_t clock = 0;
};

// Drops the half of the plans that were used longest ago.
void forget_old_plans(PerDevice& dev) {
  std::vector<uint64_t> uses;
  for (auto& kv : dev.plans) uses.push_back(kv.second.last_use);
  std::nth_element(uses.begin(), uses.begin() + uses.size() / 2, uses.end());
  const uint64_t cut = uses[uses.size() / 2];
  for (auto it = dev.plans.begin(); it != dev.plans.end();) {
    if (it->second.last_use < cut) {
      destroy(it->second);
      it = dev.plans.erase(it);
    } else {
      ++it;
    }
  }
}

std::mutex g_mutex;
std::map<int, PerDevice> g_devices;
int g_candidates = -1;  // how many of the library's candidates a new shape is tried with; -1: not read yet

int candidates_wanted() {
  if (g_candidates < 0) {
    const char* env = getenv("INFERX_GEMM_CANDIDATES");
    g_candidates = env ? std::max(1, std::min(atoi(env), kMaxCandidates)) : kDefaultCandidates;
  }
  return g_candidates;
}

bool capturing(hipStream_t stream) {
  hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &status) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  return status != hipStreamCaptureStatusNone;
}

// The library is column-major: out^T [n_out, rows] = op_T(w as [width, n_out]) . (x as [width, rows]).
int make_plan(PerDevice& dev, Plan& p, int64_t rows, int64_t n_out, int64_t width, int out_f32, int candidates) {
  if (hipblasLtMatmulDescCreate(&p.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F) != HIPBLAS_STATUS_SUCCESS) return 1;
  const hipblasOperation_t transposed = HIPBLAS_OP_T, plain = HIPBLAS_OP_N;
  if (hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &transposed, sizeof(transposed)) !=
          HIPBLAS_STATUS_SUCCESS ||
      hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &plain, sizeof(plain)) !=
          HIPBLAS_STATUS_SUCCESS)
    return 1;
  if (hipblasLtMatrixLayoutCreate(&p.w, HIP_R_16BF, width, n_out, width) != HIPBLAS_STATUS_SUCCESS ||
      hipblasLtMatrixLayoutCreate(&p.x, HIP_R_16BF, width, rows, width) != HIPBLAS_STATUS_SUCCESS ||
      hipblasLtMatrixLayoutCreate(&p.out, out_f32 ? HIP_R_32F : HIP_R_16BF, n_out, rows, n_out) !=
          HIPBLAS_STATUS_SUCCESS)
    return 1;
  hipblasLtMatmulPreference_t pref = nullptr;
  if (hipblasLtMatmulPreferenceCreate(&pref) != HIPBLAS_STATUS_SUCCESS) return 1;
  size_t limit = kWorkspaceBytes;
  hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &limit, sizeof(limit));
  hipblasLtMatmulHeuristicResult_t found[kMaxCandidates];
  int n = 0;
  const int asked = std::max(1, std::min(candidates, kMaxCandidates));
  const hipblasStatus_t st =
      hipblasLtMatmulAlgoGetHeuristic(dev.handle, p.desc, p.w, p.x, p.out, p.out, pref, asked, found, &n);
  hipblasLtMatmulPreferenceDestroy(pref);
  if (st != HIPBLAS_STATUS_SUCCESS) return 0;
  for (int i = 0; i < n; ++i)
    if (found[i].state == HIPBLAS_STATUS_SUCCESS && found[i].workspaceSize <= kWorkspaceBytes)
      p.choices.push_back({found[i].algo, found[i].workspaceSize});
  if (!p.choices.empty()) {
    p.algo = p.choices[0].algo;
    p.workspace = p.choices[0].workspace;
    p.usable = true;
  }
  if (p.choices.size() < 2) p.choices.clear();  // nothing to choose between
  return 0;
}

}  // namespace

// How many of the library's candidate kernels a shape's first product tries (1: the library's first choice, no
// timing).  Shapes already planned keep their kernel.
extern "C" int ix_gemm_set_candidates(int candidates) {
  IX_REQUIRE(candidates >= 1 && candidates <= kMaxCandidates, "between 1 and 16 candidates");
  std::lock_guard<std::mutex> lock(g_mutex);
  g_candidates = candidates;
  return 0;
}

// Returns 0 when the product was queued, 1 on an error (see ix_last_error), and 2 when the library has no kernel
// for the shape (nothing was queued; the caller takes another route).
extern "C" int ix_gemm_bf16(const void* x, const void* w, void* out, int64_t rows, int64_t n_out, int64_t width,
                            int out_f32, hipStream_t stream) {
  IX_REQUIRE(x && w && out, "operands are missing");
  IX_REQUIRE(rows > 0 && n_out > 0 && width > 0, "sizes must be positive");
  IX_REQUIRE(rows < (int64_t(1) << 31) && n_out < (int64_t(1) << 31) && width < (int64_t(1) << 31), "sizes too large");
  int device = 0;
  IX_REQUIRE(hipGetDevice(&device) == hipSuccess, "no current device");
  std::lock_guard<std::mutex> lock(g_mutex);
  PerDevice& dev = g_devices[device];
  if (!dev.handle)
    IX_REQUIRE(hipblasLtCreate(&dev.handle) == HIPBLAS_STATUS_SUCCESS, "hipblasLtCreate failed");
  const auto key = std::make_tuple(rows, n_out, width, out_f32);
  auto it = dev.plans.find(key);
  if (it == dev.plans.end()) {
    if (dev.plans.size() >= kMaxPlans) forget_old_plans(dev);
    Plan p;
    if (make_plan(dev, p, rows, n_out, width, out_f32, candidates_wanted()) != 0) {
      destroy(p);
      IX_REQUIRE(false, "hipBLASLt refused the product's description");
    }
    it = dev.plans.emplace(key, p).first;
  }
  Plan& p = it->second;
  p.last_use = ++dev.clock;
  if (!p.usable) return 2;
  const float one = 1.0f, zero = 0.0f;
  auto workspace_of = [&](size_t needed, void** workspace) -> int {
    *workspace = nullptr;
    if (needed == 0) return 0;
    auto ws = dev.workspaces.find(stream);
    if (ws == dev.workspaces.end() && !capturing(stream)) {
      void* mem = nullptr;
      IX_REQUIRE(hipMalloc(&mem, kWorkspaceBytes) == hipSuccess, "no memory for the products' workspace");
      ws = dev.workspaces.emplace(stream, mem).first;
    }
    IX_REQUIRE(ws != dev.workspaces.end(),
               "a stream's first product that needs a workspace allocates it and cannot be recorded into a graph");
    *workspace = ws->second;
    return 0;
  };
  if (!p.choices.empty() && !capturing(stream)) {
    // The shape's first product outside a capture: each of the library's candidates forms it (the same result
    // up to rounding, into `out`), timed on this stream, and the quickest is kept.  The library's own order is
    // a guess: for some shapes of few rows its first choice takes three times as long as its best.
    hipEvent_t t0 = nullptr, t1 = nullptr;
    if (hipEventCreate(&t0) == hipSuccess && hipEventCreate(&t1) == hipSuccess) {
      float best = 0.f, first = 0.f;
      int best_i = -1;
      for (size_t i = 0; i < p.choices.size(); ++i) {
        void* ws = nullptr;
        if (workspace_of(p.choices[i].workspace, &ws)) break;
        bool ok = true;
        float ms = 0.f;
        for (int run = 0; run <= kTuneRuns && ok; ++run) {  // (the first run is not timed)
          if (run == 1) ok = hipEventRecord(t0, stream) == hipSuccess;
          ok = ok && hipblasLtMatmul(dev.handle, p.desc, &one, w, p.w, x, p.x, &zero, out, p.out, out, p.out,
                                     &p.choices[i].algo, ws, p.choices[i].workspace, stream) == HIPBLAS_STATUS_SUCCESS;
        }
        ok = ok && hipEventRecord(t1, stream) == hipSuccess && hipEventSynchronize(t1) == hipSuccess &&
             hipEventElapsedTime(&ms, t0, t1) == hipSuccess;
        if (!ok) {
          (void)hipGetLastError();
          continue;
        }
        if (i == 0) first = ms;
        if (best_i < 0 || ms < best) {
          best = ms;
          best_i = static_cast<int>(i);
        }
      }
      // (the library's own first choice stays unless another is clearly quicker: which kernel forms a shape then
      // does not hang on a few per cent of one trial's timing)
      if (best_i > 0 && first > 0.f && best > kKeepFirstWithin * first) best_i = 0;
      if (best_i >= 0) {
        p.algo = p.choices[best_i].algo;
        p.workspace = p.choices[best_i].workspace;
      }
    }
    if (t0) (void)hipEventDestroy(t0);
    if (t1) (void)hipEventDestroy(t1);
    p.choices.clear();
  }
  void* workspace = nullptr;
  if (workspace_of(p.workspace, &workspace)) return 1;
  const hipblasStatus_t st = hipblasLtMatmul(dev.handle, p.desc, &one, w, p.w, x, p.x, &zero, out, p.out, out, p.out,
                                             &p.algo, workspace, p.workspace, stream);
  if (st != HIPBLAS_STATUS_SUCCESS) {
    ix_set_error("hipblasLtMatmul failed with status " + std::to_string(static_cast<int>(st)));
    return 1;
  }
  return 0;
}
