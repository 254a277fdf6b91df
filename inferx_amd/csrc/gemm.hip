// Dense products of bfloat16 operands through hipBLASLt's C interface:
//   out[rows, n_out] = x[rows, width] . w[n_out, width]^T,   32-bit accumulation, out bfloat16 or float32.
// (The reference uses the vendor's library for the same products, src/backends/cuda/ops/gemm.cu; its grouped and
// skinny products are kernels of its own, as here.)  Called straight from here a product costs the host about
// 10 us instead of the 19 us that the same call costs through the tensor library, and gives the same bits: the
// library's first heuristic choice for the shape, asked for once per shape and kept.
//
// A product may use a workspace (the library's split and stream-K kernels do).  Products on different streams may
// run at the same time, so a stream gets a workspace of its own, 64 MB, at its first product whose kernel asks for
// one (most ask for none, and then nothing is allocated); that product must not be recorded into a graph (the engine
// warms a stream up with the same shapes before it captures on it).  Workspaces live until the process ends.  The
// plans (one per shape: a descriptor, three layouts, the chosen kernel) are kept for the kMaxPlans shapes used last;
// steps of many different token counts would otherwise add one per count without bound.
#include <hipblaslt/hipblaslt.h>

#include <algorithm>
#include <map>
#include <mutex>
#include <tuple>
#include <utility>
#include <vector>

#include "common.h"

namespace {

constexpr size_t kWorkspaceBytes = size_t(64) << 20;
constexpr size_t kMaxPlans = 1024;

struct Plan {
  bool usable = false;
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

bool capturing(hipStream_t stream) {
  hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &status) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  return status != hipStreamCaptureStatusNone;
}

// The library is column-major: out^T [n_out, rows] = op_T(w as [width, n_out]) . (x as [width, rows]).
int make_plan(PerDevice& dev, Plan& p, int64_t rows, int64_t n_out, int64_t width, int out_f32) {
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
  hipblasLtMatmulHeuristicResult_t found[1];
  int n = 0;
  const hipblasStatus_t st =
      hipblasLtMatmulAlgoGetHeuristic(dev.handle, p.desc, p.w, p.x, p.out, p.out, pref, 1, found, &n);
  hipblasLtMatmulPreferenceDestroy(pref);
  if (st == HIPBLAS_STATUS_SUCCESS && n > 0 && found[0].state == HIPBLAS_STATUS_SUCCESS &&
      found[0].workspaceSize <= kWorkspaceBytes) {
    p.algo = found[0].algo;
    p.workspace = found[0].workspaceSize;
    p.usable = true;
  }
  return 0;
}

}  // namespace

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
    if (make_plan(dev, p, rows, n_out, width, out_f32) != 0) {
      destroy(p);
      IX_REQUIRE(false, "hipBLASLt refused the product's description");
    }
    it = dev.plans.emplace(key, p).first;
  }
  Plan& p = it->second;
  p.last_use = ++dev.clock;
  if (!p.usable) return 2;
  void* workspace = nullptr;
  if (p.workspace > 0) {
    auto ws = dev.workspaces.find(stream);
    if (ws == dev.workspaces.end() && !capturing(stream)) {
      void* mem = nullptr;
      IX_REQUIRE(hipMalloc(&mem, kWorkspaceBytes) == hipSuccess, "no memory for the products' workspace");
      ws = dev.workspaces.emplace(stream, mem).first;
    }
    IX_REQUIRE(ws != dev.workspaces.end(),
               "a stream's first product that needs a workspace allocates it and cannot be recorded into a graph");
    workspace = ws->second;
  }
  const float one = 1.0f, zero = 0.0f;
  const hipblasStatus_t st = hipblasLtMatmul(dev.handle, p.desc, &one, w, p.w, x, p.x, &zero, out, p.out, out, p.out,
                                             &p.algo, workspace, p.workspace, stream);
  if (st != HIPBLAS_STATUS_SUCCESS) {
    ix_set_error("hipblasLtMatmul failed with status " + std::to_string(static_cast<int>(st)));
    return 1;
  }
  return 0;
}
