// Router scores, selection and grouping for up to 16 tokens (decoding) in ONE launch:
// softmax and top-k of every token's router scores, then counts, offsets, the stable
// placement and the row-tile map.  Same arithmetic and tie rule as moe_route_kernel /
// moe_dispatch_wide_kernel in moe.hip (reference: RouteTopKKernel
// src/backends/cuda/ops/moe.cu:36-127, MoeBuildDispatch :452-513).
#include "common.h"
#include "moe_route.h"

// At most 16 tokens: scores, selection and grouping in ONE launch.  The router rows are spread over many
// workgroups, one row per wavefront, as in moe_route_logits_kernel (moe.hip); every workgroup counts itself
// off, and the one that finds all others counted goes on to select and group.
//
// The workgroups run on different dies, each with an L2 of its own.  The scores therefore travel as
// device-scope (relaxed atomic) stores and loads, which go through to where all dies see them; a wavefront
// waits for its stores' acknowledgement before its workgroup is counted.  Fences would do too, but each one
// writes back and invalidates a whole L2 (measured: 0.06 us per workgroup and launch, 20 us here).
// `arrived` is an int32 that is zero before the launch; the last workgroup sets it back to zero.
#define RF_THREADS 1024
#define RF_MAX_PER_THREAD 10  // columns of a row per thread: 40 KB of float32 over 1,024 threads
// NORM: the token's row is formed here as well, x = rmsnorm(h + delta) * gamma rounded to T as the separate norm
// kernel would leave it (every workgroup of a token forms it for itself; the first of them writes it to x_out),
// and the last of a token's workgroups to have read h[t] (they count themselves off per token as well) writes
// h[t] + delta[t] back: the residual stream is up to date when the launch ends.
template <typename T, bool NORM>
__global__ void __launch_bounds__(RF_THREADS)
moe_route_dispatch_small_kernel(const T* __restrict__ x, float* h, const T* __restrict__ delta,
                                const void* __restrict__ gamma, int gamma_dtype, float eps, T* __restrict__ x_out,
                                const void* __restrict__ wr, int wr_dtype,
                                const void* __restrict__ shared_gate_w, int sg_dtype, float* logits,
                                int32_t* arrived, int64_t width, float* __restrict__ topk_w,
                                int32_t* __restrict__ topk_e, float* __restrict__ shared_gate,
                                int32_t* __restrict__ offsets, int32_t* __restrict__ rows, int32_t* __restrict__ dest,
                                int tokens, int experts, int k, int renormalize, float scale, int tile_rows,
                                int32_t* __restrict__ tile_expert, int32_t* __restrict__ tile_row0,
                                int32_t* __restrict__ tile_info) {
  extern __shared__ __align__(16) float xs[];  // [width]
  __shared__ int is_last, updates_h;
  __shared__ float red[16];
  const int64_t t = blockIdx.x;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  float v[RF_MAX_PER_THREAD];  // NORM: this thread's columns of h[t] + delta[t]
  int ticket = 0;
  // this wavefront's router row: its first pieces are asked for now and arrive while the token's row is formed
  const int n_rows = experts + (shared_gate_w ? 1 : 0);
  const int e = blockIdx.y * (RF_THREADS / 64) + wave;
  const bool routed = e < experts;
  const void* w_row = routed ? wr : shared_gate_w;
  const int64_t w_base = routed ? static_cast<int64_t>(e) * width : 0;
  const bool preloaded = e < n_rows && route_row_preloadable(w_row, routed ? wr_dtype : sg_dtype, width);
  uint4 w_pre[ROUTE_PRELOAD];
  if (preloaded) route_row_preload(w_row, w_base, width, lane, w_pre);
  if (NORM) {
    const float* hr = h + t * width;
    const T* dr = delta + t * width;
    // (RF_MAX_PER_THREAD columns per thread at most: the entry point bounds the width; all loads are asked for
    // before the first is used, the norm weight's too)
    float gm[RF_MAX_PER_THREAD];
    float sumsq = 0.f;
#pragma unroll
    for (int u = 0; u < RF_MAX_PER_THREAD; ++u) {
      const int64_t i = tid + static_cast<int64_t>(u) * RF_THREADS;
      const bool in = i < width;
      v[u] = in ? hr[i] + ix_load(dr + i) : 0.f;
      gm[u] = in ? ix_load_rt(gamma, gamma_dtype, i) : 0.f;
    }
#pragma unroll
    for (int u = 0; u < RF_MAX_PER_THREAD; ++u) sumsq += v[u] * v[u];
    sumsq = ix_block_sum(sumsq, red);
    // every thread's part of h[t] has arrived: this workgroup is counted among those that have read the row
    // (the count comes back while the scores are formed)
    if (tid == 0) ticket = __hip_atomic_fetch_add(arrived + 1 + t, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const float inv = 1.0f / sqrtf(sumsq / static_cast<float>(width) + eps);
#pragma unroll
    for (int u = 0; u < RF_MAX_PER_THREAD; ++u) {
      const int64_t i = tid + static_cast<int64_t>(u) * RF_THREADS;
      if (i < width) {
        T rounded;
        ix_store(&rounded, v[u] * inv * gm[u]);
        xs[i] = ix_load(&rounded);
        if (blockIdx.y == 0) x_out[t * width + i] = rounded;
      }
    }
  } else {
    for (int64_t i = tid; i < width; i += RF_THREADS) xs[i] = ix_load(x + t * width + i);
  }
  __syncthreads();
  if (e < n_rows) {
    const float dot = preloaded ? route_row_dot_preloaded(xs, w_row, w_base, width, lane, w_pre)
                                : route_row_dot(xs, w_row, routed ? wr_dtype : sg_dtype, w_base, width, lane);
    if (lane == 0) __hip_atomic_store(&logits[t * (experts + 1) + e], dot, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  __builtin_amdgcn_s_waitcnt(0);  // this wavefront's loads have arrived and its store has been acknowledged
  __syncthreads();
  if (tid == 0) {
    is_last = __hip_atomic_fetch_add(arrived, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) ==
              static_cast<int>(gridDim.x * gridDim.y) - 1;
    updates_h = NORM && ticket == static_cast<int>(gridDim.y) - 1;
  }
  __syncthreads();
  if (NORM && updates_h) {  // the token's other workgroups have read h[t]: it becomes h[t] + delta[t]
    if (tid == 0) __hip_atomic_store(arrived + 1 + t, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
    for (int u = 0; u < RF_MAX_PER_THREAD; ++u) {
      const int64_t i = tid + static_cast<int64_t>(u) * RF_THREADS;
      if (i < width) h[t * width + i] = v[u];
    }
  }
  if (!is_last) return;
  if (tid == 0) __hip_atomic_store(arrived, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  if (tokens * k <= SD_FEW_ASSIGN)
    select_dispatch_few<RF_THREADS / 64>(logits, topk_w, topk_e, shared_gate, offsets, rows, dest, tokens, experts,
                                         k, renormalize, scale, tile_rows, tile_expert, tile_row0, tile_info);
  else
    select_dispatch_body<RF_THREADS / 64>(logits, topk_w, topk_e, shared_gate, offsets, rows, dest, tokens,
                                          experts, k, renormalize, scale, tile_rows, tile_expert, tile_row0,
                                          tile_info);
}

static int route_dispatch_small_launch(const void* x, float* h, const void* delta, const void* gamma, int gamma_dtype,
                                       float eps, void* x_out, int dtype, const void* wr, int wr_dtype,
                                       const void* shared_gate_w, int sg_dtype, float* logits, int32_t* arrived,
                                       int64_t width, float* topk_w, int32_t* topk_e, float* shared_gate,
                                       int32_t* offsets, int32_t* rows, int32_t* dest, int tokens, int experts,
                                       int k, int renormalize, float scale, int tile_rows, int32_t* tile_expert,
                                       int32_t* tile_row0, int32_t* tile_info, hipStream_t stream) {
  IX_REQUIRE(tokens > 0 && tokens <= 16 && experts > 0 && k > 0 && width > 0, "between 1 and 16 tokens, sizes positive");
  IX_REQUIRE(dtype == IX_F32 || dtype == IX_BF16, "dtype must be float32 or bfloat16");
  IX_REQUIRE(experts <= SD_MAX_EXPERTS, "at most 256 experts for the one-workgroup selection");
  IX_REQUIRE(k <= experts && k <= 32, "top_k must be between 1 and min(experts, 32)");
  IX_REQUIRE(static_cast<int64_t>(tokens) * k <= SD_MAX_ASSIGN, "at most 1024 assignments for the one-workgroup selection");
  IX_REQUIRE(tile_rows >= 0, "tile_rows must not be negative");
  IX_REQUIRE(tile_rows == 0 || (tile_expert && tile_row0 && tile_info), "tile map buffers needed");
  IX_REQUIRE(logits && arrived, "the scores' scratch and the arrival counter are needed");
  const size_t xs_bytes = ((width + 3) & ~3) * sizeof(float);
  IX_REQUIRE(xs_bytes <= 40 * 1024, "hidden width too large for the router kernel (limit about 10000)");
  const int n_rows = experts + (shared_gate_w ? 1 : 0);
  dim3 grid(tokens, (n_rows + RF_THREADS / 64 - 1) / (RF_THREADS / 64)), block(RF_THREADS);
#define LAUNCH(T, NORM)                                                                                             \
  hipLaunchKernelGGL((moe_route_dispatch_small_kernel<T, NORM>), grid, block, xs_bytes, stream, (const T*)x, h,     \
                     (const T*)delta, gamma, gamma_dtype, eps, (T*)x_out, wr, wr_dtype, shared_gate_w, sg_dtype,    \
                     logits, arrived, width, topk_w, topk_e, shared_gate, offsets, rows, dest, tokens, experts, k,  \
                     renormalize, scale, tile_rows, tile_expert, tile_row0, tile_info)
  if (h) {
    if (dtype == IX_F32) LAUNCH(float, true);
    else LAUNCH(bf16_t, true);
  } else {
    if (dtype == IX_F32) LAUNCH(float, false);
    else LAUNCH(bf16_t, false);
  }
#undef LAUNCH
  return ix_check_launch("ix_moe_route_dispatch_small");
}

// x [tokens <= 16, width]; logits float32 [tokens, experts + 1] (scratch); arrived: 17 int32 (one for the launch, one
// per token), zero, left zero.
// Calls that share `arrived` must not overlap.
extern "C" int ix_moe_route_dispatch_small(const void* x, int dtype, const void* wr, int wr_dtype,
                                           const void* shared_gate_w, int sg_dtype, float* logits, int32_t* arrived,
                                           int64_t width, float* topk_w, int32_t* topk_e, float* shared_gate,
                                           int32_t* offsets, int32_t* rows, int32_t* dest, int tokens, int experts,
                                           int k, int renormalize, float scale, int tile_rows, int32_t* tile_expert,
                                           int32_t* tile_row0, int32_t* tile_info, hipStream_t stream) {
  IX_REQUIRE(x != nullptr, "x needed");
  return route_dispatch_small_launch(x, nullptr, nullptr, nullptr, IX_F32, 0.f, nullptr, dtype, wr, wr_dtype,
                                     shared_gate_w, sg_dtype, logits, arrived, width, topk_w, topk_e, shared_gate,
                                     offsets, rows, dest, tokens, experts, k, renormalize, scale, tile_rows,
                                     tile_expert, tile_row0, tile_info, stream);
}

// The same with the norm before it: x_out = rmsnorm(h + delta) * gamma (in `dtype`, as ix_add_rmsnorm leaves it)
// is what is routed, and h [tokens, width] float32 becomes h + delta.  delta and x_out are of `dtype`.
extern "C" int ix_moe_norm_route_dispatch_small(float* h, const void* delta, int dtype, const void* gamma,
                                                int gamma_dtype, float eps, void* x_out, const void* wr, int wr_dtype,
                                                const void* shared_gate_w, int sg_dtype, float* logits,
                                                int32_t* arrived, int64_t width, float* topk_w, int32_t* topk_e,
                                                float* shared_gate, int32_t* offsets, int32_t* rows, int32_t* dest,
                                                int tokens, int experts, int k, int renormalize, float scale,
                                                int tile_rows, int32_t* tile_expert, int32_t* tile_row0,
                                                int32_t* tile_info, hipStream_t stream) {
  IX_REQUIRE(h && delta && gamma && x_out, "h, delta, gamma and x_out needed");
  IX_REQUIRE(gamma_dtype == IX_F32 || gamma_dtype == IX_BF16, "the norm weight must be float32 or bfloat16");
  return route_dispatch_small_launch(nullptr, h, delta, gamma, gamma_dtype, eps, x_out, dtype, wr, wr_dtype,
                                     shared_gate_w, sg_dtype, logits, arrived, width, topk_w, topk_e, shared_gate,
                                     offsets, rows, dest, tokens, experts, k, renormalize, scale, tile_rows,
                                     tile_expert, tile_row0, tile_info, stream);
}
