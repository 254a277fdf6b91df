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
template <typename T>
__global__ void __launch_bounds__(RF_THREADS)
moe_route_dispatch_small_kernel(const T* __restrict__ x, const void* __restrict__ wr, int wr_dtype,
                                const void* __restrict__ shared_gate_w, int sg_dtype, float* logits,
                                int32_t* arrived, int64_t width, float* __restrict__ topk_w,
                                int32_t* __restrict__ topk_e, float* __restrict__ shared_gate,
                                int32_t* __restrict__ offsets, int32_t* __restrict__ rows, int32_t* __restrict__ dest,
                                int tokens, int experts, int k, int renormalize, float scale, int tile_rows,
                                int32_t* __restrict__ tile_expert, int32_t* __restrict__ tile_row0,
                                int32_t* __restrict__ tile_info) {
  extern __shared__ __align__(16) float xs[];  // [width]
  __shared__ int is_last;
  const int64_t t = blockIdx.x;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  for (int64_t i = tid; i < width; i += RF_THREADS) xs[i] = ix_load(x + t * width + i);
  __syncthreads();
  const int n_rows = experts + (shared_gate_w ? 1 : 0);
  const int e = blockIdx.y * (RF_THREADS / 64) + wave;
  if (e < n_rows) {
    const bool routed = e < experts;
    const float dot = route_row_dot(xs, routed ? wr : shared_gate_w, routed ? wr_dtype : sg_dtype,
                                    routed ? static_cast<int64_t>(e) * width : 0, width, lane);
    if (lane == 0) __hip_atomic_store(&logits[t * (experts + 1) + e], dot, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  __builtin_amdgcn_s_waitcnt(0);  // this wavefront's store has been acknowledged
  __syncthreads();
  if (tid == 0)
    is_last = __hip_atomic_fetch_add(arrived, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) ==
              static_cast<int>(gridDim.x * gridDim.y) - 1;
  __syncthreads();
  if (!is_last) return;
  if (tid == 0) __hip_atomic_store(arrived, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  select_dispatch_body<RF_THREADS / 64>(logits, topk_w, topk_e, shared_gate, offsets, rows, dest, tokens,
                                              experts, k, renormalize, scale, tile_rows, tile_expert, tile_row0,
                                              tile_info);
}

// x [tokens <= 16, width]; logits float32 [tokens, experts + 1] (scratch); arrived: one int32, zero, left zero.
// Calls that share `arrived` must not overlap.
extern "C" int ix_moe_route_dispatch_small(const void* x, int dtype, const void* wr, int wr_dtype,
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
  if (dtype == IX_F32)
    hipLaunchKernelGGL(moe_route_dispatch_small_kernel<float>, grid, block, xs_bytes, stream, (const float*)x, wr,
                       wr_dtype, shared_gate_w, sg_dtype, logits, arrived, width, topk_w, topk_e, shared_gate, offsets,
                       rows, dest, tokens, experts, k, renormalize, scale, tile_rows, tile_expert, tile_row0, tile_info);
  else
    hipLaunchKernelGGL(moe_route_dispatch_small_kernel<bf16_t>, grid, block, xs_bytes, stream, (const bf16_t*)x, wr,
                       wr_dtype, shared_gate_w, sg_dtype, logits, arrived, width, topk_w, topk_e, shared_gate, offsets,
                       rows, dest, tokens, experts, k, renormalize, scale, tile_rows, tile_expert, tile_row0, tile_info);
  return ix_check_launch("ix_moe_route_dispatch_small");
}
