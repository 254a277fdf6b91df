// Selection and grouping for few tokens (decoding) in ONE workgroup: softmax and
// top-k of every token's router scores, then counts, offsets, the stable
// placement and the row-tile map.  Same arithmetic and tie rule as
// moe_route_kernel / moe_dispatch_small_kernel in moe.hip (reference:
// RouteTopKKernel src/backends/cuda/ops/moe.cu:36-127, MoeBuildDispatch :452-513).
#include "common.h"

#define SD_THREADS 1024
#define SD_MAX_ASSIGN 1024
#define SD_MAX_EXPERTS 256

__global__ void __launch_bounds__(SD_THREADS)
moe_select_dispatch_kernel(const float* __restrict__ logits, float* __restrict__ topk_w, int32_t* __restrict__ topk_e,
                           float* __restrict__ shared_gate, int32_t* __restrict__ offsets, int32_t* __restrict__ rows,
                           int32_t* __restrict__ dest, int tokens, int experts, int k, int renormalize, float scale,
                           int tile_rows, int32_t* __restrict__ tile_expert, int32_t* __restrict__ tile_row0,
                           int32_t* __restrict__ tile_info) {
  __shared__ float zs[SD_THREADS / 64][SD_MAX_EXPERTS];
  __shared__ int32_t chosen[SD_MAX_ASSIGN];
  __shared__ int32_t counts[SD_MAX_EXPERTS];
  __shared__ int32_t first_row[SD_MAX_EXPERTS];
  __shared__ int32_t first_tile[SD_MAX_EXPERTS];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  for (int e = tid; e < experts; e += SD_THREADS) counts[e] = 0;

  // ---- selection: one wavefront per token ----
  float* z = zs[wave];
  for (int t = wave; t < tokens; t += SD_THREADS / 64) {
    const float* row = logits + static_cast<int64_t>(t) * (experts + 1);
    float mx = -INFINITY;
    for (int e = lane; e < experts; e += 64) {
      z[e] = row[e];
      mx = fmaxf(mx, z[e]);
    }
    if (shared_gate && lane == 0) shared_gate[t] = 1.0f / (1.0f + expf(-row[experts]));
    mx = ix_wave_max(mx);
    float sum = 0.f;
    for (int e = lane; e < experts; e += 64) {
      const float p = expf(z[e] - mx);
      z[e] = p;
      sum += p;
    }
    sum = ix_wave_sum(sum);
    __builtin_amdgcn_wave_barrier();
    __threadfence_block();
    const float inv_sum = 1.0f / sum;
    float mine_w = 0.f, total = 0.f;
    for (int slot = 0; slot < k; ++slot) {
      float bv = -INFINITY;
      int bi = 0x7fffffff;
      for (int e = lane; e < experts; e += 64) {
        const float v = z[e];
        if (v > bv) { bv = v; bi = e; }
      }
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) {
        const float ov = __shfl_xor(bv, off, 64);
        const int oi = __shfl_xor(bi, off, 64);
        if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
      }
      if (bi < 0 || bi >= experts) bi = 0;  // only when every score is NaN
      const float wgt = bv * inv_sum;
      total += wgt;
      if (lane == slot) mine_w = wgt;
      if (lane == 0) {
        topk_e[t * k + slot] = bi;
        chosen[t * k + slot] = bi;
        z[bi] = -INFINITY;
      }
      __builtin_amdgcn_wave_barrier();
      __threadfence_block();
    }
    const float f = ((renormalize && total > 0.f) ? 1.0f / total : 1.0f) * scale;
    if (lane < k) topk_w[t * k + lane] = mine_w * f;
  }
  __syncthreads();

  // ---- grouping ----
  const int assignments = tokens * k;
  int mine = -1, rank = 0;
  if (tid < assignments) {
    mine = chosen[tid];
    for (int b = 0; b < tid; ++b) rank += (chosen[b] == mine) ? 1 : 0;
    atomicAdd(&counts[mine], 1);  // integer counts: order does not matter
  }
  __syncthreads();
  if (tid == 0) {
    int32_t run = 0, tiles = 0;
    for (int e = 0; e < experts; ++e) {
      offsets[e] = run;
      first_row[e] = run;
      first_tile[e] = tiles;
      run += counts[e];
      if (tile_rows > 0) tiles += (counts[e] + tile_rows - 1) / tile_rows;
    }
    offsets[experts] = run;
    if (tile_info) tile_info[0] = tiles;
  }
  __syncthreads();
  if (tid < assignments) {
    const int32_t r = first_row[mine] + rank;
    rows[r] = tid / k;
    dest[tid] = r;
  }
  if (tile_rows > 0 && tile_expert) {
    for (int e = tid; e < experts; e += SD_THREADS) {
      const int n = (counts[e] + tile_rows - 1) / tile_rows;
      for (int i = 0; i < n; ++i) {
        tile_expert[first_tile[e] + i] = e;
        tile_row0[first_tile[e] + i] = first_row[e] + i * tile_rows;
      }
    }
  }
}

// logits float32 [tokens, experts + 1] from ix_moe_route_logits.  tokens * k <= 1024, experts <= 256, k <= 32.
extern "C" int ix_moe_select_dispatch(const float* logits, float* topk_w, int32_t* topk_e, float* shared_gate,
                                      int32_t* offsets, int32_t* rows, int32_t* dest, int tokens, int experts, int k,
                                      int renormalize, float scale, int tile_rows, int32_t* tile_expert,
                                      int32_t* tile_row0, int32_t* tile_info, hipStream_t stream) {
  IX_REQUIRE(tokens > 0 && experts > 0 && k > 0, "sizes must be positive");
  IX_REQUIRE(experts <= SD_MAX_EXPERTS, "at most 256 experts for the one-workgroup selection");
  IX_REQUIRE(k <= experts && k <= 32, "top_k must be between 1 and min(experts, 32)");
  IX_REQUIRE(static_cast<int64_t>(tokens) * k <= SD_MAX_ASSIGN, "at most 1024 assignments for the one-workgroup selection");
  IX_REQUIRE(tile_rows >= 0, "tile_rows must not be negative");
  IX_REQUIRE(tile_rows == 0 || (tile_expert && tile_row0 && tile_info), "tile map buffers needed");
  hipLaunchKernelGGL(moe_select_dispatch_kernel, dim3(1), dim3(SD_THREADS), 0, stream, logits, topk_w, topk_e,
                     shared_gate, offsets, rows, dest, tokens, experts, k, renormalize, scale, tile_rows, tile_expert,
                     tile_row0, tile_info);
  return ix_check_launch("ix_moe_select_dispatch");
}
