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
      ix_wave_argmax(bv, bi);
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

  // ---- grouping: a wavefront per expert (in turn), 64 assignments at a time ----
  // counts: lanes compare their assignments with the expert, a ballot counts the matches
  const int assignments = tokens * k;
  if (tid >= experts && tid < SD_MAX_EXPERTS) counts[tid] = 0;
  for (int e = wave; e < experts; e += SD_THREADS / 64) {
    int count = 0;
    for (int a0 = 0; a0 < assignments; a0 += 64) {
      const int a = a0 + lane;
      count += __popcll(__ballot(a < assignments && chosen[a] == e));
    }
    if (lane == 0) counts[e] = count;
  }
  __syncthreads();
  // offsets: exclusive sums over the experts by the first wavefront, four experts per lane
  if (wave == 0) {
    int c[4], rows_before = 0, tiles_before = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      c[j] = counts[4 * lane + j];
      rows_before += c[j];
      tiles_before += tile_rows > 0 ? (c[j] + tile_rows - 1) / tile_rows : 0;
    }
    const int rows_mine = rows_before, tiles_mine = tiles_before;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {  // inclusive sums over the lanes
      const int r = __shfl_up(rows_before, off, 64), t = __shfl_up(tiles_before, off, 64);
      if (lane >= off) {
        rows_before += r;
        tiles_before += t;
      }
    }
    int run = rows_before - rows_mine, tiles = tiles_before - tiles_mine;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int e = 4 * lane + j;
      first_row[e] = run;
      first_tile[e] = tiles;
      if (e < experts) offsets[e] = run;
      run += c[j];
      tiles += tile_rows > 0 ? (c[j] + tile_rows - 1) / tile_rows : 0;
    }
    if (lane == 63) {
      offsets[experts] = run;
      if (tile_info) tile_info[0] = tiles;
    }
  }
  __syncthreads();
  // placement in the order of the assignments (stable): a match's row is the expert's first row plus the matches
  // before it; and the expert's row tiles
  const uint64_t below = (uint64_t(1) << lane) - 1;
  for (int e = wave; e < experts; e += SD_THREADS / 64) {
    int base = first_row[e];
    for (int a0 = 0; a0 < assignments; a0 += 64) {
      const int a = a0 + lane;
      const bool match = a < assignments && chosen[a] == e;
      const uint64_t mask = __ballot(match);
      if (match) {
        const int r = base + __popcll(mask & below);
        rows[r] = a / k;
        dest[a] = r;
      }
      base += __popcll(mask);
    }
    if (tile_rows > 0 && tile_expert) {
      const int n = (counts[e] + tile_rows - 1) / tile_rows;
      for (int i = lane; i < n; i += 64) {
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
