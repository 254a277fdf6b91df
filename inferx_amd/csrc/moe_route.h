// Parts of the router that more than one kernel uses: a router row against a token, and the
// selection and grouping of few tokens by one workgroup.
#pragma once
#include "common.h"

#define SD_MAX_ASSIGN 1024
#define SD_MAX_EXPERTS 256

// x . w[row] over `width`, one wavefront, x as float32 at `xs` (LDS or global)
__device__ __forceinline__ float route_row_dot(const float* __restrict__ xs, const void* __restrict__ w, int dt,
                                               int64_t base, int64_t width, int lane) {
  float dot = 0.f;
  if (dt == IX_BF16 && (width & 7) == 0 && (reinterpret_cast<uintptr_t>(w) & 15) == 0) {
    // eight weights per lane and load (16 bytes); the order of additions is fixed by the lane layout
    const uint16_t* wrow = static_cast<const uint16_t*>(w) + base;
    for (int64_t i = lane * 8; i < width; i += 512) {
      const uint4 v = *reinterpret_cast<const uint4*>(wrow + i);
      const float4 x0 = *reinterpret_cast<const float4*>(xs + i);
      const float4 x1 = *reinterpret_cast<const float4*>(xs + i + 4);
      dot += x0.x * __uint_as_float(v.x << 16) + x0.y * __uint_as_float(v.x & 0xffff0000u) +
             x0.z * __uint_as_float(v.y << 16) + x0.w * __uint_as_float(v.y & 0xffff0000u) +
             x1.x * __uint_as_float(v.z << 16) + x1.y * __uint_as_float(v.z & 0xffff0000u) +
             x1.z * __uint_as_float(v.w << 16) + x1.w * __uint_as_float(v.w & 0xffff0000u);
    }
  } else if (dt == IX_F32 && (width & 3) == 0 && (reinterpret_cast<uintptr_t>(w) & 15) == 0) {
    const float* wrow = static_cast<const float*>(w) + base;
    for (int64_t i = lane * 4; i < width; i += 256) {
      const float4 v = *reinterpret_cast<const float4*>(wrow + i);
      const float4 x0 = *reinterpret_cast<const float4*>(xs + i);
      dot += x0.x * v.x + x0.y * v.y + x0.z * v.z + x0.w * v.w;
    }
  } else {
    for (int64_t i = lane; i < width; i += 64) dot += xs[i] * ix_load_rt(w, dt, base + i);
  }
  return ix_wave_sum(dot);
}

// Selection and grouping for few tokens by ONE workgroup of NW wavefronts: softmax and top-k of every
// token's router scores, then counts, offsets, the stable placement and the row-tile map.
// `logits` float32 [tokens, experts + 1]; tokens * k <= SD_MAX_ASSIGN, experts <= SD_MAX_EXPERTS.
// The scores were written by other workgroups of the same launch (with device-scope stores): they are read with
// device-scope loads, which do not take a stale line from this die's L2.
template <int NW>
__device__ __forceinline__ void
select_dispatch_body(const float* logits, float* __restrict__ topk_w, int32_t* __restrict__ topk_e,
                     float* __restrict__ shared_gate, int32_t* __restrict__ offsets, int32_t* __restrict__ rows,
                     int32_t* __restrict__ dest, int tokens, int experts, int k, int renormalize, float scale,
                     int tile_rows, int32_t* __restrict__ tile_expert, int32_t* __restrict__ tile_row0,
                     int32_t* __restrict__ tile_info) {
  static_assert(NW >= SD_MAX_EXPERTS / 64, "a thread per possible expert clears the counts");
  auto fresh = [](const float* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); };
  __shared__ float zs[NW][SD_MAX_EXPERTS];
  __shared__ int32_t chosen[SD_MAX_ASSIGN];
  __shared__ int32_t counts[SD_MAX_EXPERTS];
  __shared__ int32_t first_row[SD_MAX_EXPERTS];
  __shared__ int32_t first_tile[SD_MAX_EXPERTS];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;

  // ---- selection: one wavefront per token ----
  float* z = zs[wave];
  for (int t = wave; t < tokens; t += NW) {
    const float* row = logits + static_cast<int64_t>(t) * (experts + 1);
    float mx = -INFINITY;
    for (int e = lane; e < experts; e += 64) {
      z[e] = fresh(row + e);
      mx = fmaxf(mx, z[e]);
    }
    if (shared_gate && lane == 0) shared_gate[t] = 1.0f / (1.0f + expf(-fresh(row + experts)));
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
  for (int e = wave; e < experts; e += NW) {
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
  for (int e = wave; e < experts; e += NW) {
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
