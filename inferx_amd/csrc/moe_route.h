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

// The same for a bfloat16 row (width a multiple of 8, 16-byte aligned) whose first ROUTE_PRELOAD pieces per lane were
// loaded before (`route_row_preload`), so that they could be on their way while x was still being formed; the same
// additions in the same order.
#define ROUTE_PRELOAD 4
__device__ __forceinline__ bool route_row_preloadable(const void* w, int dt, int64_t width) {
  return dt == IX_BF16 && (width & 7) == 0 && (reinterpret_cast<uintptr_t>(w) & 15) == 0;
}
__device__ __forceinline__ void route_row_preload(const void* __restrict__ w, int64_t base, int64_t width, int lane,
                                                  uint4 (&pre)[ROUTE_PRELOAD]) {
  const uint16_t* wrow = static_cast<const uint16_t*>(w) + base;
#pragma unroll
  for (int j = 0; j < ROUTE_PRELOAD; ++j) {
    const int64_t i = lane * 8 + 512 * j;
    pre[j] = i < width ? *reinterpret_cast<const uint4*>(wrow + i) : make_uint4(0u, 0u, 0u, 0u);
  }
}
__device__ __forceinline__ float route_row_dot_preloaded(const float* __restrict__ xs, const void* __restrict__ w,
                                                         int64_t base, int64_t width, int lane,
                                                         const uint4 (&pre)[ROUTE_PRELOAD]) {
  const uint16_t* wrow = static_cast<const uint16_t*>(w) + base;
  float dot = 0.f;
  auto piece = [&](const uint4 v, int64_t i) {
    const float4 x0 = *reinterpret_cast<const float4*>(xs + i);
    const float4 x1 = *reinterpret_cast<const float4*>(xs + i + 4);
    dot += x0.x * __uint_as_float(v.x << 16) + x0.y * __uint_as_float(v.x & 0xffff0000u) +
           x0.z * __uint_as_float(v.y << 16) + x0.w * __uint_as_float(v.y & 0xffff0000u) +
           x1.x * __uint_as_float(v.z << 16) + x1.y * __uint_as_float(v.z & 0xffff0000u) +
           x1.z * __uint_as_float(v.w << 16) + x1.w * __uint_as_float(v.w & 0xffff0000u);
  };
#pragma unroll
  for (int j = 0; j < ROUTE_PRELOAD; ++j) {
    const int64_t i = lane * 8 + 512 * j;
    if (i < width) piece(pre[j], i);
  }
  for (int64_t i = lane * 8 + 512 * ROUTE_PRELOAD; i < width; i += 512) piece(*reinterpret_cast<const uint4*>(wrow + i), i);
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

// The same for at most 64 assignments (tokens * k) and at most 64 * SD_FEW_PER_LANE experts, without a pass over
// LDS per expert: a token's scores stay in its wavefront's registers through the k rounds, and grouping takes one
// assignment per lane: an assignment's row is the number of assignments of lower experts plus those of its own
// expert before it, which one loop over the assignments counts for every lane at once (and, for the lanes taken as
// experts, each expert's first row and row count).  The same selections, weights, rows and tile
// map as select_dispatch_body, bit for bit.
#define SD_FEW_PER_LANE (SD_MAX_EXPERTS / 64)
#ifndef SD_FEW_ASSIGN
#define SD_FEW_ASSIGN 64  // assignments up to which select_dispatch_few is taken (it can take 64)
#endif
template <int NW>
__device__ __forceinline__ void
select_dispatch_few(const float* logits, float* __restrict__ topk_w, int32_t* __restrict__ topk_e,
                    float* __restrict__ shared_gate, int32_t* __restrict__ offsets, int32_t* __restrict__ rows,
                    int32_t* __restrict__ dest, int tokens, int experts, int k, int renormalize, float scale,
                    int tile_rows, int32_t* __restrict__ tile_expert, int32_t* __restrict__ tile_row0,
                    int32_t* __restrict__ tile_info) {
  auto fresh = [](const float* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); };
  static_assert(NW * 64 >= SD_MAX_EXPERTS, "a thread per possible expert clears the counts");
  __shared__ int32_t chosen[64], lower_s[64], same_s[64], first_s[SD_MAX_EXPERTS], count_s[SD_MAX_EXPERTS];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  if (tid < 64) lower_s[tid] = same_s[tid] = 0;
  if (tid < SD_MAX_EXPERTS) first_s[tid] = count_s[tid] = 0;
  // ---- selection: one wavefront per token, expert lane + 64 j in register j ----
  for (int t = wave; t < tokens; t += NW) {
    const float* row = logits + static_cast<int64_t>(t) * (experts + 1);
    float z[SD_FEW_PER_LANE];
    float mx = -INFINITY;
#pragma unroll
    for (int j = 0; j < SD_FEW_PER_LANE; ++j) {
      const int e = lane + 64 * j;
      z[j] = e < experts ? fresh(row + e) : -INFINITY;
      mx = fmaxf(mx, z[j]);
    }
    if (shared_gate && lane == 0) shared_gate[t] = 1.0f / (1.0f + expf(-fresh(row + experts)));
    mx = ix_wave_max(mx);
    float sum = 0.f;
#pragma unroll
    for (int j = 0; j < SD_FEW_PER_LANE; ++j) {
      if (lane + 64 * j < experts) {
        z[j] = expf(z[j] - mx);
        sum += z[j];
      }
    }
    sum = ix_wave_sum(sum);
    const float inv_sum = 1.0f / sum;
    float mine_w = 0.f, total = 0.f;
    for (int slot = 0; slot < k; ++slot) {
      float bv = -INFINITY;
      int bi = 0x7fffffff;
#pragma unroll
      for (int j = 0; j < SD_FEW_PER_LANE; ++j)
        if (lane + 64 * j < experts && z[j] > bv) {
          bv = z[j];
          bi = lane + 64 * j;
        }
      ix_wave_argmax(bv, bi);
      if (bi < 0 || bi >= experts) bi = 0;  // only when every score is NaN
      const float wgt = bv * inv_sum;
      total += wgt;
      if (lane == slot) mine_w = wgt;
#pragma unroll
      for (int j = 0; j < SD_FEW_PER_LANE; ++j)
        if (bi == lane + 64 * j) z[j] = -INFINITY;
      if (lane == 0) {
        topk_e[t * k + slot] = bi;
        chosen[t * k + slot] = bi;
      }
    }
    const float f = ((renormalize && total > 0.f) ? 1.0f / total : 1.0f) * scale;
    if (lane < k) topk_w[t * k + lane] = mine_w * f;
  }
  __syncthreads();

  // ---- grouping: lane a = assignment a; lane and register j also = expert lane + 64 j.  The wavefronts share the
  // loop over the assignments (each takes every NW-th) and add their counts up in LDS (whole numbers: the order
  // does not matter); the first one goes on alone.
  const int assignments = tokens * k;
  const int mine = lane < assignments ? chosen[lane] : 0x7fffffff;
  int lower = 0, same_before = 0;
  int first[SD_FEW_PER_LANE], count[SD_FEW_PER_LANE];  // of expert lane + 64 j: its first row, its rows
#pragma unroll
  for (int j = 0; j < SD_FEW_PER_LANE; ++j) first[j] = count[j] = 0;
  for (int b = wave; b < assignments; b += NW) {
    const int eb = __builtin_amdgcn_readlane(mine, b);
    lower += eb < mine ? 1 : 0;
    same_before += (eb == mine && b < lane) ? 1 : 0;
#pragma unroll
    for (int j = 0; j < SD_FEW_PER_LANE; ++j) {
      if (64 * j < experts) {
        first[j] += eb < lane + 64 * j ? 1 : 0;
        count[j] += eb == lane + 64 * j ? 1 : 0;
      }
    }
  }
  if (wave < assignments) {
    if (lane < assignments) {
      atomicAdd(&lower_s[lane], lower);
      atomicAdd(&same_s[lane], same_before);
    }
#pragma unroll
    for (int j = 0; j < SD_FEW_PER_LANE; ++j) {
      if (64 * j < experts) {
        atomicAdd(&first_s[lane + 64 * j], first[j]);
        atomicAdd(&count_s[lane + 64 * j], count[j]);
      }
    }
  }
  __syncthreads();
  if (wave != 0) return;
  lower = lower_s[lane];
  same_before = same_s[lane];
#pragma unroll
  for (int j = 0; j < SD_FEW_PER_LANE; ++j) {
    first[j] = first_s[lane + 64 * j];
    count[j] = count_s[lane + 64 * j];
  }
  if (lane < assignments) {
    const int r = lower + same_before;
    rows[r] = lane / k;
    dest[lane] = r;
  }
  // tiles before each expert: sums over the lanes of a register, registers one after the other.  Where no expert has
  // more rows than a tile holds (the usual case), an expert's tiles before it are the experts before it that have
  // rows at all, which a ballot counts; else sums over the lanes.
  int tiles_first[SD_FEW_PER_LANE], tiles_mine[SD_FEW_PER_LANE], carry = 0;
  bool plain = true;
#pragma unroll
  for (int j = 0; j < SD_FEW_PER_LANE; ++j) {
    const int e = lane + 64 * j;
    if (64 * j < experts && e < experts) offsets[e] = first[j];
    tiles_mine[j] = (tile_rows > 0 && e < experts) ? (count[j] + tile_rows - 1) / tile_rows : 0;
    plain = plain && tiles_mine[j] <= 1;
  }
  plain = __all(plain);
  const uint64_t below = (uint64_t(1) << lane) - 1;
#pragma unroll
  for (int j = 0; j < SD_FEW_PER_LANE; ++j) {
    if (64 * j >= experts || tile_rows <= 0) {
      tiles_first[j] = carry;
    } else if (plain) {
      const uint64_t has = __ballot(tiles_mine[j] > 0);
      tiles_first[j] = carry + __popcll(has & below);
      carry += __popcll(has);
    } else {
      int incl = tiles_mine[j];
#pragma unroll
      for (int off = 1; off < 64; off <<= 1) {
        const int o = __shfl_up(incl, off, 64);
        if (lane >= off) incl += o;
      }
      tiles_first[j] = carry + incl - tiles_mine[j];
      carry += __shfl(incl, 63, 64);
    }
  }
  if (tile_rows > 0 && tile_expert) {
#pragma unroll
    for (int j = 0; j < SD_FEW_PER_LANE; ++j) {
      for (int i = 0; i < tiles_mine[j]; ++i) {
        tile_expert[tiles_first[j] + i] = lane + 64 * j;
        tile_row0[tiles_first[j] + i] = first[j] + i * tile_rows;
      }
    }
  }
  if (lane == 0) {
    offsets[experts] = assignments;
    if (tile_info) tile_info[0] = carry;
  }
}
