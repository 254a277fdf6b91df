// Grouped expert products on the matrix cores (bfloat16 in, float32 accumulate).
//
//   GATE_UP: act[r, n] = silu(x[rows[r]] . W[e][n]) * (x[rows[r]] . W[e][N + n]),  W [E, 2N, K]
//   else:    y[r, n]   = a[r] . W[e][n],                                           W [E, N, K]
// for the rows r of expert e, taken from the row-tile map that the grouping
// kernel wrote (reference: GroupedGemmBf16Kernel, src/backends/cuda/ops/moe.cu:323-392,
// which uses scalar FMAs; SwiGLU src/model/moe_ffn.cc:288-291).
//
// The product is formed transposed, out^T[n][r] = W[n][:] . x[r][:], so that the
// big operand, the expert's weight rows, is the A operand and streams from
// memory straight into registers: v_mfma_f32_16x16x32_bf16, A = 16 weight rows,
// B = 16 activation rows, lane l of the result holding out-features 4*(l/16)+i
// of row l%16, i.e. four consecutive numbers of one output row.
//
// A wavefront owns 16 out-features x (16 * MT) rows.  Per iteration it covers
// 128 of K with four loads: in load j lane (m, g) reads the 16 bytes at
// k0 + 32 j + 8 g of weight row m, so the four lane groups cover 64 contiguous
// bytes of each row and the 32 reduction slots of MFMA j; the activations are
// read with the same mapping.  KSPLIT = 4 (decoding: few rows, the weights are the traffic) lets
// the four wavefronts of a workgroup take a quarter of K each and add up through
// LDS; KSPLIT = 1 gives each wavefront its own 16 out-features.
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

// The work of one wavefront (KSPLIT == 1) or workgroup (KSPLIT == 4): rows [row0, row_end) x out-features
// [n0, n0 + 16) of expert e.  `red`: LDS for the partial sums of a split reduction.
// NB: blocks of 16 out-features side by side ([n0, n0 + 16 NB)), so that the rows are read once for all of them.
template <int MT, bool GATE_UP, int KSPLIT, typename TO = __bf16, int NB = 1>
__device__ __forceinline__ void grouped_body(const __bf16* a, const __bf16* w,
                                             TO* __restrict__ out, const int32_t* __restrict__ rows, int e,
                                             int row0, int row_end, int n0, int n_out, int width, float* red) {
  constexpr int NACC = NB * (GATE_UP ? 2 : 1);  // accumulator b + NB h: block b of the gate (h = 0) or up (1) rows
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int m = lane & 15, g = lane >> 4;
  const int kper = KSPLIT > 1 ? (((width + KSPLIT - 1) / KSPLIT + 127) & ~127) : width;
  const int kbegin = KSPLIT > 1 ? wave * kper : 0;
  const int kend = min(width, kbegin + kper);

  const int64_t w_rows = GATE_UP ? 2 * static_cast<int64_t>(n_out) : n_out;
  const __bf16* wp[NACC];
#pragma unroll
  for (int u = 0; u < NACC; ++u) {
    const int wrow = min(n0 + 16 * (u % NB) + m, n_out - 1);  // rows past the end are computed and not stored
    wp[u] = w + (static_cast<int64_t>(e) * w_rows + (u / NB) * static_cast<int64_t>(n_out) + wrow) * width;
  }

  const __bf16* xr[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int r = min(row0 + 16 * t + m, row_end - 1);
    xr[t] = a + static_cast<int64_t>(rows ? rows[r] : r) * width;
  }

  f32x4 acc[NACC][MT];
#pragma unroll
  for (int u = 0; u < NACC; ++u)
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[u][t] = f32x4{0.f, 0.f, 0.f, 0.f};

  const bf16x8 zero = {(__bf16)0.f, (__bf16)0.f, (__bf16)0.f, (__bf16)0.f,
                       (__bf16)0.f, (__bf16)0.f, (__bf16)0.f, (__bf16)0.f};
  // The loads of the next 128 of K are issued before the products of the present ones, so that a wavefront
  // always has loads on their way.  Every load is unconditional (a piece past the end of a ragged last round is
  // read from the range's first piece instead, which is in the cache, and the activations' values are replaced
  // by zeros when they are used): with no branch in it the loop is one straight line, and the compiler lets the
  // younger loads stay in flight at each wait instead of waiting for all.
  bf16x8 fw[2][NACC][4], fx[2][MT][4];
  auto fetch = [&](int k0, bf16x8 (&w_)[NACC][4], bf16x8 (&x_)[MT][4]) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      int kk = k0 + 32 * j + 8 * g;  // the four lane groups cover 64 contiguous bytes of a row per load
      kk = kk < kend ? kk : kbegin;  // (the range's first piece: it exists, kbegin + 8 g need not)
#pragma unroll
      for (int u = 0; u < NACC; ++u) w_[u][j] = *reinterpret_cast<const bf16x8*>(wp[u] + kk);
#pragma unroll
      for (int t = 0; t < MT; ++t) x_[t][j] = *reinterpret_cast<const bf16x8*>(xr[t] + kk);
    }
  };
  auto multiply = [&](int k0, const bf16x8 (&w_)[NACC][4], const bf16x8 (&x_)[MT][4]) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const bool ok = k0 + 32 * j + 8 * g < kend;
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        const bf16x8 xv = ok ? x_[t][j] : zero;
#pragma unroll
        for (int u = 0; u < NACC; ++u)
          acc[u][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w_[u][j], xv, acc[u][t], 0, 0, 0);
      }
    }
  };
  // Rounds of 128 in pairs, so that the register sets are named statically; the loop runs while both rounds of a
  // turn are followed by another one and has no way out of its middle, the last one or two rounds come after it.
  const int rounds = kbegin < kend ? (kend - kbegin + 127) >> 7 : 0;
  if (rounds > 0) {
    fetch(kbegin, fw[0], fx[0]);
    int k0 = kbegin, left = rounds;
    for (; left > 2; left -= 2, k0 += 256) {
      fetch(k0 + 128, fw[1], fx[1]);
      __builtin_amdgcn_sched_barrier(0);
      multiply(k0, fw[0], fx[0]);
      __builtin_amdgcn_sched_barrier(0);
      fetch(k0 + 256, fw[0], fx[0]);
      __builtin_amdgcn_sched_barrier(0);
      multiply(k0 + 128, fw[1], fx[1]);
      __builtin_amdgcn_sched_barrier(0);
    }
    if (left == 2) {
      fetch(k0 + 128, fw[1], fx[1]);
      __builtin_amdgcn_sched_barrier(0);
      multiply(k0, fw[0], fx[0]);
      multiply(k0 + 128, fw[1], fx[1]);
    } else {
      multiply(k0, fw[0], fx[0]);
    }
  }

  if (KSPLIT > 1) {
    // wavefronts 1..3 hand their partial sums to wavefront 0
    if (wave > 0) {
      float* dst = red + ((wave - 1) * 64 + lane) * (MT * NACC * 4);
#pragma unroll
      for (int u = 0; u < NACC; ++u)
#pragma unroll
        for (int t = 0; t < MT; ++t)
#pragma unroll
          for (int i = 0; i < 4; ++i) dst[(u * MT + t) * 4 + i] = acc[u][t][i];
    }
    __syncthreads();
    if (wave > 0) return;
#pragma unroll
    for (int s = 0; s < KSPLIT - 1; ++s) {
      const float* src = red + (s * 64 + lane) * (MT * NACC * 4);
#pragma unroll
      for (int u = 0; u < NACC; ++u)
#pragma unroll
        for (int t = 0; t < MT; ++t)
#pragma unroll
          for (int i = 0; i < 4; ++i) acc[u][t][i] += src[(u * MT + t) * 4 + i];
    }
  }

  // lane holds out-features n0 + 16 u + 4 g + i of row row0 + 16 t + m
#pragma unroll
  for (int u = 0; u < NB; ++u) {
    const int nb = n0 + 16 * u + 4 * g;
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      const int r = row0 + 16 * t + m;
      if (r >= row_end) continue;
      float v[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        v[i] = acc[u][t][i];
        if constexpr (GATE_UP) v[i] = v[i] / (1.0f + __expf(-v[i])) * acc[NB + u][t][i];
      }
      TO* dst = out + static_cast<int64_t>(r) * n_out + nb;
      if (nb + 4 <= n_out && (n_out & 3) == 0) {
        if constexpr (sizeof(TO) == 4) {
          *reinterpret_cast<f32x4*>(dst) = f32x4{v[0], v[1], v[2], v[3]};
        } else {
          bf16x4 o = {(__bf16)v[0], (__bf16)v[1], (__bf16)v[2], (__bf16)v[3]};
          *reinterpret_cast<bf16x4*>(dst) = o;
        }
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (nb + i < n_out) dst[i] = (TO)v[i];
      }
    }
  }
}

// x [rows <= 16 * MT, width] . w[n_out, width]^T -> float32 [rows, n_out]: the head of a decoding step, whose
// logits stay float32 (one workgroup per 32 out-features, so that the rows, which every workgroup reads, weigh
// less beside the weights; the reduction split over its four wavefronts).
template <int MT>
__global__ void __launch_bounds__(256)
linear_skinny_f32_kernel(const __bf16* x, const __bf16* w, float* __restrict__ out,
                         int rows, int n_out, int width) {
  __shared__ float red[3 * 64 * MT * 2 * 4];
  grouped_body<MT, false, 4, float, 2>(x, w, out, nullptr, 0, 0, rows, blockIdx.x * 32, n_out, width, red);
}

template <int MT, bool GATE_UP, int KSPLIT>
__global__ void __launch_bounds__(256)
moe_grouped_mfma_kernel(const __bf16* a, const __bf16* w, __bf16* __restrict__ out,
                        const int32_t* __restrict__ offsets, const int32_t* __restrict__ rows,
                        const int32_t* __restrict__ tile_expert, const int32_t* __restrict__ tile_row0,
                        const int32_t* __restrict__ tile_info, int n_out, int width) {
  __shared__ float red[KSPLIT > 1 ? 3 * 64 * MT * (GATE_UP ? 2 : 1) * 4 : 1];
  if (static_cast<int>(blockIdx.y) >= tile_info[0]) return;
  const int e = tile_expert[blockIdx.y];
  const int n0 = (KSPLIT > 1 ? blockIdx.x : blockIdx.x * 4 + (threadIdx.x >> 6)) * 16;
  if (n0 >= n_out) return;  // whole wavefront (KSPLIT == 1) or whole workgroup
  grouped_body<MT, GATE_UP, KSPLIT>(a, w, out, rows, e, tile_row0[blockIdx.y], offsets[e + 1], n0, n_out, width, red);
}

// Routed experts and the shared expert in one launch (decoding: every launch saved counts).  The first
// n16_s * shared_tiles workgroups serve the shared expert, which is one more "expert" over all `shared_rows`
// tokens with weights and sizes of its own (first, because its reduction may be the longer one and the last
// workgroups to start set the kernel's end); the rest serve the routed experts' row tiles.
template <int MT, bool GATE_UP, int NB>
__global__ void __launch_bounds__(256)
moe_grouped_dual_kernel(const __bf16* a, const __bf16* w, __bf16* __restrict__ out,
                        const int32_t* __restrict__ offsets, const int32_t* __restrict__ rows,
                        const int32_t* __restrict__ tile_expert, const int32_t* __restrict__ tile_row0,
                        const int32_t* __restrict__ tile_info, int max_tiles, int n_out, int width,
                        const __bf16* a_s, const __bf16* w_s, __bf16* __restrict__ out_s,
                        int shared_rows, int n_out_s, int width_s) {
  __shared__ float red[3 * 64 * MT * NB * (GATE_UP ? 2 : 1) * 4];
  const int n16_s = (n_out_s + 16 * NB - 1) / (16 * NB);  // column blocks of 16 NB out-features
  const int shared_blocks = n16_s * ((shared_rows + 16 * MT - 1) / (16 * MT));
  int idx = blockIdx.x;
  if (idx < shared_blocks) {
    const int tile = idx / n16_s;
    grouped_body<MT, GATE_UP, 4, __bf16, NB>(a_s, w_s, out_s, nullptr, 0, tile * 16 * MT, shared_rows,
                                             (idx - tile * n16_s) * 16 * NB,
                                 n_out_s, width_s, red);
  } else {
    idx -= shared_blocks;
    const int n16_e = (n_out + 16 * NB - 1) / (16 * NB);
    const int tile = idx / n16_e;
    if (tile >= tile_info[0]) return;
    const int e = tile_expert[tile];
    grouped_body<MT, GATE_UP, 4, __bf16, NB>(a, w, out, rows, e, tile_row0[tile], offsets[e + 1],
                                             (idx - tile * n16_e) * 16 * NB, n_out, width, red);
  }
}

// `max_tiles` bounds the number of row tiles (the grid); the kernel reads the true number from tile_info.
// tile_rows (16, 32 or 64) must be what the grouping kernel was given.
extern "C" int ix_moe_grouped_mfma(const void* a, const void* w, void* out, const int32_t* offsets,
                                   const int32_t* rows, const int32_t* tile_expert, const int32_t* tile_row0,
                                   const int32_t* tile_info, int max_tiles, int tile_rows, int64_t n_out,
                                   int64_t width, int gate_up, int k_split, hipStream_t stream) {
  IX_REQUIRE(n_out > 0 && width > 0 && max_tiles >= 0, "sizes must be positive");
  IX_REQUIRE(width % 8 == 0, "the reduction width must be a multiple of 8 for the matrix-core kernel");
  IX_REQUIRE(n_out < (1 << 30) && width < (1 << 30), "sizes too large");
  IX_REQUIRE(tile_rows == 16 || tile_rows == 32 || tile_rows == 64, "tile_rows must be 16, 32 or 64");
  IX_REQUIRE(k_split == 1 || k_split == 4, "k_split must be 1 or 4");
  IX_REQUIRE(max_tiles <= 65535, "too many row tiles for one launch");
  if (max_tiles == 0) return 0;
  const int n_tiles16 = static_cast<int>((n_out + 15) / 16);
  dim3 grid(k_split > 1 ? n_tiles16 : (n_tiles16 + 3) / 4, max_tiles), block(256);
#define LAUNCH(MT, GU, KS)                                                                                        \
  hipLaunchKernelGGL((moe_grouped_mfma_kernel<MT, GU, KS>), grid, block, 0, stream, (const __bf16*)a,             \
                     (const __bf16*)w, (__bf16*)out, offsets, rows, tile_expert, tile_row0, tile_info, (int)n_out, \
                     (int)width)
#define PICK(MT)                                       \
  if (gate_up) {                                       \
    if (k_split > 1) LAUNCH(MT, true, 4);              \
    else LAUNCH(MT, true, 1);                          \
  } else {                                             \
    if (k_split > 1) LAUNCH(MT, false, 4);             \
    else LAUNCH(MT, false, 1);                         \
  }
  if (tile_rows == 16) { PICK(1) } else if (tile_rows == 32) { PICK(2) } else { PICK(4) }
#undef PICK
#undef LAUNCH
  return ix_check_launch("ix_moe_grouped_mfma");
}

// One launch for the routed experts (as ix_moe_grouped_mfma with k_split 4) and the shared expert
// (a_s [shared_rows, width_s] . w_s[(2) n_out_s, width_s]^T -> out_s [shared_rows, n_out_s]).
extern "C" int ix_moe_grouped_dual(const void* a, const void* w, void* out, const int32_t* offsets,
                                   const int32_t* rows, const int32_t* tile_expert, const int32_t* tile_row0,
                                   const int32_t* tile_info, int max_tiles, int tile_rows, int64_t n_out,
                                   int64_t width, const void* a_s, const void* w_s, void* out_s, int shared_rows,
                                   int64_t n_out_s, int64_t width_s, int gate_up, hipStream_t stream) {
  IX_REQUIRE(n_out > 0 && width > 0 && n_out_s > 0 && width_s > 0 && max_tiles >= 0 && shared_rows > 0,
             "sizes must be positive");
  IX_REQUIRE(width % 8 == 0 && width_s % 8 == 0, "the reduction widths must be multiples of 8");
  IX_REQUIRE(n_out < (1 << 24) && width < (1 << 30) && n_out_s < (1 << 24) && width_s < (1 << 30), "sizes too large");
  IX_REQUIRE(tile_rows == 16 || tile_rows == 32 || tile_rows == 64, "tile_rows must be 16, 32 or 64");
  // one column block per workgroup: two (the rows read once for 32 out-features) measured slower at every tile
  // height, 64 against 60 us for the gate|up product of a decoding step, for want of wavefronts in flight
  const int nb = 1;
  const int64_t n16_e = (n_out + 16 * nb - 1) / (16 * nb), n16_s = (n_out_s + 16 * nb - 1) / (16 * nb);
  const int64_t shared_tiles = (shared_rows + tile_rows - 1) / tile_rows;
  const int64_t blocks = n16_e * max_tiles + n16_s * shared_tiles;
  IX_REQUIRE(blocks < (1ll << 31), "too many workgroups");
  dim3 grid(static_cast<unsigned>(blocks)), block(256);
#define LAUNCH(MT, GU, NB)                                                                                        \
  hipLaunchKernelGGL((moe_grouped_dual_kernel<MT, GU, NB>), grid, block, 0, stream, (const __bf16*)a, (const __bf16*)w, \
                     (__bf16*)out, offsets, rows, tile_expert, tile_row0, tile_info, max_tiles, (int)n_out,        \
                     (int)width, (const __bf16*)a_s, (const __bf16*)w_s, (__bf16*)out_s, shared_rows, (int)n_out_s, \
                     (int)width_s)
#define PICK(MT, NB)                 \
  if (gate_up) LAUNCH(MT, true, NB); \
  else LAUNCH(MT, false, NB);
  if (tile_rows == 16) { PICK(1, 1) } else if (tile_rows == 32) { PICK(2, 1) } else { PICK(4, 1) }
#undef PICK
#undef LAUNCH
  return ix_check_launch("ix_moe_grouped_dual");
}

// out float32 [rows, n_out] = x [rows, width] . w[n_out, width]^T, rows <= 64, bfloat16 operands.
extern "C" int ix_linear_skinny_f32(const void* x, const void* w, float* out, int rows, int64_t n_out, int64_t width,
                                    hipStream_t stream) {
  IX_REQUIRE(rows > 0 && rows <= 64 && n_out > 0 && width > 0, "between 1 and 64 rows, positive sizes");
  IX_REQUIRE(width % 8 == 0, "the reduction width must be a multiple of 8");
  IX_REQUIRE(n_out < (1ll << 31) - 16 && width < (1 << 30), "sizes too large");
  dim3 grid(static_cast<unsigned>((n_out + 31) / 32)), block(256);
  if (rows <= 16)
    hipLaunchKernelGGL(linear_skinny_f32_kernel<1>, grid, block, 0, stream, (const __bf16*)x, (const __bf16*)w, out,
                       rows, (int)n_out, (int)width);
  else if (rows <= 32)
    hipLaunchKernelGGL(linear_skinny_f32_kernel<2>, grid, block, 0, stream, (const __bf16*)x, (const __bf16*)w, out,
                       rows, (int)n_out, (int)width);
  else
    hipLaunchKernelGGL(linear_skinny_f32_kernel<4>, grid, block, 0, stream, (const __bf16*)x, (const __bf16*)w, out,
                       rows, (int)n_out, (int)width);
  return ix_check_launch("ix_linear_skinny_f32");
}
