// Grouped expert products for many rows per expert (prompt portions), bfloat16,
// staged through LDS.  Same results as moe_mfma.hip's kernel; that one streams
// each operand per wavefront, which is right when the weights are the traffic
// (decoding) and wasteful when dozens of rows share them.
//
// A workgroup owns up to 160 rows of one expert (a row tile of the grouping
// kernel's map; with a few hundred tokens that is all rows of the expert, so
// its weights are read once) x 128 weight rows: for the gate|up product 64 gate
// rows and the 64 up rows that belong to them (64 output columns after SwiGLU),
// for the down product 128 output columns.  Only the sixteens of rows that the
// tile really holds are multiplied.  The reduction runs in stages of 64: the
// next stage's global loads are issued into registers before the current stage
// is multiplied out of LDS.  LDS rows are padded to 144 bytes so that the
// 16-byte operand reads of a wavefront quarter fall on distinct banks.
//
// As in moe_mfma.hip the product is formed transposed (A = weight rows,
// B = activation rows), so lane l ends up with four consecutive output
// columns of one row.  The four wavefronts are laid out 2 x 2: wavefront
// (wi, xi) owns 64 of the weight rows (for gate|up: 32 gate rows and their up
// rows) and every second sixteen of activation rows, so it reads 4 + 5 operand
// pieces for 20 products.
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

#define TL_ROWS 160   // the row-tile map is made for tiles of this many rows
#define TL_WROWS 128
#define TL_K 64
#define TL_STRIDE 72  // elements per LDS row: 64 + 8 of padding

// One row tile x 128 weight rows.  NP: pairs of sixteens of activation rows the tile holds (1..5); with it a
// template parameter, and every load unconditional (a stage past the end asks for the last stage again, a piece
// past the row's end for the row's start, and what comes back is replaced by zero on its way into LDS), the loop is one straight line, so the
// compiler can count exactly how many loads may stay in flight at each wait.  With branches in the loop it
// waited for all of them, also those of three stages ahead.
template <bool GATE_UP, int NP>
__device__ __forceinline__ void
tiled_body(const __bf16* a, const __bf16* w, __bf16* out, const int32_t* __restrict__ rows, int n_out, int width, int e, int row0, int row_end, __bf16* ws,
           __bf16* xs) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int m = lane & 15, g = lane >> 4;
  const int wi = wave & 1, xi = wave >> 1;
  constexpr int COLS = GATE_UP ? 64 : 128;  // output columns of this workgroup
  const int n0 = blockIdx.x * COLS;

  // what this thread copies per stage: 4 pieces of 8 weights, NP pieces of 8 activations
  const int64_t w_rows = GATE_UP ? 2 * static_cast<int64_t>(n_out) : n_out;
  // (32-bit offsets: the entry point has checked that one expert's weights and the activations stay below 2^31)
  const __bf16* w_expert = w + static_cast<int64_t>(e) * w_rows * width;
  const int kc_mine = (tid & 7) * 8;  // the same for all of this thread's pieces
  int wsrc[4], wdst[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int c = tid + 256 * i, r = c >> 3;
    int src_row;
    if (GATE_UP)
      src_row = (r < 64 ? 0 : n_out) + min(n0 + (r & 63), n_out - 1);
    else
      src_row = min(n0 + r, n_out - 1);
    wsrc[i] = src_row * width;
    wdst[i] = r * TL_STRIDE + kc_mine;
  }
  int xsrc[NP];
#pragma unroll
  for (int i = 0; i < NP; ++i) {
    const int r = (tid >> 3) + 32 * i;
    const int gr = min(row0 + r, row_end - 1);  // rows past the end repeat the last one; their results are dropped
    xsrc[i] = (rows ? rows[gr] : gr) * width;
  }
  const int xdst = (tid >> 3) * TL_STRIDE + kc_mine;

  const bf16x8 zero = {(__bf16)0.f, (__bf16)0.f, (__bf16)0.f, (__bf16)0.f,
                       (__bf16)0.f, (__bf16)0.f, (__bf16)0.f, (__bf16)0.f};
  // The weights come from memory and are what the kernel waits for: three register sets keep the loads of three
  // stages on their way while a fourth stage is multiplied out of LDS.  The activations are asked for two stages
  // ahead, in two sets.
  bf16x8 wreg[3][4], xreg[2][NP];
  // Row tiles walk the reduction in the same order but start at different stages (and wrap round): were all
  // workgroups at the same offset of their weight rows at the same time, a row length that is a power of two
  // would send their loads to the same few memory channels (measured with few rows per expert: 4.0 instead of
  // 5.0 TB/s at rows of 4,096 bytes).  The order of a workgroup's additions depends only on its place in the
  // grid, so results repeat bit for bit.
  const int kspan = ((width + TL_K - 1) / TL_K) * TL_K;
  const int rot = (width % 512 == 0)  // rows of a multiple of 1,024 bytes; workgroups of one row tile stay together
                      ? static_cast<int>((blockIdx.y * 3u) % static_cast<unsigned>(kspan / TL_K)) * TL_K
                      : 0;         // (they read the same activations, which then stay in L2)
  // where this thread's pieces of stage k0 start in a row, and whether they exist
  auto place = [&](int k0, bool& ok) {
    k0 = min(k0, kspan - TL_K);
    const int k = (k0 + rot < kspan ? k0 + rot : k0 + rot - kspan) + kc_mine;
    ok = k < width;
    return ok ? k : 0;
  };
  auto fetch_w = [&](int k0, bf16x8 (&wr)[4]) {
    bool ok;
    const int k = place(k0, ok);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      wr[i] = *reinterpret_cast<const bf16x8*>(w_expert + wsrc[i] + k);
    }
  };
  auto fetch_x = [&](int k0, bf16x8 (&xr)[NP]) {
    bool ok;
    const int k = place(k0, ok);
#pragma unroll
    for (int i = 0; i < NP; ++i) {
      xr[i] = *reinterpret_cast<const bf16x8*>(a + xsrc[i] + k);
    }
  };
  // (what was loaded for a piece that does not exist becomes zero here, not at the load: the loads' results are
  // not touched before they are needed)
  auto stage = [&](int k0, const bf16x8 (&wr)[4], const bf16x8 (&xr)[NP]) {
    bool ok;
    place(k0, ok);
#pragma unroll
    for (int i = 0; i < 4; ++i) *reinterpret_cast<bf16x8*>(ws + wdst[i]) = ok ? wr[i] : zero;
#pragma unroll
    for (int i = 0; i < NP; ++i) *reinterpret_cast<bf16x8*>(xs + xdst + 32 * i * TL_STRIDE) = ok ? xr[i] : zero;
  };

  // weight blocks of this wavefront: gate|up 32 wi + {0, 16} and the same + 64; down 64 wi + 16 j
  int wblock[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) wblock[j] = GATE_UP ? 32 * wi + 16 * (j & 1) + 64 * (j >> 1) : 64 * wi + 16 * j;
  f32x4 acc[4][NP];
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int t = 0; t < NP; ++t) acc[j][t] = f32x4{0.f, 0.f, 0.f, 0.f};

  auto multiply = [&]() {
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      const int col = 32 * kk + 8 * g;
      bf16x8 wa[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) wa[j] = *reinterpret_cast<const bf16x8*>(ws + (wblock[j] + m) * TL_STRIDE + col);
#pragma unroll
      for (int t = 0; t < NP; ++t) {  // sixteen 2 t + xi (an odd count of sixteens: the last one of xi = 1 is idle work)
        const bf16x8 xb = *reinterpret_cast<const bf16x8*>(xs + (16 * (2 * t + xi) + m) * TL_STRIDE + col);
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[j][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa[j], xb, acc[j][t], 0, 0, 0);
      }
    }
  };

  fetch_w(0, wreg[0]);
  fetch_x(0, xreg[0]);
  stage(0, wreg[0], xreg[0]);
  fetch_w(TL_K, wreg[1]);
  fetch_x(TL_K, xreg[1]);
  fetch_w(2 * TL_K, wreg[2]);
  __syncthreads();
  // One stage s: ask for the weights of stage s + 3 and the activations of stage s + 2 (into the sets that held
  // stage s, which is in LDS), multiply, then move stage s + 1 into LDS.  Six stages per turn, so that the
  // register sets (three of weights, two of activations) are named statically.
#define TL_STAGE(K0, W_FREE, W_NEXT, X_FREE, X_NEXT)                              \
  {                                                                               \
    fetch_w((K0) + 3 * TL_K, wreg[W_FREE]);                                       \
    fetch_x((K0) + 2 * TL_K, xreg[X_FREE]);                                       \
    __builtin_amdgcn_sched_barrier(0); /* the loads stay ahead of the products */ \
    multiply();                                                                   \
    __builtin_amdgcn_sched_barrier(0);                                            \
    __syncthreads();                                                              \
    if ((K0) + TL_K >= width) break;                                              \
    stage((K0) + TL_K, wreg[W_NEXT], xreg[X_NEXT]);                               \
    __syncthreads();                                                              \
  }
  for (int k0 = 0;; k0 += 6 * TL_K) {
    TL_STAGE(k0, 0, 1, 0, 1)
    TL_STAGE(k0 + TL_K, 1, 2, 1, 0)
    TL_STAGE(k0 + 2 * TL_K, 2, 0, 0, 1)
    TL_STAGE(k0 + 3 * TL_K, 0, 1, 1, 0)
    TL_STAGE(k0 + 4 * TL_K, 1, 2, 0, 1)
    TL_STAGE(k0 + 5 * TL_K, 2, 0, 1, 0)
  }
#undef TL_STAGE

  // lane holds weight rows (block) + 4 g + i of activation row row0 + 16 (2 t + xi) + m
  const bool vec = (n_out & 3) == 0;
#pragma unroll
  for (int t = 0; t < NP; ++t) {
    const int r = row0 + 16 * (2 * t + xi) + m;
    if (r >= row_end) continue;
    if (GATE_UP) {
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int nb = n0 + 32 * wi + 16 * j + 4 * g;
        float v[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float gate = acc[j][t][i];
          v[i] = gate / (1.0f + __expf(-gate)) * acc[2 + j][t][i];
        }
        __bf16* dst = out + static_cast<int64_t>(r) * n_out + nb;
        if (nb + 4 <= n_out && vec) {
          bf16x4 o = {(__bf16)v[0], (__bf16)v[1], (__bf16)v[2], (__bf16)v[3]};
          *reinterpret_cast<bf16x4*>(dst) = o;
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (nb + i < n_out) dst[i] = (__bf16)v[i];
        }
      }
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int nb = n0 + 64 * wi + 16 * j + 4 * g;
        __bf16* dst = out + static_cast<int64_t>(r) * n_out + nb;
        if (nb + 4 <= n_out && vec) {
          bf16x4 o = {(__bf16)acc[j][t][0], (__bf16)acc[j][t][1], (__bf16)acc[j][t][2], (__bf16)acc[j][t][3]};
          *reinterpret_cast<bf16x4*>(dst) = o;
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (nb + i < n_out) dst[i] = (__bf16)acc[j][t][i];
        }
      }
    }
  }
}

template <bool GATE_UP>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2)))
moe_grouped_tiled_kernel(const __bf16* a, const __bf16* w, __bf16* out, const int32_t* __restrict__ offsets, const int32_t* __restrict__ rows,
                         const int32_t* __restrict__ tile_expert, const int32_t* __restrict__ tile_row0,
                         const int32_t* __restrict__ tile_info, int n_out, int width) {
  __shared__ __attribute__((aligned(16))) __bf16 ws[TL_WROWS * TL_STRIDE];
  __shared__ __attribute__((aligned(16))) __bf16 xs[TL_ROWS * TL_STRIDE];
  if (static_cast<int>(blockIdx.y) >= tile_info[0]) return;
  const int e = tile_expert[blockIdx.y];
  const int row0 = tile_row0[blockIdx.y];
  const int row_end = offsets[e + 1];
  const int held = min(TL_ROWS, row_end - row0);
  if (held <= 0) return;
  switch ((held + 31) >> 5) {  // pairs of sixteens of rows this tile holds
    case 1: tiled_body<GATE_UP, 1>(a, w, out, rows, n_out, width, e, row0, row_end, ws, xs); break;
    case 2: tiled_body<GATE_UP, 2>(a, w, out, rows, n_out, width, e, row0, row_end, ws, xs); break;
    case 3: tiled_body<GATE_UP, 3>(a, w, out, rows, n_out, width, e, row0, row_end, ws, xs); break;
    case 4: tiled_body<GATE_UP, 4>(a, w, out, rows, n_out, width, e, row0, row_end, ws, xs); break;
    default: tiled_body<GATE_UP, 5>(a, w, out, rows, n_out, width, e, row0, row_end, ws, xs); break;
  }
}

// The row-tile map must have been made for tiles of TL_ROWS (160) rows.
extern "C" int ix_moe_grouped_tiled(const void* a, const void* w, void* out, const int32_t* offsets,
                                    const int32_t* rows, const int32_t* tile_expert, const int32_t* tile_row0,
                                    const int32_t* tile_info, int max_tiles, int64_t a_rows, int64_t n_out,
                                    int64_t width, int gate_up, hipStream_t stream) {
  IX_REQUIRE(n_out > 0 && width > 0 && max_tiles >= 0, "sizes must be positive");
  IX_REQUIRE(width % 8 == 0, "the reduction width must be a multiple of 8 for the matrix-core kernel");
  IX_REQUIRE(n_out < (1 << 30) && width < (1 << 30), "sizes too large");
  IX_REQUIRE(a_rows >= 0 && a_rows * width < (int64_t(1) << 31) && (gate_up ? 2 : 1) * n_out * width < (int64_t(1) << 31),
             "the activations, and one expert's weights, must hold fewer than 2^31 numbers");
  IX_REQUIRE(max_tiles <= 65535, "too many row tiles for one launch");
  if (max_tiles == 0) return 0;
  const int cols = gate_up ? 64 : 128;
  dim3 grid(static_cast<unsigned>((n_out + cols - 1) / cols), max_tiles), block(256);
  if (gate_up)
    hipLaunchKernelGGL(moe_grouped_tiled_kernel<true>, grid, block, 0, stream, (const __bf16*)a, (const __bf16*)w,
                       (__bf16*)out, offsets, rows, tile_expert, tile_row0, tile_info, (int)n_out, (int)width);
  else
    hipLaunchKernelGGL(moe_grouped_tiled_kernel<false>, grid, block, 0, stream, (const __bf16*)a, (const __bf16*)w,
                       (__bf16*)out, offsets, rows, tile_expert, tile_row0, tile_info, (int)n_out, (int)width);
  return ix_check_launch("ix_moe_grouped_tiled");
}
