// Grouped expert products for many rows per expert (prompt portions), bfloat16,
// staged through LDS.  Same results as moe_mfma.hip's kernel; that one streams
// each operand per wavefront, which is right when the weights are the traffic
// (decoding) and wasteful when dozens of rows share them.
//
// A workgroup owns 64 rows of one expert (a row tile of the grouping kernel's
// map) x 128 weight rows: for the gate|up product 64 gate rows and the 64 up
// rows that belong to them (64 output columns after SwiGLU), for the down
// product 128 output columns.  The reduction runs in stages of 64: the next
// stage's global loads are issued into registers before the current stage is
// multiplied out of LDS.  LDS rows are padded to 144 bytes so that the sixteen
// 16-byte operand reads of a wavefront quarter fall on distinct banks.
//
// As in moe_mfma.hip the product is formed transposed (A = weight rows,
// B = activation rows), so lane l ends up with four consecutive output
// columns of one row.  Wavefront w owns weight blocks (w, 4 + w) [gate|up] or
// (2w, 2w + 1) [down] and all four row blocks.
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

#define TL_ROWS 64
#define TL_WROWS 128
#define TL_K 64
#define TL_STRIDE 72  // elements per LDS row: 64 + 8 of padding

template <bool GATE_UP>
__global__ void __launch_bounds__(256)
moe_grouped_tiled_kernel(const __bf16* __restrict__ a, const __bf16* __restrict__ w, __bf16* __restrict__ out,
                         const int32_t* __restrict__ offsets, const int32_t* __restrict__ rows,
                         const int32_t* __restrict__ tile_expert, const int32_t* __restrict__ tile_row0,
                         const int32_t* __restrict__ tile_info, int n_out, int width) {
  __shared__ __attribute__((aligned(16))) __bf16 ws[TL_WROWS * TL_STRIDE];
  __shared__ __attribute__((aligned(16))) __bf16 xs[TL_ROWS * TL_STRIDE];
  if (static_cast<int>(blockIdx.y) >= tile_info[0]) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int m = lane & 15, g = lane >> 4;
  const int e = tile_expert[blockIdx.y];
  const int row0 = tile_row0[blockIdx.y];
  const int row_end = offsets[e + 1];
  constexpr int COLS = GATE_UP ? 64 : 128;  // output columns of this workgroup
  const int n0 = blockIdx.x * COLS;

  // what this thread copies per stage: 4 chunks of 8 weights, 2 chunks of 8 activations
  const int64_t w_rows = GATE_UP ? 2 * static_cast<int64_t>(n_out) : n_out;
  const __bf16* wsrc[4];
  int wdst[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int c = tid + 256 * i, r = c >> 3, kc = (c & 7) * 8;
    int64_t src_row;
    if (GATE_UP)
      src_row = (r < 64 ? 0 : n_out) + min(n0 + (r & 63), n_out - 1);
    else
      src_row = min(n0 + r, n_out - 1);
    wsrc[i] = w + (static_cast<int64_t>(e) * w_rows + src_row) * width + kc;
    wdst[i] = r * TL_STRIDE + kc;
  }
  const __bf16* xsrc[2];
  int xdst[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int c = tid + 256 * i, r = c >> 3, kc = (c & 7) * 8;
    const int gr = min(row0 + r, row_end - 1);
    xsrc[i] = a + static_cast<int64_t>(rows ? rows[gr] : gr) * width + kc;
    xdst[i] = r * TL_STRIDE + kc;
  }
  const int kc_mine = (tid & 7) * 8;  // the same for all of this thread's chunks

  const bf16x8 zero = {(__bf16)0.f, (__bf16)0.f, (__bf16)0.f, (__bf16)0.f,
                       (__bf16)0.f, (__bf16)0.f, (__bf16)0.f, (__bf16)0.f};
  bf16x8 wreg[4], xreg[2];
  auto fetch = [&](int k0) {
    const bool ok = k0 + kc_mine < width;
#pragma unroll
    for (int i = 0; i < 4; ++i) wreg[i] = ok ? *reinterpret_cast<const bf16x8*>(wsrc[i] + k0) : zero;
#pragma unroll
    for (int i = 0; i < 2; ++i) xreg[i] = ok ? *reinterpret_cast<const bf16x8*>(xsrc[i] + k0) : zero;
  };
  auto stage = [&]() {
#pragma unroll
    for (int i = 0; i < 4; ++i) *reinterpret_cast<bf16x8*>(ws + wdst[i]) = wreg[i];
#pragma unroll
    for (int i = 0; i < 2; ++i) *reinterpret_cast<bf16x8*>(xs + xdst[i]) = xreg[i];
  };

  const int wblock0 = GATE_UP ? 16 * wave : 32 * wave;
  const int wblock1 = GATE_UP ? 64 + 16 * wave : 32 * wave + 16;
  f32x4 acc[2][4];
#pragma unroll
  for (int j = 0; j < 2; ++j)
#pragma unroll
    for (int t = 0; t < 4; ++t) acc[j][t] = f32x4{0.f, 0.f, 0.f, 0.f};

  fetch(0);
  stage();
  __syncthreads();
  for (int k0 = 0; k0 < width; k0 += TL_K) {
    const bool more = k0 + TL_K < width;
    if (more) fetch(k0 + TL_K);
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      const int col = 32 * kk + 8 * g;
      const bf16x8 wa0 = *reinterpret_cast<const bf16x8*>(ws + (wblock0 + m) * TL_STRIDE + col);
      const bf16x8 wa1 = *reinterpret_cast<const bf16x8*>(ws + (wblock1 + m) * TL_STRIDE + col);
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const bf16x8 xb = *reinterpret_cast<const bf16x8*>(xs + (16 * t + m) * TL_STRIDE + col);
        acc[0][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa0, xb, acc[0][t], 0, 0, 0);
        acc[1][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa1, xb, acc[1][t], 0, 0, 0);
      }
    }
    __syncthreads();
    if (more) {
      stage();
      __syncthreads();
    }
  }

  // lane holds weight rows (block) + 4 g + i of activation row row0 + 16 t + m
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    const int r = row0 + 16 * t + m;
    if (r >= row_end) continue;
    if (GATE_UP) {
      const int nb = n0 + 16 * wave + 4 * g;
      float v[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float gate = acc[0][t][i];
        v[i] = gate / (1.0f + __expf(-gate)) * acc[1][t][i];
      }
      __bf16* dst = out + static_cast<int64_t>(r) * n_out + nb;
      if (nb + 4 <= n_out && (n_out & 3) == 0) {
        bf16x4 o = {(__bf16)v[0], (__bf16)v[1], (__bf16)v[2], (__bf16)v[3]};
        *reinterpret_cast<bf16x4*>(dst) = o;
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (nb + i < n_out) dst[i] = (__bf16)v[i];
      }
    } else {
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int nb = n0 + 32 * wave + 16 * j + 4 * g;
        __bf16* dst = out + static_cast<int64_t>(r) * n_out + nb;
        if (nb + 4 <= n_out && (n_out & 3) == 0) {
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

// The row-tile map must have been made for tiles of 64 rows.
extern "C" int ix_moe_grouped_tiled(const void* a, const void* w, void* out, const int32_t* offsets,
                                    const int32_t* rows, const int32_t* tile_expert, const int32_t* tile_row0,
                                    const int32_t* tile_info, int max_tiles, int64_t n_out, int64_t width, int gate_up,
                                    hipStream_t stream) {
  IX_REQUIRE(n_out > 0 && width > 0 && max_tiles >= 0, "sizes must be positive");
  IX_REQUIRE(width % 8 == 0, "the reduction width must be a multiple of 8 for the matrix-core kernel");
  IX_REQUIRE(n_out < (1 << 30) && width < (1 << 30), "sizes too large");
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
