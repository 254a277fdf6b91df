// Grouped expert products for many rows per expert (prompt portions), bfloat16,
// staged through LDS.  Same results as moe_mfma.hip's kernel; that one streams
// each operand per wavefront, which is right when the weights are the traffic
// (decoding) and wasteful when dozens of rows share them.
//
// A workgroup owns up to 160 rows of one expert, 192 in the wide form (a row
// tile of the grouping kernel's map; with a few hundred tokens that is all rows
// of the expert, so its weights are read once) x 128 weight rows: for the gate|up product 64 gate
// rows and the 64 up rows that belong to them (64 output columns after SwiGLU),
// for the down product 128 output columns.  Only the pairs of sixteens of rows
// that the tile really holds are multiplied.  The reduction runs in stages of
// 64 through two LDS buffers: while one stage is multiplied, the next one is
// already in the other buffer, the weights of three further stages and the
// activations of two are on their way from memory into registers, and one
// barrier per stage is enough.  LDS rows are 128 bytes with their 16-byte
// pieces permuted, so that operand reads and writes fall on distinct banks.
//
// As in moe_mfma.hip the product is formed transposed (A = weight rows,
// B = activation rows), so lane l ends up with four consecutive output
// columns of one row.  The four wavefronts are laid out 2 x 2: wavefront
// (wi, xi) owns 64 of the weight rows (for gate|up: 32 gate rows and their up
// rows) and every second sixteen of activation rows, so it reads 4 + 5 operand
// pieces for 20 products.
//
// The wide form has eight wavefronts, 4 x 2, and 256 weight rows per workgroup
// (template parameter NWW = 4): per product it moves less through LDS and L2,
// and it fills a compute unit's LDS alone.
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

// the row-tile map is made for tiles of this many rows (the wide form has LDS for 192)
#define TL_ROWS(NWW) ((NWW) == 2 ? 160 : 192)
#define TL_K 64
#define TL_STRIDE 64  // elements per LDS row: no padding; the eight 16-byte pieces of a row are stored permuted
// NWW: wavefronts along the weight rows (2 or 4; two along the activation rows): 64 NWW weight rows and 128 NWW
// threads per workgroup.  With four, a row tile's activations are read for half as many column blocks.
#define TL_WROWS(NWW) (64 * (NWW))
#define TL_THREADS(NWW) (128 * (NWW))
#define TL_WTILE(NWW) (TL_WROWS(NWW) * TL_STRIDE)
#define TL_XROWS(NWW) ((NWW) == 2 ? 160 : 192)  // staged in steps of 16 NWW rows
#define TL_XTILE(NWW) (TL_XROWS(NWW) * TL_STRIDE)
// piece p of row r lies at piece p ^ ((r >> 1) & 7): the sixteen rows that a quarter of a wavefront reads at one
// piece index then fall on sixteen different groups of four banks, as do the pieces that sixteen lanes write
__device__ __forceinline__ int tl_at(int row, int piece) { return row * TL_STRIDE + ((piece ^ ((row >> 1) & 7)) << 3); }

// One row tile x 128 weight rows.  NP: pairs of sixteens of activation rows the tile holds (1..5).  With it a
// template parameter, and every load unconditional (a stage past the end asks for the last stage again, a piece
// past the row's end for the row's start, and zeros are written over it in LDS), the loop is one straight line,
// so the compiler can count exactly how many loads may stay in flight at each wait.  With branches in the loop
// it waited for all of them, also those of three stages ahead.
template <bool GATE_UP, int NP, int NWW>
__device__ __forceinline__ void
tiled_body(const __bf16* a, const __bf16* w, __bf16* out, const int32_t* __restrict__ rows, int n_out, int width,
           int e, int row0, int row_end, int tile, int col_block, __bf16* ws, __bf16* xs) {
  // (a and w are plain pointers on purpose: loads through `const __restrict__` ones may be moved by the
  // optimiser, which sinks them to their first use and so undoes the prefetch)
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int m = lane & 15, g = lane >> 4;
  const int wi = wave % NWW, xi = wave / NWW;
  constexpr int THREADS = TL_THREADS(NWW), WROWS = TL_WROWS(NWW), HALF = WROWS / 2;
  constexpr int STEP = THREADS / 8;                     // rows that the workgroup's threads stage at once
  constexpr int NPX = (32 * NP + STEP - 1) / STEP;      // pieces of activations per thread and stage
  constexpr int COLS = GATE_UP ? HALF : WROWS;          // output columns of this workgroup
  const int n0 = col_block * COLS;

  // what this thread copies per stage: 4 pieces of 8 weights, NP pieces of 8 activations
  const int64_t w_rows = GATE_UP ? 2 * static_cast<int64_t>(n_out) : n_out;
  // (32-bit offsets: the entry point has checked that one expert's weights and the activations stay below 2^31)
  const __bf16* w_expert = w + static_cast<int64_t>(e) * w_rows * width;
  const int kc_mine = (tid & 7) * 8;  // the same for all of this thread's pieces
  int wsrc[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int c = tid + THREADS * i, r = c >> 3;
    int src_row;
    if (GATE_UP)
      src_row = (r < HALF ? 0 : n_out) + min(n0 + (r % HALF), n_out - 1);
    else
      src_row = min(n0 + r, n_out - 1);
    wsrc[i] = src_row * width;
  }
  int xsrc[NPX];
#pragma unroll
  for (int i = 0; i < NPX; ++i) {
    const int r = (tid >> 3) + STEP * i;
    const int gr = min(row0 + r, row_end - 1);  // rows past the end repeat the last one; their results are dropped
    xsrc[i] = (rows ? rows[gr] : gr) * width;
  }
  const int xdst = tl_at(tid >> 3, tid & 7);  // rows STEP further on have the same permutation

  // The weights come from memory and are what the kernel waits for: three register sets keep the loads of three
  // stages on their way while one stage is multiplied and the next one lies in the other LDS buffer.  The
  // activations, which mostly come from L2, are in two sets.
  bf16x8 wreg[3][4], xreg[2][NPX];
  // Row tiles walk the reduction in the same order but start at different stages (and wrap round): were all
  // workgroups at the same offset of their weight rows at the same time, a row length that is a power of two
  // would send their loads to the same few memory channels (measured with few rows per expert: 4.0 instead of
  // 5.0 TB/s at rows of 4,096 bytes).  The order of a workgroup's additions depends only on its place in the
  // grid, so results repeat bit for bit.
  const int kspan = ((width + TL_K - 1) / TL_K) * TL_K;
  const int rot = (width % 512 == 0)  // rows of a multiple of 1,024 bytes; workgroups of one row tile stay together
                      ? static_cast<int>((static_cast<unsigned>(tile) * 3u) % static_cast<unsigned>(kspan / TL_K)) * TL_K
                      : 0;         // (they read the same activations, which then stay in L2)
  // Where this thread's pieces of stage k0 start in a row, and whether they exist.  A piece that does not exist
  // (the reduction width is no multiple of 64) is loaded from the row's start instead and overwritten with
  // zeros in LDS by the thread that put it there: no loaded value is touched before its use, and the branch
  // that does it holds nothing but LDS writes.
  const bool ragged = (width & (TL_K - 1)) != 0;
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
    for (int i = 0; i < 4; ++i) wr[i] = *reinterpret_cast<const bf16x8*>(w_expert + wsrc[i] + k);
  };
  auto fetch_x = [&](int k0, bf16x8 (&xr)[NPX]) {
    bool ok;
    const int k = place(k0, ok);
#pragma unroll
    for (int i = 0; i < NPX; ++i) xr[i] = *reinterpret_cast<const bf16x8*>(a + xsrc[i] + k);
  };
  auto stage = [&](int k0, int buf, const bf16x8 (&wr)[4], const bf16x8 (&xr)[NPX]) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      *reinterpret_cast<bf16x8*>(ws + buf * TL_WTILE(NWW) + xdst + STEP * i * TL_STRIDE) = wr[i];
#pragma unroll
    for (int i = 0; i < NPX; ++i)
      *reinterpret_cast<bf16x8*>(xs + buf * TL_XTILE(NWW) + xdst + STEP * i * TL_STRIDE) = xr[i];
    if (ragged) {
      bool ok;
      place(k0, ok);
      if (!ok) {
        const bf16x8 zero = {(__bf16)0.f, (__bf16)0.f, (__bf16)0.f, (__bf16)0.f,
                             (__bf16)0.f, (__bf16)0.f, (__bf16)0.f, (__bf16)0.f};
#pragma unroll
        for (int i = 0; i < 4; ++i)
          *reinterpret_cast<bf16x8*>(ws + buf * TL_WTILE(NWW) + xdst + STEP * i * TL_STRIDE) = zero;
#pragma unroll
        for (int i = 0; i < NPX; ++i)
          *reinterpret_cast<bf16x8*>(xs + buf * TL_XTILE(NWW) + xdst + STEP * i * TL_STRIDE) = zero;
      }
    }
  };

  f32x4 acc[4][NP];
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int t = 0; t < NP; ++t) acc[j][t] = f32x4{0.f, 0.f, 0.f, 0.f};

  // this lane's operand pieces: row (block) + m, piece 4 kk + g.  Blocks start at multiples of 16 rows, so the
  // permutation depends on m only and a block is a constant distance from the wavefront's first one.
  int wat[2], xat[2];
#pragma unroll
  for (int kk = 0; kk < 2; ++kk) {
    wat[kk] = tl_at((GATE_UP ? 32 : 64) * wi + m, 4 * kk + g);
    xat[kk] = tl_at(16 * xi + m, 4 * kk + g);
  }
  auto multiply = [&](int buf) {
    const __bf16* wt = ws + buf * TL_WTILE(NWW);
    const __bf16* xt = xs + buf * TL_XTILE(NWW);
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      bf16x8 wa[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {  // gate|up: blocks 32 wi + {0, 16} and the same + 64; down: 64 wi + 16 j
        const int block = GATE_UP ? 16 * (j & 1) + HALF * (j >> 1) : 16 * j;
        wa[j] = *reinterpret_cast<const bf16x8*>(wt + wat[kk] + block * TL_STRIDE);
      }
#pragma unroll
      for (int t = 0; t < NP; ++t) {  // sixteen 2 t + xi (an odd count of sixteens: the last one of xi = 1 is idle work)
        const bf16x8 xb = *reinterpret_cast<const bf16x8*>(xt + xat[kk] + 32 * t * TL_STRIDE);
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[j][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa[j], xb, acc[j][t], 0, 0, 0);
      }
    }
  };

  // (the loads are asked for in the order in which the loop leaves them behind, so that the count of loads that
  // may stay in flight at the loop's first wait is the same on the way in and on the way round)
  fetch_w(0, wreg[0]);
  __builtin_amdgcn_sched_barrier(0);
  fetch_w(TL_K, wreg[1]);
  __builtin_amdgcn_sched_barrier(0);
  fetch_x(0, xreg[0]);
  __builtin_amdgcn_sched_barrier(0);
  fetch_w(2 * TL_K, wreg[2]);
  __builtin_amdgcn_sched_barrier(0);
  fetch_x(TL_K, xreg[1]);
  __builtin_amdgcn_sched_barrier(0);
  stage(0, 0, wreg[0], xreg[0]);
  fetch_w(3 * TL_K, wreg[0]);
  __builtin_amdgcn_sched_barrier(0);
  fetch_x(2 * TL_K, xreg[0]);
  __builtin_amdgcn_sched_barrier(0);
  __syncthreads();
  // Stage s is in LDS buffer s & 1.  First stage s + 1 goes from its registers into the other buffer (whose last
  // readers passed the previous barrier); the registers it leaves take the loads of the weights of stage s + 4 and
  // the activations of stage s + 3; then stage s is multiplied; one barrier.  Six stages per turn, so that the
  // register sets (three of weights, two of activations) are named statically.
  // The loads stay ahead of the products; LDS reads and writes may be moved across that line (mask: DS), so that
  // this stage's operand reads start while the next stage's writes are still going out: 188 + 108 against
  // 207 + 115 us at 2,048 tokens of 60 experts of 1,408, 1,023 + 541 against 1,114 + 547 in the wide form at 64
  // experts of 2,560, same bits, the kernels alone with even routing.  (Nothing may cross: the slower figures; plain
  // arithmetic as well: as slow.)  Inside the model, beside the shared expert's products and with the router's
  // uneven rows per expert, a step gains 1 % at most.
#define TL_STAGE(K0, BUF, W_NEXT, X_NEXT)                                         \
  {                                                                               \
    stage((K0) + TL_K, 1 - (BUF), wreg[W_NEXT], xreg[X_NEXT]);                    \
    fetch_w((K0) + 4 * TL_K, wreg[W_NEXT]);                                       \
    fetch_x((K0) + 3 * TL_K, xreg[X_NEXT]);                                       \
    __builtin_amdgcn_sched_barrier(0x100 | 0x200 | 0x80);                         \
    if ((K0) < kspan) multiply(BUF);                                              \
    __builtin_amdgcn_sched_barrier(0);                                            \
    __syncthreads();                                                              \
  }
  // Whole turns only, and no way out of a turn's middle: a way out would join the states of the loads of all
  // stages, and the loop's first wait would have to be for the worst of them.  Stages past the end ask for the
  // last stage's operands again and multiply nothing (that branch holds no loads).
  for (int k0 = 0; k0 < kspan; k0 += 6 * TL_K) {
    TL_STAGE(k0, 0, 1, 1)
    TL_STAGE(k0 + TL_K, 1, 2, 0)
    TL_STAGE(k0 + 2 * TL_K, 0, 0, 1)
    TL_STAGE(k0 + 3 * TL_K, 1, 1, 0)
    TL_STAGE(k0 + 4 * TL_K, 0, 2, 1)
    TL_STAGE(k0 + 5 * TL_K, 1, 0, 0)
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

template <bool GATE_UP, int NWW>
__global__ void __launch_bounds__(TL_THREADS(NWW)) __attribute__((amdgpu_waves_per_eu(2, 2)))
moe_grouped_tiled_kernel(const __bf16* a, const __bf16* w, __bf16* out, const int32_t* __restrict__ offsets,
                         const int32_t* __restrict__ rows,
                         const int32_t* __restrict__ tile_expert, const int32_t* __restrict__ tile_row0,
                         const int32_t* __restrict__ tile_info, int n_out, int width, int n_col_blocks) {
  __shared__ __attribute__((aligned(16))) __bf16 ws[2 * TL_WTILE(NWW)];
  __shared__ __attribute__((aligned(16))) __bf16 xs[2 * TL_XTILE(NWW)];
  // Workgroups go to the chip's eight dies in turn, by their number.  All column blocks of a row tile read the
  // same activations: they are numbered so that they land on one die and share its L2 (tile t on die t % 8).
  const int slot = blockIdx.x >> 3;
  const int tile = (slot / n_col_blocks) * 8 + (blockIdx.x & 7), col_block = slot % n_col_blocks;
  if (tile >= tile_info[0]) return;
  const int e = tile_expert[tile];
  const int row0 = tile_row0[tile];
  const int row_end = offsets[e + 1];
  const int held = min(TL_ROWS(NWW), row_end - row0);
  if (held <= 0) return;
  switch ((held + 31) >> 5) {  // pairs of sixteens of rows this tile holds
    case 1: tiled_body<GATE_UP, 1, NWW>(a, w, out, rows, n_out, width, e, row0, row_end, tile, col_block, ws, xs); break;
    case 2: tiled_body<GATE_UP, 2, NWW>(a, w, out, rows, n_out, width, e, row0, row_end, tile, col_block, ws, xs); break;
    case 3: tiled_body<GATE_UP, 3, NWW>(a, w, out, rows, n_out, width, e, row0, row_end, tile, col_block, ws, xs); break;
    case 4: tiled_body<GATE_UP, 4, NWW>(a, w, out, rows, n_out, width, e, row0, row_end, tile, col_block, ws, xs); break;
    case 5: tiled_body<GATE_UP, 5, NWW>(a, w, out, rows, n_out, width, e, row0, row_end, tile, col_block, ws, xs); break;
    default:  // (six pairs of sixteens in the wide form only)
      tiled_body<GATE_UP, NWW == 4 ? 6 : 5, NWW>(a, w, out, rows, n_out, width, e, row0, row_end, tile, col_block, ws, xs);
      break;
  }
}

// The row-tile map must have been made for tiles of 160 rows, for the wide form of 192.  `wide`: see below.
extern "C" int ix_moe_grouped_tiled(const void* a, const void* w, void* out, const int32_t* offsets,
                                    const int32_t* rows, const int32_t* tile_expert, const int32_t* tile_row0,
                                    const int32_t* tile_info, int max_tiles, int64_t a_rows, int64_t n_out,
                                    int64_t width, int gate_up, int wide, hipStream_t stream) {
  IX_REQUIRE(n_out > 0 && width > 0 && max_tiles >= 0, "sizes must be positive");
  IX_REQUIRE(width % 8 == 0, "the reduction width must be a multiple of 8 for the matrix-core kernel");
  IX_REQUIRE(n_out < (1 << 30) && width < (1 << 30), "sizes too large");
  IX_REQUIRE(a_rows >= 0 && a_rows * width < (int64_t(1) << 31) && (gate_up ? 2 : 1) * n_out * width < (int64_t(1) << 31),
             "the activations, and one expert's weights, must hold fewer than 2^31 numbers");
  IX_REQUIRE(max_tiles <= 65535, "too many row tiles for one launch");
  if (max_tiles == 0) return 0;
  // wide: four wavefronts along the weight rows instead of two (256 weight rows per workgroup, 112 KB of LDS, one
  // workgroup per compute unit): the activations are staged for half as many column blocks.  Same sums in the
  // same order either way.
  const int nww = wide ? 4 : 2;
  const int cols = gate_up ? 32 * nww : 64 * nww;
  const int n_col_blocks = static_cast<int>((n_out + cols - 1) / cols);
  const int64_t groups = 8 * static_cast<int64_t>(n_col_blocks) * ((max_tiles + 7) / 8);
  IX_REQUIRE(groups < (int64_t(1) << 31), "too many workgroups for one launch");
  dim3 grid(static_cast<unsigned>(groups)), block(TL_THREADS(nww));
#define LAUNCH(GU, NWW)                                                                                             \
  hipLaunchKernelGGL((moe_grouped_tiled_kernel<GU, NWW>), grid, block, 0, stream, (const __bf16*)a, (const __bf16*)w, \
                     (__bf16*)out, offsets, rows, tile_expert, tile_row0, tile_info, (int)n_out, (int)width,         \
                     n_col_blocks)
  if (nww == 4) {
    if (gate_up) LAUNCH(true, 4);
    else LAUNCH(false, 4);
  } else {
    if (gate_up) LAUNCH(true, 2);
    else LAUNCH(false, 2);
  }
#undef LAUNCH
  return ix_check_launch("ix_moe_grouped_tiled");
}
