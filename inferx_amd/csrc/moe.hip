// Mixture-of-experts feed-forward: router (product, softmax, top-k in float32),
// grouping of assignments by expert, the plain grouped matrix products, and
// the weighted sum with the shared expert.
//
// Placement is deterministic: no floating-point atomics anywhere, rows of one
// expert keep token order (reference: ops/moe.h:26-33, moe.cu:130-221).
#include "common.h"
#include "moe_route.h"

#define ROUTE_THREADS 256
#define IX_MAX_TOP_K 32
#define IX_MAX_EXPERTS 1024

// ---------------------------------------------------------------------------
// Router.  z_e = x . Wr[e] in float32 (the reference rounds z to bfloat16 first,
// moe_ffn.cc:200-203); p = softmax(z) over all experts with the maximum
// subtracted; k rounds of argmax with strict '>' so that the lowest index wins
// a tie; optional renormalisation by the sum of the chosen; times `scale`
// (reference: RouteTopKKernel, moe.cu:36-127).  Output order: descending score.
// If `shared_gate_w` is given, sigmoid(x . shared_gate_w) is written too
// (reference: AddSharedExpertKernel, moe.cu:275-287).
// softmax over z[0..experts) (LDS, overwritten) and k rounds of argmax, by the whole workgroup
// `always` further slots follow the k chosen ones in every token's row of topk_w / topk_e (rows of k + always):
// experts number experts .. experts + always - 1, each with the weight `always_w`: experts that every token uses (a
// shared expert cut into pieces of the routed experts' width), so that grouping, products and the weighted sum treat
// them like the chosen ones.
__device__ __forceinline__ void route_select(float* z, float* red, float* __restrict__ topk_w,
                                             int32_t* __restrict__ topk_e, int64_t t, int experts, int k,
                                             int renormalize, float scale, int always = 0, float always_w = 1.0f) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  float mx = -INFINITY;
  for (int e = tid; e < experts; e += blockDim.x) mx = fmaxf(mx, z[e]);
  mx = ix_block_max(mx, red);
  float sum = 0.f;
  for (int e = tid; e < experts; e += blockDim.x) {
    const float p = expf(z[e] - mx);
    z[e] = p;
    sum += p;
  }
  sum = ix_block_sum(sum, red);  // its barriers also publish z
  if (wave != 0) return;
  const float inv_sum = 1.0f / sum;
  float chosen = 0.f;  // lane s keeps the weight of slot s
  float total = 0.f;
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
    if (lane == slot) chosen = wgt;
    if (lane == 0) {
      topk_e[t * (k + always) + slot] = bi;
      z[bi] = -INFINITY;
    }
    __builtin_amdgcn_wave_barrier();
    __threadfence_block();
  }
  const float f = ((renormalize && total > 0.f) ? 1.0f / total : 1.0f) * scale;
  if (lane < k) topk_w[t * (k + always) + lane] = chosen * f;
  if (lane < always) {
    topk_e[t * (k + always) + k + lane] = experts + lane;
    topk_w[t * (k + always) + k + lane] = always_w;
  }
}

// One workgroup per token: x row in LDS, every router row against it (many tokens: prompt portions).
template <typename T>
__global__ void __launch_bounds__(ROUTE_THREADS)
moe_route_kernel(const T* __restrict__ x, const void* __restrict__ wr, int wr_dtype,
                 const void* __restrict__ shared_gate_w, int sg_dtype, float* __restrict__ topk_w,
                 int32_t* __restrict__ topk_e, float* __restrict__ shared_gate, int64_t width, int experts, int k,
                 int renormalize, float scale, int always) {
  extern __shared__ __align__(16) float smem[];
  float* xs = smem;                        // [width rounded up to 4]
  float* z = smem + ((width + 3) & ~3);    // [experts + 1]
  __shared__ float red[16];
  const int64_t t = blockIdx.x;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  for (int64_t i = tid; i < width; i += ROUTE_THREADS) xs[i] = ix_load(x + t * width + i);
  __syncthreads();
  const int rows = experts + (shared_gate_w ? 1 : 0);
  for (int e = wave; e < rows; e += ROUTE_THREADS / 64) {
    const bool routed = e < experts;
    const float dot = route_row_dot(xs, routed ? wr : shared_gate_w, routed ? wr_dtype : sg_dtype,
                                    routed ? static_cast<int64_t>(e) * width : 0, width, lane);
    if (lane == 0) z[e] = dot;
  }
  __syncthreads();
  const float gate = shared_gate_w ? 1.0f / (1.0f + expf(-z[experts])) : 1.0f;
  if (shared_gate_w && tid == 0) shared_gate[t] = gate;
  route_select(z, red, topk_w, topk_e, t, experts, k, renormalize, scale, always, gate);
}

// Few tokens (decoding): the router rows are spread over many workgroups, one row per wavefront,
// scores go to `logits` [tokens, experts + 1]; a second small kernel selects.
template <typename T>
__global__ void __launch_bounds__(ROUTE_THREADS)
moe_route_logits_kernel(const T* __restrict__ x, const void* __restrict__ wr, int wr_dtype,
                        const void* __restrict__ shared_gate_w, int sg_dtype, float* __restrict__ logits,
                        int64_t width, int experts) {
  extern __shared__ __align__(16) float xs[];  // [width]
  const int64_t t = blockIdx.x;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  for (int64_t i = tid; i < width; i += ROUTE_THREADS) xs[i] = ix_load(x + t * width + i);
  __syncthreads();
  const int rows = experts + (shared_gate_w ? 1 : 0);
  const int e = blockIdx.y * (ROUTE_THREADS / 64) + wave;
  if (e >= rows) return;
  const bool routed = e < experts;
  const float dot = route_row_dot(xs, routed ? wr : shared_gate_w, routed ? wr_dtype : sg_dtype,
                                  routed ? static_cast<int64_t>(e) * width : 0, width, lane);
  if (lane == 0) logits[t * (experts + 1) + e] = dot;
}

__global__ void __launch_bounds__(64)
moe_route_select_kernel(const float* __restrict__ logits, float* __restrict__ topk_w, int32_t* __restrict__ topk_e,
                        float* __restrict__ shared_gate, int experts, int k, int renormalize, float scale,
                        int always) {
  extern __shared__ __align__(16) float z[];  // [experts]
  __shared__ float red[16];
  const int64_t t = blockIdx.x;
  for (int e = threadIdx.x; e < experts; e += 64) z[e] = logits[t * (experts + 1) + e];
  const float gate = shared_gate ? 1.0f / (1.0f + expf(-logits[t * (experts + 1) + experts])) : 1.0f;
  if (shared_gate && threadIdx.x == 0) shared_gate[t] = gate;
  __syncthreads();
  route_select(z, red, topk_w, topk_e, t, experts, k, renormalize, scale, always, gate);
}

// Many tokens, bfloat16 activations and weights: the scores on the matrix cores (exact products of bfloat16
// numbers, float32 sums), to `logits` as above.  A workgroup takes 16 tokens and 16 rows (of the router, then the
// shared gate's row); its four wavefronts split the reduction (32-wide pieces in turn, four of them in flight)
// and add up through LDS.  As in the grouped products the weight rows are the A operand, so a lane ends up with
// four consecutive scores of one token.
typedef __bf16 route_bf16x8 __attribute__((ext_vector_type(8)));
typedef float route_f32x4 __attribute__((ext_vector_type(4)));
__global__ void __launch_bounds__(256)
moe_route_logits_mfma_kernel(const __bf16* __restrict__ x, const __bf16* __restrict__ wr,
                             const __bf16* __restrict__ shared_gate_w, float* __restrict__ logits, int64_t tokens,
                             int width, int experts) {
  __shared__ route_f32x4 part[4][64];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int m = lane & 15, g = lane >> 4;
  const int64_t t0 = static_cast<int64_t>(blockIdx.x) * 16;
  const int rows = experts + (shared_gate_w ? 1 : 0);
  const int r = 16 * blockIdx.y + m;  // this lane's weight row
  const __bf16* xrow = x + min(t0 + m, tokens - 1) * width;  // tokens past the end repeat the last; not written
  const __bf16* wrow = r < experts ? wr + static_cast<int64_t>(r) * width : (r < rows ? shared_gate_w : nullptr);
  route_bf16x8 zero;
  for (int j = 0; j < 8; ++j) zero[j] = (__bf16)0.f;
  route_f32x4 acc = route_f32x4{0.f, 0.f, 0.f, 0.f};
  for (int kc = 32 * wave; kc < width; kc += 512) {  // uniform over the wavefront
    route_bf16x8 xb[4], wa[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int k0 = kc + 128 * u + 8 * g;
      const bool ok = k0 < width;  // width is a multiple of 8: a lane's piece is whole or absent
      xb[u] = ok ? *reinterpret_cast<const route_bf16x8*>(xrow + k0) : zero;
      wa[u] = (ok && wrow) ? *reinterpret_cast<const route_bf16x8*>(wrow + k0) : zero;
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa[u], xb[u], acc, 0, 0, 0);
  }
  part[wave][lane] = acc;
  __syncthreads();
  if (wave == 0) {
    const route_f32x4 sum = part[0][lane] + part[1][lane] + part[2][lane] + part[3][lane];
    const int64_t t = t0 + m;  // lane holds rows 16 y + 4 g + i of token t0 + m
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int row = 16 * blockIdx.y + 4 * g + i;
      if (t < tokens && row < rows) logits[t * (experts + 1) + row] = sum[i];
    }
  }
}

// `logits_scratch`: float32 [tokens, experts + 1], used when tokens <= ROUTE_SMALL_TOKENS, and for more tokens when
// activations and weights are bfloat16 (may be null: then one kernel per token computes and selects).
#define ROUTE_SMALL_TOKENS 128
extern "C" int ix_moe_route(const void* x, int dtype, const void* wr, int wr_dtype, const void* shared_gate_w,
                            int sg_dtype, float* topk_w, int32_t* topk_e, float* shared_gate, float* logits_scratch,
                            int64_t tokens, int64_t width, int experts, int k, int renormalize, float scale,
                            int always, hipStream_t stream) {
  IX_REQUIRE(tokens >= 0 && width > 0, "sizes must be positive");
  IX_REQUIRE(always >= 0 && always <= 32 && experts + always <= IX_MAX_EXPERTS,
             "between 0 and 32 experts that every token uses, within the limit of all experts");
  IX_REQUIRE(experts > 0 && experts <= IX_MAX_EXPERTS, "number of experts must be between 1 and 1024");
  IX_REQUIRE(k > 0 && k <= experts && k <= IX_MAX_TOP_K, "top_k must be between 1 and min(experts, 32)");
  IX_REQUIRE(dtype == IX_F32 || dtype == IX_BF16, "dtype must be float32 or bfloat16");
  const size_t smem = (((width + 3) & ~3) + experts + 1) * sizeof(float);
  IX_REQUIRE(smem <= 60 * 1024, "hidden width too large for the router kernel (limit about 15000)");
  if (tokens == 0) return 0;
  if (tokens <= ROUTE_SMALL_TOKENS && logits_scratch != nullptr) {
    const int rows = experts + (shared_gate_w ? 1 : 0);
    dim3 grid(tokens, (rows + ROUTE_THREADS / 64 - 1) / (ROUTE_THREADS / 64)), block(ROUTE_THREADS);
    const size_t xs_bytes = ((width + 3) & ~3) * sizeof(float);
    if (dtype == IX_F32)
      hipLaunchKernelGGL(moe_route_logits_kernel<float>, grid, block, xs_bytes, stream, (const float*)x, wr, wr_dtype,
                         shared_gate_w, sg_dtype, logits_scratch, width, experts);
    else
      hipLaunchKernelGGL(moe_route_logits_kernel<bf16_t>, grid, block, xs_bytes, stream, (const bf16_t*)x, wr,
                         wr_dtype, shared_gate_w, sg_dtype, logits_scratch, width, experts);
    hipLaunchKernelGGL(moe_route_select_kernel, dim3(tokens), dim3(64), experts * sizeof(float), stream,
                       logits_scratch, topk_w, topk_e, shared_gate_w ? shared_gate : nullptr, experts, k, renormalize,
                       scale, always);
    return ix_check_launch("ix_moe_route");
  }
  if (logits_scratch != nullptr && dtype == IX_BF16 && wr_dtype == IX_BF16 &&
      (shared_gate_w == nullptr || sg_dtype == IX_BF16) && width % 8 == 0 && width < (1 << 30) &&
      ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(wr) | reinterpret_cast<uintptr_t>(shared_gate_w)) & 15) == 0) {
    const int row_blocks = (experts + (shared_gate_w ? 1 : 0) + 15) / 16;
    hipLaunchKernelGGL(moe_route_logits_mfma_kernel, dim3(static_cast<unsigned>((tokens + 15) / 16), row_blocks),
                       dim3(256), 0, stream, (const __bf16*)x, (const __bf16*)wr, (const __bf16*)shared_gate_w, logits_scratch,
                       tokens, (int)width, experts);
    hipLaunchKernelGGL(moe_route_select_kernel, dim3(tokens), dim3(64), experts * sizeof(float), stream,
                       logits_scratch, topk_w, topk_e, shared_gate_w ? shared_gate : nullptr, experts, k, renormalize,
                       scale, always);
    return ix_check_launch("ix_moe_route");
  }
  dim3 grid(tokens), block(ROUTE_THREADS);
  if (dtype == IX_F32)
    hipLaunchKernelGGL(moe_route_kernel<float>, grid, block, smem, stream, (const float*)x, wr, wr_dtype,
                       shared_gate_w, sg_dtype, topk_w, topk_e, shared_gate, width, experts, k, renormalize, scale,
                       always);
  else
    hipLaunchKernelGGL(moe_route_kernel<bf16_t>, grid, block, smem, stream, (const bf16_t*)x, wr, wr_dtype,
                       shared_gate_w, sg_dtype, topk_w, topk_e, shared_gate, width, experts, k, renormalize, scale,
                       always);
  return ix_check_launch("ix_moe_route");
}

// ---------------------------------------------------------------------------
// Grouping.  From topk_e[A] (assignment a = token * k + slot) make
//   offsets[E + 1]  rows of expert e are [offsets[e], offsets[e + 1])
//   rows[A]         grouped row -> token
//   dest[A]         assignment  -> grouped row
// stable: within an expert, rows keep assignment order
// (reference: MoeBuildDispatch, moe.cu:452-513; kernels :130-221).
// Also, for the matrix-core product, a map of row tiles: tile i covers rows
// [tile_row0[i], min(tile_row0[i] + tile_rows, end of its expert)) of expert
// tile_expert[i]; tile_info[0] = number of tiles.
// Many assignments: one workgroup of sixteen wavefronts per expert, one launch.  Every workgroup counts the
// assignments of all experts (a sweep over topk_e with integer atomics in LDS: order does not matter), adds up
// the rows and row tiles of the experts before its own, writes its own offset and tiles, and then places its
// own assignments in a second sweep: a wavefront takes 512 consecutive assignments of a pass of 8,192, finds
// its matches by ballot, and their rows follow from the counts of the wavefronts before it.
#define DW_THREADS 1024
#define DW_WAVES (DW_THREADS / 64)
#define DW_ROUNDS 8
__global__ void __launch_bounds__(DW_THREADS)
moe_dispatch_wide_kernel(const int32_t* __restrict__ topk_e, int32_t* __restrict__ offsets,
                         int32_t* __restrict__ rows, int32_t* __restrict__ dest, int64_t assignments, int experts,
                         int k, int tile_rows, int32_t* __restrict__ tile_expert, int32_t* __restrict__ tile_row0,
                         int32_t* __restrict__ tile_info) {
  __shared__ int32_t counts[IX_MAX_EXPERTS];
  __shared__ int32_t wave_count[DW_WAVES];
  __shared__ int32_t part[2][DW_WAVES];
  const int e = blockIdx.x;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  for (int i = tid; i < experts; i += DW_THREADS) counts[i] = 0;
  __syncthreads();
  for (int64_t a = tid; a < assignments; a += DW_THREADS) {
    const int v = topk_e[a];
    if (v >= 0 && v < experts) atomicAdd(&counts[v], 1);
  }
  __syncthreads();
  int rows_before = 0, tiles_before = 0;
  for (int i = tid; i < e; i += DW_THREADS) {
    const int c = counts[i];
    rows_before += c;
    tiles_before += tile_rows > 0 ? (c + tile_rows - 1) / tile_rows : 0;
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    rows_before += __shfl_xor(rows_before, off, 64);
    tiles_before += __shfl_xor(tiles_before, off, 64);
  }
  if (lane == 0) {
    part[0][wave] = rows_before;
    part[1][wave] = tiles_before;
  }
  __syncthreads();
  rows_before = tiles_before = 0;
#pragma unroll
  for (int w = 0; w < DW_WAVES; ++w) {
    rows_before += part[0][w];
    tiles_before += part[1][w];
  }
  const int mine = counts[e];
  const int my_tiles = tile_rows > 0 ? (mine + tile_rows - 1) / tile_rows : 0;
  if (tid == 0) {
    offsets[e] = rows_before;
    if (e == experts - 1) {
      offsets[experts] = rows_before + mine;
      if (tile_info) tile_info[0] = tiles_before + my_tiles;
    }
  }
  if (tile_expert)
    for (int i = tid; i < my_tiles; i += DW_THREADS) {
      tile_expert[tiles_before + i] = e;
      tile_row0[tiles_before + i] = rows_before + i * tile_rows;
    }
  if (mine == 0) return;  // uniform over the workgroup

  const uint64_t below = (uint64_t(1) << lane) - 1;
  int base = rows_before;
  for (int64_t p0 = 0; p0 < assignments; p0 += DW_WAVES * DW_ROUNDS * 64) {
    const int64_t a0 = p0 + static_cast<int64_t>(wave) * DW_ROUNDS * 64 + lane;
    uint64_t match[DW_ROUNDS];
    int found = 0;
#pragma unroll
    for (int r = 0; r < DW_ROUNDS; ++r) {
      const int64_t a = a0 + 64 * r;
      match[r] = __ballot(a < assignments && topk_e[a] == e);
      found += __popcll(match[r]);
    }
    if (lane == 0) wave_count[wave] = found;
    __syncthreads();
    int before = 0, total = 0;
#pragma unroll
    for (int w = 0; w < DW_WAVES; ++w) {
      const int c = wave_count[w];
      before += w < wave ? c : 0;
      total += c;
    }
    int run = base + before;
#pragma unroll
    for (int r = 0; r < DW_ROUNDS; ++r) {
      if ((match[r] >> lane) & 1) {
        const int64_t a = a0 + 64 * r;
        const int32_t row = run + __popcll(match[r] & below);
        rows[row] = static_cast<int32_t>(a / k);
        dest[a] = row;
      }
      run += __popcll(match[r]);
    }
    base += total;
    __syncthreads();
  }
}

// tile_expert / tile_row0 need room for min(A, ceil(A / tile_rows) + E) entries; tile_rows 0 skips the map.
extern "C" int ix_moe_dispatch(const int32_t* topk_e, int32_t* offsets, int32_t* rows, int32_t* dest,
                               int64_t assignments, int experts, int k, int tile_rows, int32_t* tile_expert,
                               int32_t* tile_row0, int32_t* tile_info, hipStream_t stream) {
  IX_REQUIRE(assignments >= 0 && k > 0, "sizes must be positive");
  IX_REQUIRE(experts > 0 && experts <= IX_MAX_EXPERTS, "number of experts must be between 1 and 1024");
  IX_REQUIRE(tile_rows >= 0, "tile_rows must not be negative");
  IX_REQUIRE(tile_rows == 0 || (tile_expert && tile_row0 && tile_info), "tile map buffers needed");
  hipLaunchKernelGGL(moe_dispatch_wide_kernel, dim3(experts), dim3(DW_THREADS), 0, stream, topk_e, offsets, rows, dest,
                     assignments, experts, k, tile_rows, tile_expert, tile_row0, tile_info);
  return ix_check_launch("ix_moe_dispatch");
}

// ---------------------------------------------------------------------------
// Plain grouped product over device-resident offsets.
//   GATE_UP: out[r, n] = silu(x[src(r)] . W[e][n]) * (x[src(r)] . W[e][inner + n]),  n < inner
//            with src(r) = rows[r] (the gather is fused), W [E, 2*inner, width]
//   else:    out[r, n] = a[r] . W[e][n],  W [E, n_out, width]
// (reference: GroupedGemmBf16Kernel, moe.cu:323-392; SwiGLU moe_ffn.cc:288-291).
// 64 x 64 output tile per workgroup, 4 x 4 per thread, float32 accumulation.
// Tile index -> expert: experts are walked in order, each owning ceil(count/64) tiles.
#define GG_BM 64
#define GG_BN 64
#define GG_BK 16

template <typename TA, typename TW, typename TO, bool GATE_UP>
__global__ void __launch_bounds__(256)
moe_grouped_plain_kernel(const TA* __restrict__ a, const TW* __restrict__ w, TO* __restrict__ out,
                         const int32_t* __restrict__ offsets, const int32_t* __restrict__ rows, int experts,
                         int64_t n_out, int64_t width) {
  __shared__ float As[GG_BK][GG_BM + 4];
  __shared__ float Ws[GATE_UP ? 2 : 1][GG_BK][GG_BN + 4];
  __shared__ int32_t src_row[GG_BM];

  // which expert owns m-tile blockIdx.y
  int tile = blockIdx.y, e = 0, row0 = 0, row_end = 0;
  for (; e < experts; ++e) {
    const int begin = offsets[e], end = offsets[e + 1];
    const int tiles = (end - begin + GG_BM - 1) / GG_BM;
    if (tile < tiles) {
      row0 = begin + tile * GG_BM;
      row_end = end;
      break;
    }
    tile -= tiles;
  }
  if (e == experts) return;

  const int tid = threadIdx.x;
  const int64_t n0 = static_cast<int64_t>(blockIdx.x) * GG_BN;
  const int64_t w_rows = GATE_UP ? 2 * n_out : n_out;
  const TW* we = w + static_cast<int64_t>(e) * w_rows * width;
  if (tid < GG_BM) {
    const int r = row0 + tid;
    src_row[tid] = r < row_end ? (rows ? rows[r] : r) : -1;
  }
  __syncthreads();

  const int tx = tid & 15, ty = tid >> 4;  // thread owns rows ty*4.., cols tx*4..
  float acc[GATE_UP ? 2 : 1][4][4] = {};
  for (int64_t k0 = 0; k0 < width; k0 += GG_BK) {
    // stage A: 64 rows x 16 k, W: 64 cols x 16 k (x2 with the gate)
    for (int i = tid; i < GG_BM * GG_BK; i += 256) {
      const int r = i / GG_BK, kk = i % GG_BK;
      const int sr = src_row[r];
      const int64_t kc = k0 + kk;
      As[kk][r] = (sr >= 0 && kc < width) ? ix_load(a + static_cast<int64_t>(sr) * width + kc) : 0.f;
    }
    for (int i = tid; i < GG_BN * GG_BK; i += 256) {
      const int c = i / GG_BK, kk = i % GG_BK;
      const int64_t n = n0 + c, kc = k0 + kk;
      const bool ok = n < n_out && kc < width;
      Ws[0][kk][c] = ok ? ix_load(we + n * width + kc) : 0.f;
      if (GATE_UP) Ws[1][kk][c] = ok ? ix_load(we + (n_out + n) * width + kc) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < GG_BK; ++kk) {
      float av[4], wv[GATE_UP ? 2 : 1][4];
#pragma unroll
      for (int i = 0; i < 4; ++i) av[i] = As[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        wv[0][j] = Ws[0][kk][tx * 4 + j];
        if (GATE_UP) wv[1][j] = Ws[1][kk][tx * 4 + j];
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          acc[0][i][j] += av[i] * wv[0][j];
          if (GATE_UP) acc[1][i][j] += av[i] * wv[1][j];
        }
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = row0 + ty * 4 + i;
    if (r >= row_end) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int64_t n = n0 + tx * 4 + j;
      if (n >= n_out) continue;
      float v = acc[0][i][j];
      if (GATE_UP) v = v / (1.0f + expf(-v)) * acc[1][i][j];
      ix_store(out + static_cast<int64_t>(r) * n_out + n, v);
    }
  }
}

template <bool GATE_UP>
static int launch_grouped_plain(const void* a, int a_dtype, const void* w, int w_dtype, void* out,
                                const int32_t* offsets, const int32_t* rows, int64_t assignments, int experts,
                                int64_t n_out, int64_t width, hipStream_t stream) {
  const int64_t m_tiles = std::min<int64_t>(assignments, (assignments + GG_BM - 1) / GG_BM + experts);
  dim3 grid((n_out + GG_BN - 1) / GG_BN, m_tiles), block(256);
#define LAUNCH(TA, TW)                                                                                            \
  hipLaunchKernelGGL((moe_grouped_plain_kernel<TA, TW, TA, GATE_UP>), grid, block, 0, stream, (const TA*)a,        \
                     (const TW*)w, (TA*)out, offsets, rows, experts, n_out, width)
  if (a_dtype == IX_F32 && w_dtype == IX_F32) LAUNCH(float, float);
  else if (a_dtype == IX_F32 && w_dtype == IX_BF16) LAUNCH(float, bf16_t);
  else if (a_dtype == IX_BF16 && w_dtype == IX_F32) LAUNCH(bf16_t, float);
  else if (a_dtype == IX_BF16 && w_dtype == IX_BF16) LAUNCH(bf16_t, bf16_t);
  else { ix_set_error("grouped product: dtypes must be float32 or bfloat16"); return 1; }
#undef LAUNCH
  return ix_check_launch("ix_moe_grouped_plain");
}

extern "C" int ix_moe_grouped_plain(const void* a, int a_dtype, const void* w, int w_dtype, void* out,
                                    const int32_t* offsets, const int32_t* rows, int64_t assignments, int experts,
                                    int64_t n_out, int64_t width, int gate_up, hipStream_t stream) {
  IX_REQUIRE(assignments >= 0 && n_out > 0 && width > 0 && experts > 0, "sizes must be positive");
  IX_REQUIRE(assignments < (1ll << 31) / GG_BM, "too many assignments");
  if (assignments == 0) return 0;
  return gate_up ? launch_grouped_plain<true>(a, a_dtype, w, w_dtype, out, offsets, rows, assignments, experts, n_out,
                                              width, stream)
                 : launch_grouped_plain<false>(a, a_dtype, w, w_dtype, out, offsets, rows, assignments, experts,
                                               n_out, width, stream);
}

// ---------------------------------------------------------------------------
// out[t, :] = sum over slots, in slot order, of topk_w[t, s] * y[dest[t*k + s], :]
//             (+ shared_gate[t] * shared[t, :], or + shared[t, :] without a gate)
// (reference: CombineRowsKernel moe.cu:237-255, AddSharedExpertKernel :275-287)
template <typename T>
__global__ void moe_combine_kernel(const T* __restrict__ y, const int32_t* __restrict__ dest,
                                   const float* __restrict__ topk_w, const T* __restrict__ shared,
                                   const float* __restrict__ shared_gate, T* __restrict__ out, int64_t width, int k) {
  const int64_t t = blockIdx.x;
  const float sg = shared ? (shared_gate ? shared_gate[t] : 1.0f) : 0.f;
  for (int64_t c = threadIdx.x; c < width; c += blockDim.x) {
    float acc = 0.f;
    for (int s = 0; s < k; ++s) {
      const int64_t a = t * k + s;
      acc += topk_w[a] * ix_load(y + static_cast<int64_t>(dest[a]) * width + c);
    }
    if (shared) acc += sg * ix_load(shared + t * width + c);
    ix_store(out + t * width + c, acc);
  }
}

extern "C" int ix_moe_combine(const void* y, int dtype, const int32_t* dest, const float* topk_w, const void* shared,
                              const float* shared_gate, void* out, int64_t tokens, int64_t width, int k,
                              hipStream_t stream) {
  IX_REQUIRE(tokens >= 0 && width > 0 && k > 0, "sizes must be positive");
  if (tokens == 0) return 0;
  dim3 grid(tokens), block(256);
  if (dtype == IX_F32)
    hipLaunchKernelGGL(moe_combine_kernel<float>, grid, block, 0, stream, (const float*)y, dest, topk_w,
                       (const float*)shared, shared_gate, (float*)out, width, k);
  else if (dtype == IX_BF16)
    hipLaunchKernelGGL(moe_combine_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)y, dest, topk_w,
                       (const bf16_t*)shared, shared_gate, (bf16_t*)out, width, k);
  else
    IX_REQUIRE(false, "dtype must be float32 or bfloat16");
  return ix_check_launch("ix_moe_combine");
}
