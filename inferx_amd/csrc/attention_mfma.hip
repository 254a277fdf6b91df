// Paged attention on the matrix cores (bfloat16), for prompt portions and for
// decoding alike.  Same arithmetic as the plain kernel (attention_plain.hip):
// keys [start, p] through the block table, scores * scale, softmax online in
// float32, PV accumulated in float32.
//
// Unit of work = one wavefront: a tile of up to 16 consecutive queries of one
// request and one query head, over one slice of that tile's keys (split-KV).
// There is no LDS and no barrier: a workgroup is four independent wavefronts.
//
// The transposed products are formed so that no operand has to be shuffled:
//   S^T[key][query]  = K[key][:] . Q[query][:]     (A = K rows, B = Q rows)
//   O^T[d][query]   += V^T[d][key] * P^T[key][query]  (A = V^T rows, B = P^T)
// v_mfma_f32_16x16x32_bf16 gives lane l of the result rows 4*(l/16)+i, column
// l%16.  Row m of the first key block of an iteration is key 8*(m/4) + m%4 and
// of the second key 8*(m/4) + 4 + m%4, so a lane ends up with the scores of
// eight consecutive keys (8*(l/16) .. +7) of its query: exactly the B operand
// of the second product, while V^T (values are stored [d][offset] within a
// page) supplies eight consecutive keys of one column as 16 contiguous bytes.
//
// With more than one split, each wavefront writes (max, sum, unnormalised O)
// and `attn_combine_kernel` merges them.
//
// GQ (grouped queries, for tiles of ONE token): the sixteen columns of a tile are
// the query heads that share a key/value head instead of consecutive tokens of
// one head, and a wavefront serves a (token, key/value head) pair.  Keys and
// values are then read once per key/value head, not once per query head.
#include "common.h"
#include "inferx_hip.h"

#include <mutex>

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

#define ATTN_KEYS_PER_ITER 32

// head_dim = 16 * NB; a tile holds up to 16 * QT queries; PF: request the next iteration's keys and values
// before this iteration's are multiplied (pays when few wavefronts are resident: decoding)
template <int NB, int QT, bool PF, bool GQ = false>
__global__ void __launch_bounds__(256)
attn_mfma_kernel(const __bf16* __restrict__ q, const __bf16* __restrict__ k_cache, const __bf16* __restrict__ v_cache,
                 const int32_t* __restrict__ block_table, const int32_t* __restrict__ tile_seq,
                 const int32_t* __restrict__ tile_q0, const int32_t* __restrict__ tile_rows,
                 const int32_t* __restrict__ positions, __bf16* __restrict__ out, float* __restrict__ part_o,
                 float* __restrict__ part_ml, int n_tiles, int n_splits, int heads, int kv_heads, int page_size,
                 int max_blocks, float scale_log2, int window, int page_shift) {
  constexpr int D = 16 * NB;
  constexpr int NC = (NB + 1) / 2;  // 32-wide chunks of the head dimension
  const int lane = threadIdx.x & 63;
  // (wavefronts of a workgroup share nothing: a workgroup is four of them, or fewer where a step has so few that
  // whole compute units would stay idle otherwise)
  const int unit = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (unit >= n_tiles * n_splits) return;
  const int tile = unit / n_splits, split = unit - tile * n_splits;
  const int group = heads / kv_heads;
  // GQ: blockIdx.y is the key/value head, column n of the tile is query head kvh * group + n of token tq0
  const int kvh = GQ ? blockIdx.y : blockIdx.y / group;
  const int n = lane & 15, g = lane >> 4;
  const int head = GQ ? kvh * group + min(n, group - 1) : blockIdx.y;

  const int tq0 = tile_q0[tile];
  const int rows = GQ ? group : tile_rows[tile];  // columns of the tile that hold a query
  const int pos0 = positions[tq0];
  const int32_t* table = block_table + static_cast<int64_t>(tile_seq[tile]) * max_blocks;

  // keys this tile reads at all: [lo, hi); this wavefront's slice [ks, ke)
  const int lo = (window > 0 && pos0 + 1 > window) ? pos0 + 1 - window : 0;
  const int hi = pos0 + (GQ ? 1 : rows);
  const int lo_al = lo & ~(ATTN_KEYS_PER_ITER - 1);
  const int per = (((hi - lo_al + n_splits - 1) / n_splits) + ATTN_KEYS_PER_ITER - 1) & ~(ATTN_KEYS_PER_ITER - 1);
  const int ks = lo_al + split * per;
  const int ke = min(hi, ks + per);

  // Q as B operand: lane (n, g) holds Q[query 16 t + n][32 c + 8 g .. +8]
  bf16x8 qf[QT][NC];
#pragma unroll
  for (int t = 0; t < QT; ++t)
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      const int d0 = 32 * c + 8 * g;
      if (16 * t + n < rows && d0 < D)
        qf[t][c] =
            *reinterpret_cast<const bf16x8*>(q + (static_cast<int64_t>(tq0 + (GQ ? 0 : 16 * t + n)) * heads + head) * D + d0);
      else
        for (int j = 0; j < 8; ++j) qf[t][c][j] = (__bf16)0.f;
    }

  f32x4 o[QT][NB];
  float m[QT], lsum[QT];
#pragma unroll
  for (int t = 0; t < QT; ++t) {
    m[t] = -INFINITY;
    lsum[t] = 0.f;
#pragma unroll
    for (int b = 0; b < NB; ++b) o[t][b] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  // K fragments for the 32 keys from kb on (two blocks of 16 rows) and V^T fragments
  // (lane (dd = n, g) holds V^T[16 blk + dd][kb + 8 g .. +8])
  // a page size that is a power of two (page_shift >= 0, the usual case) spares the divisions
  auto page_of = [&](int key) { return page_shift >= 0 ? key >> page_shift : key / page_size; };
  // The pages of the 32 keys from kb on, as this lane needs them: for its row of the two key blocks and for its
  // eight values.  They are looked up one iteration before the keys and values themselves are asked for, so that
  // no load in the loop has to wait for another one's result.
  auto ask_pages = [&](int kb, int (&pg)[3]) {
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      const int key = min(kb + 8 * (n >> 2) + 4 * b + (n & 3), hi - 1);  // A row n of block b
      pg[b] = table[page_of(key)];
    }
    pg[2] = table[page_of(min(kb + 8 * g, hi - 1) & ~7)];
  };
  auto load_kv = [&](int kb, const int (&pg)[3], bf16x8 (&kf)[2][NC], bf16x8 (&vf)[NB]) {
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      int key = kb + 8 * (n >> 2) + 4 * b + (n & 3);
      key = min(key, hi - 1);                          // rows past the end are masked below
      const int pi = page_of(key);
      const int page = max(pg[b], 0);                  // a page the window has passed: masked below
      const __bf16* kr =
          k_cache + ((static_cast<int64_t>(page) * kv_heads + kvh) * page_size + (key - pi * page_size)) * D;
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        const int d0 = 32 * c + 8 * g;
        if (d0 < D)
          kf[b][c] = *reinterpret_cast<const bf16x8*>(kr + d0);
        else
          for (int j = 0; j < 8; ++j) kf[b][c][j] = (__bf16)0.f;
      }
    }
    const int key = min(kb + 8 * g, hi - 1) & ~7;
    const int pi = page_of(key);
    const int page = max(pg[2], 0);
    const __bf16* vr = v_cache + (static_cast<int64_t>(page) * kv_heads + kvh) * D * page_size + (key - pi * page_size);
#pragma unroll
    for (int b = 0; b < NB; ++b)
      vf[b] = *reinterpret_cast<const bf16x8*>(vr + static_cast<int64_t>(16 * b + n) * page_size);
  };

  bf16x8 kf_next[PF ? 2 : 1][PF ? NC : 1], vf_next[PF ? NB : 1];
  int pg[3], pg_next[3];
  if (ks < ke) {
    ask_pages(ks, pg);
    if constexpr (PF) {
      ask_pages(ks + ATTN_KEYS_PER_ITER, pg_next);
      load_kv(ks, pg, kf_next, vf_next);
    }
  }
  for (int kb = ks; kb < ke; kb += ATTN_KEYS_PER_ITER) {
    bf16x8 kf[2][NC], vf[NB];
    if constexpr (PF) {
#pragma unroll
      for (int b = 0; b < 2; ++b)
#pragma unroll
        for (int c = 0; c < NC; ++c) kf[b][c] = kf_next[b][c];
#pragma unroll
      for (int b = 0; b < NB; ++b) vf[b] = vf_next[b];
      if (kb + ATTN_KEYS_PER_ITER < ke) {
        load_kv(kb + ATTN_KEYS_PER_ITER, pg_next, kf_next, vf_next);
        ask_pages(kb + 2 * ATTN_KEYS_PER_ITER, pg_next);
      }
    } else {
      ask_pages(kb + ATTN_KEYS_PER_ITER, pg_next);
      load_kv(kb, pg, kf, vf);
#pragma unroll
      for (int i = 0; i < 3; ++i) pg[i] = pg_next[i];
    }
    // Values of keys that no query of the tile may read (past the tile's last key in the same page, or on a page
    // that the window has passed, read from wherever the table's filler points) are made zero: their probability
    // is zero, but zero times whatever an earlier request left there need not be.  Only rounds at the edges.
    if (kb + ATTN_KEYS_PER_ITER > hi || kb < lo) {
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int key = (min(kb + 8 * g, hi - 1) & ~7) + j;
        if (key >= hi || key < lo) {
#pragma unroll
          for (int b = 0; b < NB; ++b) vf[b][j] = (__bf16)0.f;
        }
      }
    }
#pragma unroll
    for (int t = 0; t < QT; ++t) {
      if (QT > 1 && (16 * t >= rows || kb > pos0 + 16 * t + 15)) continue;  // no query of this block reads these keys
      // ---- S^T = K Q^T ----
      f32x4 s[2];
#pragma unroll
      for (int b = 0; b < 2; ++b) {
        s[b] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int c = 0; c < NC; ++c) s[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[b][c], qf[t][c], s[b], 0, 0, 0);
      }
      // ---- mask, online softmax for this lane's query over its 8 keys ----
      const int my_pos = pos0 + (GQ ? 0 : 16 * t + n);
      const bool my_row = 16 * t + n < rows;
      const int my_lo = (window > 0 && my_pos + 1 > window) ? my_pos + 1 - window : 0;
      // scores stay unscaled: the scale (times log2 e) enters with the reference point in one fused multiply-add
      float sv[8];
      float mx = -INFINITY;
      // keys that every query of these sixteen sees need no mask (uniform over the wavefront)
      // (GQ: the columns without a query head hold zeros for q; what they sum is not stored)
      const bool inner = (GQ || 16 * t + 16 <= rows) && kb + ATTN_KEYS_PER_ITER <= ke &&
                         kb + ATTN_KEYS_PER_ITER - 1 <= pos0 + (GQ ? 0 : 16 * t) &&
                         (window == 0 || kb > pos0 + (GQ ? 0 : 16 * t + 15) - window);
      if (inner) {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          sv[j] = s[j >> 2][j & 3];
          mx = fmaxf(mx, sv[j]);
        }
      } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int key = kb + 8 * g + j;
          const bool ok = my_row && key >= my_lo && key <= my_pos && key < ke;
          sv[j] = ok ? s[j >> 2][j & 3] : -INFINITY;
          mx = fmaxf(mx, sv[j]);
        }
      }
      mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
      // The reference point m of the exponentials (in units of log2) follows the running maximum lazily: it moves
      // only when some query's maximum has outgrown it by more than 2^8, so the accumulators are seldom rescaled.
      // Any m gives the same quotient; probabilities up to 2^8 keep the relative precision of bfloat16.
      const float top = mx * scale_log2;
      if (__any(top > m[t] + 8.f)) {
        const float m_new = fmaxf(m[t], top);
        // v_exp_f32 as it is: a result below the smallest normal number may become 0
        const float alpha = __builtin_amdgcn_exp2f(m[t] - ((m_new == -INFINITY) ? 0.f : m_new));
        lsum[t] *= alpha;
#pragma unroll
        for (int b = 0; b < NB; ++b) o[t][b] *= alpha;
        m[t] = m_new;
      }
      const float m_safe = (m[t] == -INFINITY) ? 0.f : m[t];
      float psum = 0.f;
      bf16x8 pf;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float p = __builtin_amdgcn_exp2f(fmaf(sv[j], scale_log2, -m_safe));
        psum += p;
        pf[j] = (__bf16)p;
      }
      lsum[t] += psum;
      // ---- O^T += V^T P^T ----
#pragma unroll
      for (int b = 0; b < NB; ++b) o[t][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[b], pf, o[t][b], 0, 0, 0);
    }
  }

#pragma unroll
  for (int t = 0; t < QT; ++t) {
    float l = lsum[t];
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);
    if (16 * t + n >= rows) continue;
    // lane holds O^T rows d = 16 b + 4 g + i of column n
    const int64_t token = tq0 + (GQ ? 0 : 16 * t + n);
    if (n_splits == 1) {
      const float inv = 1.0f / l;
      __bf16* dst = out + (token * heads + head) * D + 4 * g;
#pragma unroll
      for (int b = 0; b < NB; ++b) {
        bf16x4 v;
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = (__bf16)(o[t][b][i] * inv);
        *reinterpret_cast<bf16x4*>(dst + 16 * b) = v;
      }
    } else {
      const int64_t p = (token * heads + head) * n_splits + split;
      float* dst = part_o + p * D + 4 * g;
#pragma unroll
      for (int b = 0; b < NB; ++b) *reinterpret_cast<f32x4*>(dst + 16 * b) = o[t][b];
      if (g == 0) {
        part_ml[2 * p] = m[t];
        part_ml[2 * p + 1] = l;
      }
    }
  }
}

// out[t, h, :] = sum_s o_s 2^(m_s - M) / sum_s l_s 2^(m_s - M),  M = max_s m_s
// One workgroup per (token, head); the slices' weights are worked out once, then every thread
// sums its columns with independent loads.
__global__ void __launch_bounds__(128)
attn_combine_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml, __bf16* __restrict__ out,
                    int n_splits, int head_dim) {
  __shared__ float wgt[256];
  __shared__ float inv_l;
  const int64_t th = blockIdx.x;  // token * heads + head
  const float* ml = part_ml + th * n_splits * 2;
  if (threadIdx.x < 64) {
    float mloc = -INFINITY;
    for (int s = threadIdx.x; s < n_splits; s += 64) mloc = fmaxf(mloc, ml[2 * s]);
    const float M = ix_wave_max(mloc);
    float lloc = 0.f;
    for (int s = threadIdx.x; s < n_splits; s += 64) {
      const float m_s = ml[2 * s];
      const float w = (m_s == -INFINITY) ? 0.f : exp2f(m_s - M);
      wgt[s] = w;
      lloc += w * ml[2 * s + 1];
    }
    const float L = ix_wave_sum(lloc);
    if (threadIdx.x == 0) inv_l = 1.0f / L;
  }
  __syncthreads();
  const float* po = part_o + th * n_splits * head_dim;
  for (int d = threadIdx.x; d < head_dim; d += blockDim.x) {
    float acc = 0.f;
#pragma unroll 8
    for (int s = 0; s < n_splits; ++s) acc += wgt[s] * po[s * head_dim + d];
    out[th * head_dim + d] = (__bf16)(acc * inv_l);
  }
}

int ix_attention_combine(const float* part_o, const float* part_ml, void* out, int64_t tokens, int heads,
                         int n_splits, int head_dim, hipStream_t stream) {
  hipLaunchKernelGGL(attn_combine_kernel, dim3(static_cast<unsigned>(tokens * heads)), dim3(128), 0, stream, part_o,
                     part_ml, (__bf16*)out, n_splits, head_dim);
  return ix_check_launch("ix_attention_combine");
}

template <int NB, int QT, bool PF, bool GQ = false>
static void launch_attn(dim3 grid, hipStream_t stream, const void* q, const void* k, const void* v,
                        const int32_t* table, const int32_t* tile_seq, const int32_t* tile_q0,
                        const int32_t* tile_rows, const int32_t* positions, void* out, float* part_o, float* part_ml,
                        int n_tiles, int n_splits, int heads, int kv_heads, int page_size, int max_blocks,
                        float scale_log2, int window) {
  int page_shift = -1;  // log2 of the page size if it is a power of two
  for (int b = 4; b < 31; ++b)
    if (page_size == (1 << b)) page_shift = b;
  // four wavefronts per workgroup (grid.x counts such workgroups), two or one while that makes fewer than two
  // workgroups per compute unit of the 256 (one request of 16 heads with its keys in 32 slices: 512 wavefronts)
  const int64_t waves = static_cast<int64_t>(n_tiles) * n_splits * grid.y;
  const int per_group = waves >= 4 * 512 ? 4 : (waves >= 2 * 512 ? 2 : 1);
  grid.x = static_cast<unsigned>((static_cast<int64_t>(n_tiles) * n_splits + per_group - 1) / per_group);
  hipLaunchKernelGGL((attn_mfma_kernel<NB, QT, PF, GQ>), grid, dim3(64 * per_group), 0, stream, (const __bf16*)q, (const __bf16*)k,
                     (const __bf16*)v, table, tile_seq, tile_q0, tile_rows, positions, (__bf16*)out, part_o, part_ml,
                     n_tiles, n_splits, heads, kv_heads, page_size, max_blocks, scale_log2, window, page_shift);
}

// Workspace (when n_splits > 1): part_o float32 [tokens * heads * n_splits * head_dim],
// part_ml float32 [tokens * heads * n_splits * 2].
// grouped: every tile is ONE token (tile_rows is not read), and a wavefront serves the query heads of one key/value
// head together (at most 16 of them; tile_queries 16).
extern "C" int ix_attention_mfma(const void* q, const void* k_cache, const void* v_cache, const int32_t* block_table,
                                 const int32_t* tile_seq, const int32_t* tile_q0, const int32_t* tile_rows,
                                 const int32_t* positions, void* out, float* part_o, float* part_ml, int64_t tokens,
                                 int n_tiles, int tile_queries, int n_splits, int heads, int kv_heads, int head_dim,
                                 int page_size, int max_blocks, float scale, int window, int prefetch, int grouped,
                                 hipStream_t stream) {
  IX_REQUIRE(tile_queries == 16 || tile_queries == 32, "a query tile holds up to 16 or 32 queries");
  IX_REQUIRE(tile_queries == 16 || head_dim <= 128, "tiles of 32 queries need head_dim <= 128");
  IX_REQUIRE(tokens >= 0 && n_tiles >= 0 && heads > 0 && kv_heads > 0 && max_blocks > 0, "sizes must be positive");
  IX_REQUIRE(heads % kv_heads == 0, "heads must be a multiple of kv_heads");
  IX_REQUIRE(head_dim % 16 == 0 && head_dim >= 16 && head_dim <= 256, "head_dim must be a multiple of 16 up to 256");
  IX_REQUIRE(page_size % 16 == 0 && page_size > 0, "page_size must be a multiple of 16");
  IX_REQUIRE(n_splits >= 1 && n_splits <= 256, "n_splits must be between 1 and 256");
  IX_REQUIRE(n_splits == 1 || (part_o != nullptr && part_ml != nullptr), "workspace needed for split keys");
  IX_REQUIRE(window >= 0, "window must not be negative");
  IX_REQUIRE(heads <= 65535, "too many heads");
  IX_REQUIRE(!grouped || (tile_queries == 16 && heads / kv_heads <= 16),
             "grouped queries: tiles of 16, at most 16 query heads per key/value head");
  if (n_tiles == 0 || tokens == 0) return 0;
  const int64_t units = static_cast<int64_t>(n_tiles) * n_splits;
  dim3 grid(static_cast<unsigned>((units + 3) / 4), grouped ? kv_heads : heads);
  const float scale_log2 = scale * 1.4426950408889634f;
#define ARGS                                                                                                    \
  grid, stream, q, k_cache, v_cache, block_table, tile_seq, tile_q0, tile_rows, positions, out, part_o, part_ml, \
      n_tiles, n_splits, heads, kv_heads, page_size, max_blocks, scale_log2, window
#define CASE(NB)                                                    \
  case NB:                                                          \
    if (grouped) {                                                  \
      if (prefetch) launch_attn<NB, 1, true, true>(ARGS);           \
      else launch_attn<NB, 1, false, true>(ARGS);                   \
    } else if (prefetch) launch_attn<NB, 1, true>(ARGS);            \
    else launch_attn<NB, 1, false>(ARGS);                           \
    break;
#define CASE4(NB)                        \
  case NB:                               \
    launch_attn<NB, 2, false>(ARGS);     \
    break;
  if (tile_queries == 16) {
    switch (head_dim / 16) {
      CASE(1) CASE(2) CASE(3) CASE(4) CASE(5) CASE(6) CASE(7) CASE(8)
      CASE(9) CASE(10) CASE(11) CASE(12) CASE(13) CASE(14) CASE(15) CASE(16)
    }
  } else {
    switch (head_dim / 16) {
      CASE4(1) CASE4(2) CASE4(3) CASE4(4) CASE4(5) CASE4(6) CASE4(7) CASE4(8)
    }
  }
#undef CASE
#undef CASE4
#undef ARGS
  if (ix_check_launch("ix_attention_mfma")) return 1;
  if (n_splits > 1) return ix_attention_combine(part_o, part_ml, out, tokens, heads, n_splits, head_dim, stream);
  return 0;
}

// ---- the same operation without a workspace argument -----------------------------------------------------------
// The slices' parts go to an array that is part of the library's image on every device.  In host code the
// array's name stands for the symbol, not for device memory: its address on the current device is looked up
// once per device and only that pointer is handed to kernels.
static __device__ __align__(256) float scratch[IX_ATTENTION_SCRATCH_BYTES / sizeof(float)];

#define IX_MAX_DEVICES 64
static float* g_scratch_of_device[IX_MAX_DEVICES];  // null until the device's first call
static std::mutex g_scratch_mutex;

// the current device's copy of `scratch`; 0 on success
static int scratch_of_current_device(float** ptr) {
  int device = -1;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) {
    ix_set_error(std::string("ix_attention_mfma_noalloc: hipGetDevice: ") + hipGetErrorString(e));
    return 1;
  }
  if (device < 0 || device >= IX_MAX_DEVICES) {
    ix_set_error("ix_attention_mfma_noalloc: device index " + std::to_string(device) + " is beyond " +
                 std::to_string(IX_MAX_DEVICES));
    return 1;
  }
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_of_device[device] == nullptr) {
    float* found = nullptr;
    e = hipGetSymbolAddress(reinterpret_cast<void**>(&found), HIP_SYMBOL(scratch));
    if (e != hipSuccess || found == nullptr) {
      ix_set_error(std::string("ix_attention_mfma_noalloc: hipGetSymbolAddress: ") + hipGetErrorString(e));
      return 1;
    }
    g_scratch_of_device[device] = found;
  }
  *ptr = g_scratch_of_device[device];
  return 0;
}

extern "C" int ix_attention_mfma_noalloc(const void* q, const void* k_cache, const void* v_cache,
                                         const int32_t* block_table, const int32_t* tile_seq, const int32_t* tile_q0,
                                         const int32_t* tile_rows, const int32_t* positions, void* out, int64_t tokens,
                                         int n_tiles, int tile_queries, int n_splits, int heads, int kv_heads,
                                         int head_dim, int page_size, int max_blocks, float scale, int window,
                                         int prefetch, int grouped, hipStream_t stream) {
  IX_REQUIRE(tokens >= 0 && heads > 0 && head_dim > 0 && n_splits >= 1 && n_splits <= 256, "sizes must be positive");
  float* part_o = nullptr;
  float* part_ml = nullptr;
  if (n_splits > 1) {
    const int64_t capacity = IX_ATTENTION_SCRATCH_BYTES / sizeof(float);
    IX_REQUIRE(tokens <= capacity && heads <= capacity, "sizes beyond the library's buffer");
    const int64_t parts = tokens * heads * n_splits;  // at most 2^22 * 2^22 * 2^8: no overflow
    if (parts > capacity || parts * (head_dim + 2) > capacity) {
      ix_set_error("ix_attention_mfma_noalloc: tokens * heads * n_splits * (head_dim + 2) = " +
                   std::to_string(parts) + " * " + std::to_string(head_dim + 2) + " floats do not fit the library's " +
                   std::to_string(IX_ATTENTION_SCRATCH_BYTES) + " bytes: fewer slices or tokens per call, or " +
                   "ix_attention_mfma with a workspace of the caller's");
      return 1;
    }
    float* base = nullptr;
    if (scratch_of_current_device(&base)) return 1;
    part_o = base;
    part_ml = base + parts * head_dim;
  }
  return ix_attention_mfma(q, k_cache, v_cache, block_table, tile_seq, tile_q0, tile_rows, positions, out, part_o,
                           part_ml, tokens, n_tiles, tile_queries, n_splits, heads, kv_heads, head_dim, page_size,
                           max_blocks, scale, window, prefetch, grouped, stream);
}
