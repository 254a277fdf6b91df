// Paged attention for prompt portions (bfloat16): the four wavefronts of a
// workgroup share each tile of keys and values through LDS.
//
// A workgroup owns up to 64 consecutive queries of one request and one query
// head (wavefront w: queries 16 w ..), and walks that tile's keys [lo, hi) 64
// at a time.  Keys are staged as [64][128] rows whose 16-byte pieces are
// permuted, values as [D][64 + 8] (they are stored transposed within a page),
// so that the sixteen 16-byte operand reads of a quarter wavefront fall on
// distinct banks.  Tiles are double-buffered: a tile's global loads are issued
// two rounds ahead into registers and written to LDS one round ahead.
// Arithmetic, masking and the operand mapping are those of the wavefront-level
// kernel in attention_mfma.hip (S^T = K Q^T, O^T += V^T P^T with
// v_mfma_f32_16x16x32_bf16, a lane ending up with eight consecutive keys of one
// query), which remains the kernel for decoding and for small steps.
//
// QT is the number of sixteens of queries per wavefront.  Only 1 is launched:
// 2 halves the LDS reads per product but leaves one wavefront per SIMD, and
// measured slower on MI355X.
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

#define PF_KEYS 64

template <int NB, int QT>  // head_dim = 16 * NB
__global__ void __launch_bounds__(256)
attn_prefill_kernel(const __bf16* __restrict__ q, const __bf16* __restrict__ k_cache,
                    const __bf16* __restrict__ v_cache, const int32_t* __restrict__ block_table,
                    const int32_t* __restrict__ tile_seq, const int32_t* __restrict__ tile_q0,
                    const int32_t* __restrict__ tile_rows, const int32_t* __restrict__ pair_a,
                    const int32_t* __restrict__ pair_b, const int32_t* __restrict__ positions,
                    __bf16* __restrict__ out, float* __restrict__ part_o, float* __restrict__ part_ml, int n_splits,
                    int heads, int kv_heads, int page_size, int max_blocks, float scale_log2,
                    int window, int page_shift) {
  constexpr int D = 16 * NB;
  constexpr int NC = (NB + 1) / 2;          // 32-wide chunks of the head dimension
  constexpr int KS = 128;                   // elements per LDS row of the key tile: sixteen 16-byte pieces,
                                            // piece p of row r kept at place p ^ swz(r) (see key_place)
  constexpr int VS = PF_KEYS;               // elements per LDS row of the value tile: eight 16-byte pieces,
                                            // piece p of row r kept at place p ^ ((r >> 1) & 7)
  constexpr int K_CHUNKS = PF_KEYS * 2 * NB;  // 16-byte pieces of a key tile
  constexpr int V_CHUNKS = D * (PF_KEYS / 8);
  constexpr int K_PER = (K_CHUNKS + 255) / 256, V_PER = (V_CHUNKS + 255) / 256;
  __shared__ __attribute__((aligned(16))) __bf16 k_tiles[2][PF_KEYS * KS];  // one tile is read while the next is written
  __shared__ __attribute__((aligned(16))) __bf16 v_tiles[2][D * VS];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n = lane & 15, g = lane >> 4;
  // A workgroup takes two tiles, one after the other: the host pairs a tile that reads many keys with one that
  // reads few, so that workgroups take about equally long whichever compute unit they land on.
#pragma unroll 1
  for (int which = 0; which < 2; ++which) {
  // a unit of work is a tile, or (n_splits > 1) one slice of a tile's keys: unit = tile * n_splits + slice
  const int unit = which ? pair_b[blockIdx.x] : pair_a[blockIdx.x], head = blockIdx.y;
  if (unit < 0) break;
  const int tile = unit / n_splits, split = unit - tile * n_splits;
  const int kvh = head / (heads / kv_heads);
  const int tq0 = tile_q0[tile];
  const int rows = tile_rows[tile];
  const int pos0 = positions[tq0];
  const int32_t* table = block_table + static_cast<int64_t>(tile_seq[tile]) * max_blocks;
  const int lo = (window > 0 && pos0 + 1 > window) ? pos0 + 1 - window : 0;
  // this workgroup's keys [kb0, hi): all that the tile reads, or one slice of them.  Slices are whole rounds of 64
  // keys from the tile's first round on, so a slice ends at a round's edge or where the tile's keys end, and the
  // masks below need not know of it.  A slice may be empty: then nothing is summed, and (-inf, 0, 0) is written.
  const int hi_tile = pos0 + rows;
  int kb0 = lo & ~(PF_KEYS - 1);
  int hi = hi_tile;
  if (n_splits > 1) {
    const int per = (((hi_tile - kb0 + n_splits - 1) / n_splits) + PF_KEYS - 1) & ~(PF_KEYS - 1);
    kb0 += split * per;
    hi = min(hi_tile, kb0 + per);
  }
  const int wq0 = 16 * QT * wave;  // this wavefront's first query within the tile

  bf16x8 qf[QT][NC];
#pragma unroll
  for (int t = 0; t < QT; ++t)
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      const int d0 = 32 * c + 8 * g, r = wq0 + 16 * t + n;
      if (r < rows && d0 < D)
        qf[t][c] = *reinterpret_cast<const bf16x8*>(q + (static_cast<int64_t>(tq0 + r) * heads + head) * D + d0);
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

  // Staging.  A tile is four groups of 16 consecutive keys; a group starts at a multiple of 16, so it lies within
  // one page, and which page that is, is the same for every thread: the table is read with uniform addresses, one
  // tile ahead of the keys and values it points to.  Of every tile a thread moves K_PER 16-byte pieces of key rows
  // and V_PER of value rows; piece c of a group is (key c / 2NB, piece c % 2NB of its row) for keys and
  // (row c / 2, keys 8 (c % 2) ..) for values, so that neighbouring threads read neighbouring memory.
  // Keys past the tile's last one, and pages that a window has passed (-1 in the table), are read from some page of
  // the pool and masked where they are used; their values are written to LDS as zeros (see stage), because a
  // probability of zero times whatever an earlier request left in a page need not be zero.
  constexpr int GROUPS = PF_KEYS / 16, GROUP_CHUNKS = 32 * NB;
  __builtin_assume(tid < 256);
  int k_grp[K_PER], k_src[K_PER], k_dst[K_PER], v_grp[V_PER], v_src[V_PER], v_dst[V_PER], v_key[V_PER];
#pragma unroll
  for (int i = 0; i < K_PER; ++i) {
    const int c = min(tid + 256 * i, K_CHUNKS - 1), w = c % GROUP_CHUNKS;
    const int key = w / (2 * NB), d0 = (w % (2 * NB)) * 8, row = (c / GROUP_CHUNKS) * 16 + key;
    k_grp[i] = c / GROUP_CHUNKS;
    k_src[i] = key * D + d0;
    // piece p of row r sits at place p ^ swz(r): the sixteen rows that a quarter wavefront reads together are
    // r = 8 a + 4 b + e (a, e < 4) plus a multiple of 32, and (e, a) gives each a place of its own
    k_dst[i] = row * KS + ((d0 >> 3) ^ ((row & 3) | (((row >> 3) & 3) << 2))) * 8;
  }
#pragma unroll
  for (int i = 0; i < V_PER; ++i) {
    const int c = min(tid + 256 * i, V_CHUNKS - 1), w = c % GROUP_CHUNKS;
    // sixteen lanes take the same half (8 keys) of sixteen rows: with the permutation below they write to, and a
    // quarter wavefront later reads from, sixteen different groups of four banks
    const int half = (w >> 4) & 1, dd = (w & 15) | ((w >> 5) << 4);
    v_grp[i] = c / GROUP_CHUNKS;
    v_src[i] = dd * page_size + half * 8;
    v_key[i] = 16 * (c / GROUP_CHUNKS) + 8 * half;  // the piece's first key within the tile
    v_dst[i] = dd * VS + (((2 * (c / GROUP_CHUNKS) + half) ^ ((dd >> 1) & 7)) << 3);
  }
  const int64_t page_elems = static_cast<int64_t>(kv_heads) * page_size * D;
  const __bf16* k_head = k_cache + static_cast<int64_t>(kvh) * page_size * D;
  const __bf16* v_head = v_cache + static_cast<int64_t>(kvh) * page_size * D;
  const int last_page = (hi_tile - 1) >> page_shift;
  // The table entries of a tile's groups are asked for one round before they are used, with vector loads (every
  // lane the same address): a scalar load would share its counter with the LDS reads of the round and be waited
  // for at the first of them.
  int pages[GROUPS];
  int vzero = 0;
  asm volatile("" : "+v"(vzero));  // zero in a vector register that the compiler takes for any number
  auto ask_pages = [&](int kb) {
#pragma unroll
    for (int j = 0; j < GROUPS; ++j) pages[j] = table[min((kb + 16 * j) >> page_shift, last_page) + vzero];
  };
  int64_t k_at[GROUPS], v_at[GROUPS];  // where each group of the tile to fetch starts (uniform)
  auto locate = [&](int kb) {
#pragma unroll
    for (int j = 0; j < GROUPS; ++j) {
      const int off = (kb + 16 * j) & (page_size - 1);
      const int64_t page = max(__builtin_amdgcn_readfirstlane(pages[j]), 0);
      k_at[j] = page * page_elems + off * D;
      v_at[j] = page * page_elems + off;
    }
  };
  auto pick = [&](const int64_t (&at)[GROUPS], int grp) {
    int64_t r = at[0];
#pragma unroll
    for (int j = 1; j < GROUPS; ++j) r = grp == j ? at[j] : r;
    return r;
  };
  bf16x8 kreg[K_PER], vreg[V_PER];
  auto fetch = [&]() {
#pragma unroll
    for (int i = 0; i < K_PER; ++i) kreg[i] = *reinterpret_cast<const bf16x8*>(k_head + pick(k_at, k_grp[i]) + k_src[i]);
#pragma unroll
    for (int i = 0; i < V_PER; ++i) vreg[i] = *reinterpret_cast<const bf16x8*>(v_head + pick(v_at, v_grp[i]) + v_src[i]);
  };
  auto key_place = [&](int row, int d0) { return row * KS + ((d0 >> 3) ^ ((row & 3) | (((row >> 3) & 3) << 2))) * 8; };
  // `tile_kb`: the first key of the tile that the registers hold.  At the tile's edges (uniform) the values of keys
  // that no query may read become zeros on their way into LDS.
  auto stage = [&](int buf, int tile_kb) {
    __bf16* ks = k_tiles[buf];
    __bf16* vs = v_tiles[buf];
#pragma unroll
    for (int i = 0; i < K_PER; ++i)
      if (tid + 256 * i < K_CHUNKS) *reinterpret_cast<bf16x8*>(ks + k_dst[i]) = kreg[i];
    if (tile_kb + PF_KEYS > hi_tile || tile_kb < lo) {
#pragma unroll
      for (int i = 0; i < V_PER; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int key = tile_kb + v_key[i] + j;
          if (key >= hi_tile || key < lo) vreg[i][j] = (__bf16)0.f;
        }
    }
#pragma unroll
    for (int i = 0; i < V_PER; ++i)
      if (tid + 256 * i < V_CHUNKS) *reinterpret_cast<bf16x8*>(vs + v_dst[i]) = vreg[i];
  };

  // a tile has at least one query, so kb0 < hi (but for an empty slice, whose staged keys are then not used): the
  // first key tile is staged without a condition (the wait for
  // it also covers the loads of the queries above, which the loop then need not wait for again)
  ask_pages(kb0);
  locate(kb0);
  fetch();
  ask_pages(kb0 + PF_KEYS);
  stage(0, kb0);
  if (kb0 + PF_KEYS < hi) {
    locate(kb0 + PF_KEYS);
    fetch();
    ask_pages(kb0 + 2 * PF_KEYS);
  }
  __syncthreads();
  const int bp16 = (lane ^ 16) << 2, bp32 = (lane ^ 32) << 2;  // ds_bpermute addresses of the lanes 16 and 32 away
  int buf = 0;
  for (int kb = kb0; kb < hi; kb += PF_KEYS, buf ^= 1) {
    // The registers hold tile kb + 64 (loaded while tile kb - 64 was multiplied): it goes into the buffer that
    // the previous round read, which every wavefront has left (the barrier below); then tile kb + 128 is asked for.
    if (kb + PF_KEYS < hi) {
      stage(buf ^ 1, kb + PF_KEYS);
      if (kb + 2 * PF_KEYS < hi) {
        locate(kb + 2 * PF_KEYS);
        fetch();
        ask_pages(kb + 3 * PF_KEYS);
      }
    }
    const __bf16* ks = k_tiles[buf];
    const __bf16* vs = v_tiles[buf];
#pragma unroll
    for (int h2 = 0; h2 < 2; ++h2) {
      const int kb2 = kb + 32 * h2;
      // does any query of this wavefront read keys from kb2 on?  (uniform over the wavefront)
      if (kb2 >= hi || wq0 >= rows || kb2 > pos0 + min(wq0 + 16 * QT, rows) - 1) continue;
      bf16x8 kf[2][NC], vf[NB];
#pragma unroll
      for (int b = 0; b < 2; ++b) {
        const int kl = 32 * h2 + 8 * (n >> 2) + 4 * b + (n & 3);  // A row n of block b
#pragma unroll
        for (int c = 0; c < NC; ++c) {
          const int d0 = 32 * c + 8 * g;
          if (d0 < D)
            kf[b][c] = *reinterpret_cast<const bf16x8*>(ks + key_place(kl, d0));
          else
            for (int j = 0; j < 8; ++j) kf[b][c][j] = (__bf16)0.f;
        }
      }
#pragma unroll
      for (int b = 0; b < NB; ++b)  // row 16 b + n, piece 4 h2 + g; (row >> 1) & 7 = (n >> 1) & 7
        vf[b] = *reinterpret_cast<const bf16x8*>(vs + (16 * b + n) * VS + (((4 * h2 + g) ^ ((n >> 1) & 7)) << 3));
#pragma unroll
      for (int t = 0; t < QT; ++t) {
        if (wq0 + 16 * t >= rows || kb2 > pos0 + wq0 + 16 * t + 15) continue;
        f32x4 s[2];
#pragma unroll
        for (int b = 0; b < 2; ++b) {
          s[b] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int c = 0; c < NC; ++c)
            s[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[b][c], qf[t][c], s[b], 0, 0, 0);
        }
        const int my_pos = pos0 + wq0 + 16 * t + n;
        const bool my_row = wq0 + 16 * t + n < rows;
        const int my_lo = (window > 0 && my_pos + 1 > window) ? my_pos + 1 - window : 0;
        // scores stay unscaled: the scale (times log2 e) enters with the running maximum in one fused multiply-add
        float sv[8];
        float mx = -INFINITY;
        // keys that every query of these sixteen sees need no mask (uniform over the wavefront)
        const bool inner = wq0 + 16 * t + 16 <= rows && kb2 + 31 <= pos0 + wq0 + 16 * t &&
                           (window == 0 || kb2 > pos0 + wq0 + 16 * t + 15 - window);
        if (inner) {
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            sv[j] = s[j >> 2][j & 3];
            mx = fmaxf(mx, sv[j]);
          }
        } else {
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            const int key = kb2 + 8 * g + j;
            const bool ok = my_row && key >= my_lo && key <= my_pos;
            sv[j] = ok ? s[j >> 2][j & 3] : -INFINITY;
            mx = fmaxf(mx, sv[j]);
          }
        }
        mx = fmaxf(mx, __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(bp16, __builtin_bit_cast(int, mx))));
        mx = fmaxf(mx, __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(bp32, __builtin_bit_cast(int, mx))));
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
#pragma unroll
        for (int b = 0; b < NB; ++b) o[t][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[b], pf, o[t][b], 0, 0, 0);
      }
    }
    __syncthreads();
  }

#pragma unroll
  for (int t = 0; t < QT; ++t) {
    float l = lsum[t];
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);
    const int r = wq0 + 16 * t + n;
    if (r >= rows) continue;
    if (n_splits > 1) {  // this slice's part: reference point, sum and unnormalised output, for attn_combine_kernel
      const int64_t p = (static_cast<int64_t>(tq0 + r) * heads + head) * n_splits + split;
      float* dst = part_o + p * D + 4 * g;
#pragma unroll
      for (int b = 0; b < NB; ++b) *reinterpret_cast<f32x4*>(dst + 16 * b) = o[t][b];
      if (g == 0) {
        part_ml[2 * p] = m[t];
        part_ml[2 * p + 1] = l;
      }
      continue;
    }
    const float inv = 1.0f / l;
    __bf16* dst = out + (static_cast<int64_t>(tq0 + r) * heads + head) * D + 4 * g;  // rows d = 16 b + 4 g + i
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      bf16x4 v;
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] = (__bf16)(o[t][b][i] * inv);
      *reinterpret_cast<bf16x4*>(dst + 16 * b) = v;
    }
  }
  }  // the two tiles
}

template <int NB>
static void launch_prefill(int tile_queries, dim3 grid, hipStream_t stream, const void* q, const void* k,
                           const void* v, const int32_t* table, const int32_t* tile_seq, const int32_t* tile_q0,
                           const int32_t* tile_rows, const int32_t* pair_a, const int32_t* pair_b,
                           const int32_t* positions, void* out, float* part_o, float* part_ml, int n_splits,
                           int heads, int kv_heads, int page_size, int max_blocks, float scale_log2, int window) {
  int page_shift = 4;  // log2 of the page size, a power of two (the entry point has checked)
  while ((1 << page_shift) < page_size) ++page_shift;
  (void)tile_queries;  // 64: the entry point has checked
  hipLaunchKernelGGL((attn_prefill_kernel<NB, 1>), grid, dim3(256), 0, stream, (const __bf16*)q, (const __bf16*)k,
                     (const __bf16*)v, table, tile_seq, tile_q0, tile_rows, pair_a, pair_b, positions, (__bf16*)out, part_o,
                     part_ml, n_splits, heads, kv_heads, page_size, max_blocks, scale_log2, window, page_shift);
}

// Tiles of up to `tile_queries` (64) consecutive queries of one request; head_dim a multiple of 16 up to 128; pages
// of a power of two (from 16) of keys.
// Workgroup p (per head) takes units pair_a[p] and then pair_b[p] (or none if that is -1); the caller names every
// unit exactly once (a tile left out stays unwritten).  A unit is a tile, or with n_splits > 1 the slice
// unit % n_splits of the keys of tile unit / n_splits: then the slices' parts go to part_o float32
// [tokens * heads * n_splits * head_dim] and part_ml float32 [tokens * heads * n_splits * 2], and a second kernel
// puts them together for ALL `tokens` rows of `out` (rows of no tile get what their unwritten parts give).
extern "C" int ix_attention_prefill(const void* q, const void* k_cache, const void* v_cache,
                                    const int32_t* block_table, const int32_t* tile_seq, const int32_t* tile_q0,
                                    const int32_t* tile_rows, const int32_t* pair_a, const int32_t* pair_b,
                                    int n_pairs, const int32_t* positions, void* out, float* part_o,
                                    float* part_ml, int n_splits, int64_t tokens, int n_tiles,
                                    int tile_queries, int heads, int kv_heads, int head_dim, int page_size,
                                    int max_blocks, float scale, int window, hipStream_t stream) {
  IX_REQUIRE(n_tiles >= 0 && heads > 0 && kv_heads > 0 && max_blocks > 0, "sizes must be positive");
  IX_REQUIRE(heads % kv_heads == 0, "heads must be a multiple of kv_heads");
  IX_REQUIRE(head_dim % 16 == 0 && head_dim >= 16 && head_dim <= 128, "head_dim must be a multiple of 16 up to 128");
  IX_REQUIRE(page_size >= 16 && (page_size & (page_size - 1)) == 0, "page_size must be a power of two from 16 on");
  IX_REQUIRE(tile_queries == 64, "a query tile holds up to 64 queries");
  IX_REQUIRE(window >= 0, "window must not be negative");
  IX_REQUIRE(heads <= 65535, "too many heads");
  IX_REQUIRE(n_splits >= 1 && n_splits <= 256, "n_splits must be between 1 and 256");
  IX_REQUIRE(n_splits == 1 || (part_o != nullptr && part_ml != nullptr && tokens > 0), "workspace needed for split keys");
  IX_REQUIRE(n_pairs >= 0 && n_pairs <= static_cast<int64_t>(n_tiles) * n_splits, "there are at most as many pairs as units");
  if (n_tiles == 0 || n_pairs == 0) return 0;
  dim3 grid(n_pairs, heads);
  const float scale_log2 = scale * 1.4426950408889634f;
#define CASE(NB)                                                                                                   \
  case NB:                                                                                                         \
    launch_prefill<NB>(tile_queries, grid, stream, q, k_cache, v_cache, block_table, tile_seq, tile_q0, tile_rows, \
                       pair_a, pair_b, positions, out, part_o, part_ml, n_splits, heads, kv_heads, page_size, max_blocks,  \
                       scale_log2, window);                                                                        \
    break;
  switch (head_dim / 16) { CASE(1) CASE(2) CASE(3) CASE(4) CASE(5) CASE(6) CASE(7) CASE(8) }
#undef CASE
  if (ix_check_launch("ix_attention_prefill")) return 1;
  if (n_splits > 1) return ix_attention_combine(part_o, part_ml, out, tokens, heads, n_splits, head_dim, stream);
  return 0;
}
