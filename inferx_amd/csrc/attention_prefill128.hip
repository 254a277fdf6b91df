// Paged attention for prompt portions (bfloat16), tiles of 128 queries: four
// wavefronts multiply, four others only move keys and values into LDS.
//
// The kernel with tiles of 64 queries (attention_prefill.hip) gives each
// wavefront 16 queries; every wavefront reads every key and value tile from LDS
// for them, 32 KB per 32 products of 16 x 16 x 32, and a compute unit's LDS then
// delivers operands more slowly than its matrix cores take them.  Here a
// wavefront owns 32 queries and multiplies with v_mfma_f32_32x32x16_bf16: the
// same 32 KB feed twice the work (32 products of twice the size), which is about
// what the matrix cores take in the time the LDS needs to deliver it.
//
// A workgroup is 8 wavefronts on one tile of up to 128 consecutive queries of
// one request and one query head.  Wavefronts 0..3 (one per SIMD) hold the
// queries and form  S^T = K Q^T  and  O^T += V^T P^T  (so that no operand is
// turned round: the products' results are the next products' operands).
// Wavefronts 4..7 (one per SIMD, beside them) load: each round they write the
// tile that arrived from memory into the LDS buffer that is not being read and
// ask for the tile three rounds ahead (two register sets, so a load has two
// rounds to arrive).  One barrier per round of 64 keys is all the two kinds
// share; a wait for memory stalls a loading wavefront, never a multiplying one.
//
// Layouts.  The matrix cores' 32 x 32 result leaves lane l with column l % 32
// and rows 8 b + 4 (l / 32) + e (b, e < 4).  For S^T (rows = keys) that is, per
// sixteen keys, keys 4 h + e and 8 + 4 h + e of lane half h = l / 32: exactly the
// eight reduction indices that the lane must supply as the B operand of the next
// product if the A operand (values, transposed) names the keys in the same
// order.  Values are kept transposed within a page, so a row of the value tile
// (one d, 16 keys of a page) is 32 contiguous bytes; the loading wavefronts
// write it as [keys 0-3, 8-11 | 4-7, 12-15], and a lane half's operand is one
// 16-byte piece.  Key rows are stored as they are.  16-byte pieces of both tiles
// are permuted so that the sixteen lanes that LDS serves together touch all banks.
//
// Masking, the lazily moving reference point of the exponentials, slices of a
// tile's keys with their parts, pairs of units per workgroup and the rule that
// values of keys that no query may read enter LDS as zeros are those of
// attention_prefill.hip.
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

#define PW_KEYS 64      // keys per round
#define PW_QUERIES 128  // queries per workgroup
#define PW_LOADERS 256  // threads that load

template <int NB2>  // head_dim = 32 * NB2
__global__ void __launch_bounds__(512)
attn_prefill128_kernel(const __bf16* __restrict__ q, const __bf16* k_cache, const __bf16* v_cache,
                       const int32_t* __restrict__ block_table, const int32_t* __restrict__ tile_seq,
                       const int32_t* __restrict__ tile_q0, const int32_t* __restrict__ tile_rows,
                       const int32_t* __restrict__ pair_a, const int32_t* __restrict__ pair_b,
                       const int32_t* __restrict__ positions, __bf16* __restrict__ out, float* __restrict__ part_o,
                       float* __restrict__ part_ml, int n_splits, int heads, int kv_heads, int page_size,
                       int max_blocks, float scale_log2, int window, int page_shift) {
  constexpr int D = 32 * NB2;
  constexpr int NS = D / 16;                          // steps of 16 of the head dimension in K Q^T
  constexpr int RS = D <= 32 ? 4 : (D <= 64 ? 8 : 16);  // 16-byte pieces per LDS row of the key tile
  constexpr int KS = RS * 8;                          // elements per LDS row of the key tile
  constexpr int VS = PW_KEYS;                         // elements per LDS row of the value tile (one d, 64 keys)
  constexpr int K_PIECES = PW_KEYS * (D / 8);         // 16-byte pieces of a key tile
  constexpr int V_UNITS = D * (PW_KEYS / 16);         // (d, sixteen keys) units of a value tile, 32 bytes each
  constexpr int K_PER = (K_PIECES + PW_LOADERS - 1) / PW_LOADERS, V_PER = (V_UNITS + PW_LOADERS - 1) / PW_LOADERS;
  __shared__ __attribute__((aligned(16))) __bf16 k_tiles[2][PW_KEYS * KS];
  __shared__ __attribute__((aligned(16))) __bf16 v_tiles[2][D * VS];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // (uniform: what depends on it is decided by scalar code)
  const bool loads = wave >= 4;
  // piece p of key row r lies at place p ^ ((r / rows per 256 bytes) % RS): sixteen consecutive rows read at one
  // piece index then fall on sixteen different groups of four banks
  auto key_place = [&](int row, int piece) { return row * KS + ((piece ^ ((row / (16 / RS)) & (RS - 1))) << 3); };
  // piece p of value row d lies at place p ^ ((d >> 1) & 7)
  auto value_place = [&](int d, int piece) { return d * VS + ((piece ^ ((d >> 1) & 7)) << 3); };

  // id of the workgroup: heads fastest, so that the tiles of one head (which read the same keys) go to the same die
  const int head = blockIdx.x % heads, slot = blockIdx.x / heads;
#pragma unroll 1
  for (int which = 0; which < 2; ++which) {
    const int unit = which ? pair_b[slot] : pair_a[slot];
    if (unit < 0) break;
    const int tile = unit / n_splits, split = unit - tile * n_splits;
    const int kvh = head / (heads / kv_heads);
    const int tq0 = tile_q0[tile];
    const int rows = tile_rows[tile];
    const int pos0 = positions[tq0];
    const int32_t* table = block_table + static_cast<int64_t>(tile_seq[tile]) * max_blocks;
    const int lo = (window > 0 && pos0 + 1 > window) ? pos0 + 1 - window : 0;
    // this workgroup's keys [kb0, hi): all that the tile reads, or one slice of them (whole rounds from the tile's
    // first round on; a slice may be empty: then (-inf, 0, 0) is written)
    const int hi_tile = pos0 + rows;
    int kb0 = lo & ~(PW_KEYS - 1);
    int hi = hi_tile;
    if (n_splits > 1) {
      const int per = (((hi_tile - kb0 + n_splits - 1) / n_splits) + PW_KEYS - 1) & ~(PW_KEYS - 1);
      kb0 += split * per;
      hi = min(hi_tile, kb0 + per);
    }
    const int rounds = hi > kb0 ? (hi - kb0 + PW_KEYS - 1) / PW_KEYS : 0;
    const int rounds2 = (rounds + 1) & ~1;  // both kinds of wavefronts pass 1 + rounds2 barriers per unit

    if (loads) {
      // ---------------------------------------------------------------- the loading wavefronts
      const int ltid = tid - PW_LOADERS;
      // Of every tile a thread moves K_PER pieces of key rows (piece c: key c / (D / 8), piece c % (D / 8) of its row,
      // so neighbouring threads read neighbouring memory) and V_PER units of value rows (unit u: sixteen keys
      // u / D, row u % D; neighbouring threads read neighbouring rows, which lie 2 * page_size bytes apart).
      int k_grp[K_PER], k_src[K_PER], k_dst[K_PER], v_grp[V_PER], v_src[V_PER], v_dst[V_PER];
#pragma unroll
      for (int i = 0; i < K_PER; ++i) {
        const int c = min(ltid + PW_LOADERS * i, K_PIECES - 1);
        const int key = c / (D / 8), piece = c % (D / 8);
        k_grp[i] = key >> 4;
        k_src[i] = (key & 15) * D + piece * 8;
        k_dst[i] = key_place(key, piece);
      }
#pragma unroll
      for (int i = 0; i < V_PER; ++i) {
        const int u = min(ltid + PW_LOADERS * i, V_UNITS - 1);
        const int grp = u / D, d = u % D;
        v_grp[i] = grp;
        v_src[i] = d * page_size;
        v_dst[i] = d;  // (the places of its two pieces follow from d and the group)
      }
      const int64_t page_elems = static_cast<int64_t>(kv_heads) * page_size * D;
      const __bf16* k_head = k_cache + static_cast<int64_t>(kvh) * page_size * D;
      const __bf16* v_head = v_cache + static_cast<int64_t>(kvh) * page_size * D;
      const int last_page = (hi_tile - 1) >> page_shift;
      const int last_round = max(rounds - 1, 0);
      // Every load is unconditional (a round past the last asks for the last round's tile again; a key past the
      // tile's last one for some page of the pool, masked where it is used): the loop below is then one straight
      // line, and the compiler can count how many loads may stay in flight at each wait.
      auto page_of = [&](int round, int grp) {
        const int kb = kb0 + PW_KEYS * min(round, last_round) + 16 * grp;
        return table[min(kb >> page_shift, last_page)];
      };
      struct Regs {
        bf16x8 k[K_PER];
        bf16x8 v[V_PER][2];
      };
      struct Pages {
        int k[K_PER];
        int v[V_PER];
      };
      auto fetch = [&](int round, Regs& r, const Pages& pg) {
        const int kb = kb0 + PW_KEYS * min(round, last_round);
#pragma unroll
        for (int i = 0; i < K_PER; ++i) {
          const int off = (kb + 16 * k_grp[i]) & (page_size - 1);
          r.k[i] = *reinterpret_cast<const bf16x8*>(k_head + max(pg.k[i], 0) * page_elems + off * D + k_src[i]);
        }
#pragma unroll
        for (int i = 0; i < V_PER; ++i) {
          const int off = (kb + 16 * v_grp[i]) & (page_size - 1);
          const __bf16* src = v_head + max(pg.v[i], 0) * page_elems + off + v_src[i];
          r.v[i][0] = *reinterpret_cast<const bf16x8*>(src);
          r.v[i][1] = *reinterpret_cast<const bf16x8*>(src + 8);
        }
      };
      auto ask_pages = [&](int round, Pages& pg) {
#pragma unroll
        for (int i = 0; i < K_PER; ++i) pg.k[i] = page_of(round, k_grp[i]);
#pragma unroll
        for (int i = 0; i < V_PER; ++i) pg.v[i] = page_of(round, v_grp[i]);
      };
      // `round`: the round whose tile the registers hold.  At the tile's edges (uniform) the values of keys that no
      // query may read become zeros on their way into LDS: a probability of zero times whatever an earlier request
      // left in a page need not be zero.
      auto stage = [&](int round, Regs& r) {
        if (round >= rounds) return;
        const int buf = round & 1, tile_kb = kb0 + PW_KEYS * round;
        __bf16* ks = k_tiles[buf];
        __bf16* vs = v_tiles[buf];
#pragma unroll
        for (int i = 0; i < K_PER; ++i)
          if (ltid + PW_LOADERS * i < K_PIECES) *reinterpret_cast<bf16x8*>(ks + k_dst[i]) = r.k[i];
        const bool edge = tile_kb + PW_KEYS > hi_tile || tile_kb < lo;
#pragma unroll
        for (int i = 0; i < V_PER; ++i) {
          if (edge) {
#pragma unroll
            for (int j = 0; j < 16; ++j) {
              const int key = tile_kb + 16 * v_grp[i] + j;
              if (key >= hi_tile || key < lo) r.v[i][j >> 3][j & 7] = (__bf16)0.f;
            }
          }
          // keys 0-3, 8-11 to the piece of lane half 0, keys 4-7, 12-15 to that of lane half 1
          bf16x8 t0, t1;
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            t0[j] = r.v[i][0][j];
            t0[4 + j] = r.v[i][1][j];
            t1[j] = r.v[i][0][4 + j];
            t1[4 + j] = r.v[i][1][4 + j];
          }
          if (ltid + PW_LOADERS * i < V_UNITS) {
            *reinterpret_cast<bf16x8*>(vs + value_place(v_dst[i], 2 * v_grp[i])) = t0;
            *reinterpret_cast<bf16x8*>(vs + value_place(v_dst[i], 2 * v_grp[i] + 1)) = t1;
          }
        }
      };

      // Tiles of even and of odd rounds have a register set each, and so have their table entries.  A tile's loads
      // are issued three rounds before it is multiplied and its table entries one round before that, so that
      // neither the loads nor the writes into LDS ever wait for the loads issued last.
      Regs even, odd;
      Pages pg_even, pg_odd;
      ask_pages(0, pg_even);
      ask_pages(1, pg_odd);
      fetch(0, even, pg_even);
      ask_pages(2, pg_even);
      fetch(1, odd, pg_odd);
      ask_pages(3, pg_odd);
      stage(0, even);
      fetch(2, even, pg_even);
      __syncthreads();
      // round r is being multiplied from buffer r & 1: tile r + 1 goes into the other buffer (whose readers have
      // passed the barrier), the table entries of tile r + 4 are asked for, and tile r + 3 takes the registers
      for (int r = 0; r < rounds2; r += 2) {
        stage(r + 1, odd);
        ask_pages(r + 4, pg_even);
        fetch(r + 3, odd, pg_odd);
        __syncthreads();
        stage(r + 2, even);
        ask_pages(r + 5, pg_odd);
        fetch(r + 4, even, pg_even);
        __syncthreads();
      }
      continue;
    }

    // ------------------------------------------------------------------ the multiplying wavefronts
    const int qn = lane & 31, h = lane >> 5;
    const int wq0 = 32 * wave;                      // this wavefront's first query within the tile
    const bool active = wq0 < rows;
    const int wfirst = pos0 + wq0;                  // position of its first query and of its last one
    const int wlast = pos0 + min(wq0 + 32, rows) - 1;
    const int wlo = (window > 0 && wfirst + 1 > window) ? wfirst + 1 - window : 0;  // the first key any of them reads
    const int my_pos = wfirst + qn;
    const bool my_row = wq0 + qn < rows;
    const int my_lo = (window > 0 && my_pos + 1 > window) ? my_pos + 1 - window : 0;

    bf16x8 qf[NS];  // B operand of K Q^T: column qn, reduction indices 16 s + 8 h + j
#pragma unroll
    for (int s = 0; s < NS; ++s) {
      if (my_row)
        qf[s] = *reinterpret_cast<const bf16x8*>(q + (static_cast<int64_t>(tq0 + wq0 + qn) * heads + head) * D + 16 * s + 8 * h);
      else
        for (int j = 0; j < 8; ++j) qf[s][j] = (__bf16)0.f;
    }
    f32x16 o[NB2];
#pragma unroll
    for (int b = 0; b < NB2; ++b)
#pragma unroll
      for (int i = 0; i < 16; ++i) o[b][i] = 0.f;
    float m = -INFINITY, lsum = 0.f;
    const int swap32 = (lane ^ 32) << 2;  // ds_bpermute address of the lane that holds the other keys of this query
    // operand places: key row 32 b + qn has the permutation of row qn (32 is a multiple of what it repeats after),
    // value row 32 b + qn that of row qn likewise
    int k_at[NS], v_at[4];
#pragma unroll
    for (int s = 0; s < NS; ++s) k_at[s] = key_place(qn, 2 * s + h);
#pragma unroll
    for (int s = 0; s < 4; ++s) v_at[s] = value_place(qn, 2 * s + h);

    __syncthreads();
    for (int r = 0; r < rounds2; ++r) {
      const int kb = kb0 + PW_KEYS * r;
      const __bf16* ks = k_tiles[r & 1];
      const __bf16* vs = v_tiles[r & 1];
      // does any query of this wavefront read a key of this round?  (uniform over the wavefront)
      if (active && r < rounds && kb <= wlast && kb + PW_KEYS > wlo) {
        // All operand pieces of the round's keys are asked for at once; the products start as they arrive.  (At the
        // diagonal's end the second 32 keys may lie beyond every query: they are multiplied all the same and masked.)
        // Eight operand pieces of the round's keys are asked for at once, and one more with every product: enough in
        // flight to hide the way from LDS, in a quarter of the registers that all of them would take.
        constexpr int AHEAD = NS < 4 ? 2 * NS : 8;
        bf16x8 ka[2 * NS];  // piece i: step i / 2, key rows 32 (i % 2) + qn
#pragma unroll
        for (int i = 0; i < AHEAD; ++i) ka[i] = *reinterpret_cast<const bf16x8*>(ks + k_at[i >> 1] + 32 * (i & 1) * KS);
        __builtin_amdgcn_sched_barrier(0);
        f32x16 s[2];
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
          for (int i = 0; i < 16; ++i) s[b][i] = 0.f;
#pragma unroll
        for (int i = 0; i < 2 * NS; ++i) {
          s[i & 1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka[i], qf[i >> 1], s[i & 1], 0, 0, 0);
          if (i + AHEAD < 2 * NS)
            ka[i + AHEAD] = *reinterpret_cast<const bf16x8*>(ks + k_at[(i + AHEAD) >> 1] + 32 * ((i + AHEAD) & 1) * KS);
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // one product, then one LDS read
          __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
        // the first half of the values' operand pieces is asked for before the exponentials, behind which it arrives;
        // the second half when the scores' registers are free, and arrives behind the first half's products
        bf16x8 va[4][NB2];
#pragma unroll
        for (int g = 0; g < 2; ++g)
#pragma unroll
          for (int b = 0; b < NB2; ++b) va[g][b] = *reinterpret_cast<const bf16x8*>(vs + v_at[g] + 32 * b * VS);
        __builtin_amdgcn_sched_barrier(0);
        // this lane: query qn, keys kb + 32 b + 8 c + 4 h + e for element 4 c + e of s[b]
        // keys that every query of the wavefront sees need no mask (uniform)
        const bool inner = wq0 + 32 <= rows && kb + PW_KEYS - 1 <= wfirst && (window == 0 || kb > wlast - window);
        float mx = -INFINITY;
        if (inner) {
#pragma unroll
          for (int b = 0; b < 2; ++b)
#pragma unroll
            for (int i = 0; i < 16; ++i) mx = fmaxf(mx, s[b][i]);
        } else {
#pragma unroll
          for (int b = 0; b < 2; ++b)
#pragma unroll
            for (int i = 0; i < 16; ++i) {
              const int key = kb + 32 * b + 8 * (i >> 2) + 4 * h + (i & 3);
              const bool ok = my_row && key >= my_lo && key <= my_pos;
              s[b][i] = ok ? s[b][i] : -INFINITY;
              mx = fmaxf(mx, s[b][i]);
            }
        }
        mx = fmaxf(mx, __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(swap32, __builtin_bit_cast(int, mx))));
        // The reference point m of the exponentials (in units of log2) follows the running maximum lazily: it moves
        // only when some query's maximum has outgrown it by more than 2^8, so the accumulators are seldom rescaled.
        // Scores stay unscaled: the scale (times log2 e) enters with the reference point in one fused multiply-add.
        const float top = mx * scale_log2;
        if (__any(top > m + 8.f)) {
          const float m_new = fmaxf(m, top);
          const float alpha = __builtin_amdgcn_exp2f(m - ((m_new == -INFINITY) ? 0.f : m_new));
          lsum *= alpha;
#pragma unroll
          for (int b = 0; b < NB2; ++b)
#pragma unroll
            for (int i = 0; i < 16; ++i) o[b][i] *= alpha;
          m = m_new;
        }
        const float m_safe = (m == -INFINITY) ? 0.f : m;
        // B operands of V^T P^T: sixteen keys 16 g per step, this lane's keys 4 h + e and 8 + 4 h + e of them,
        // which are elements 8 (g % 2) + e and 8 (g % 2) + 4 + e of s[g / 2]
        bf16x8 pf[4];
        float psum = 0.f;
#pragma unroll
        for (int g = 0; g < 4; ++g)
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            const float p = __builtin_amdgcn_exp2f(fmaf(s[g >> 1][8 * (g & 1) + j], scale_log2, -m_safe));
            psum += p;
            pf[g][j] = (__bf16)p;
          }
        lsum += psum;
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int g = 2; g < 4; ++g)
#pragma unroll
          for (int b = 0; b < NB2; ++b) va[g][b] = *reinterpret_cast<const bf16x8*>(vs + v_at[g] + 32 * b * VS);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int g = 0; g < 4; ++g)
#pragma unroll
          for (int b = 0; b < NB2; ++b) o[b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va[g][b], pf[g], o[b], 0, 0, 0);
      }
      __syncthreads();
    }

    float l = lsum;
    l += __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(swap32, __builtin_bit_cast(int, l)));
    if (!my_row) continue;
    // this lane: query qn, output elements d = 32 b + 8 c + 4 h + e
    if (n_splits > 1) {  // this slice's part: reference point, sum and unnormalised output, for attn_combine_kernel
      const int64_t p = (static_cast<int64_t>(tq0 + wq0 + qn) * heads + head) * n_splits + split;
      float* dst = part_o + p * D + 4 * h;
#pragma unroll
      for (int b = 0; b < NB2; ++b)
#pragma unroll
        for (int c = 0; c < 4; ++c)
          *reinterpret_cast<f32x4*>(dst + 32 * b + 8 * c) = f32x4{o[b][4 * c], o[b][4 * c + 1], o[b][4 * c + 2], o[b][4 * c + 3]};
      if (h == 0) {
        part_ml[2 * p] = m;
        part_ml[2 * p + 1] = l;
      }
      continue;
    }
    const float inv = 1.0f / l;
    __bf16* dst = out + (static_cast<int64_t>(tq0 + wq0 + qn) * heads + head) * D + 4 * h;
#pragma unroll
    for (int b = 0; b < NB2; ++b)
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        bf16x4 v;
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = (__bf16)(o[b][4 * c + e] * inv);
        *reinterpret_cast<bf16x4*>(dst + 32 * b + 8 * c) = v;
      }
  }  // the two units
}

// As ix_attention_prefill (attention_prefill.hip), with tiles of up to 128 consecutive queries of one request and
// head_dim a multiple of 32 up to 128.
extern "C" int ix_attention_prefill128(const void* q, const void* k_cache, const void* v_cache,
                                       const int32_t* block_table, const int32_t* tile_seq, const int32_t* tile_q0,
                                       const int32_t* tile_rows, const int32_t* pair_a, const int32_t* pair_b,
                                       int n_pairs, const int32_t* positions, void* out, float* part_o,
                                       float* part_ml, int n_splits, int64_t tokens, int n_tiles, int heads,
                                       int kv_heads, int head_dim, int page_size, int max_blocks, float scale,
                                       int window, hipStream_t stream) {
  IX_REQUIRE(n_tiles >= 0 && heads > 0 && kv_heads > 0 && max_blocks > 0, "sizes must be positive");
  IX_REQUIRE(heads % kv_heads == 0, "heads must be a multiple of kv_heads");
  IX_REQUIRE(head_dim % 32 == 0 && head_dim >= 32 && head_dim <= 128, "head_dim must be a multiple of 32 up to 128");
  IX_REQUIRE(page_size >= 16 && (page_size & (page_size - 1)) == 0, "page_size must be a power of two from 16 on");
  IX_REQUIRE(window >= 0, "window must not be negative");
  IX_REQUIRE(n_splits >= 1 && n_splits <= 256, "n_splits must be between 1 and 256");
  IX_REQUIRE(n_splits == 1 || (part_o != nullptr && part_ml != nullptr && tokens > 0), "workspace needed for split keys");
  IX_REQUIRE(n_pairs >= 0 && n_pairs <= static_cast<int64_t>(n_tiles) * n_splits, "there are at most as many pairs as units");
  IX_REQUIRE(static_cast<int64_t>(n_pairs) * heads < (int64_t(1) << 31), "too many workgroups for one launch");
  if (n_tiles == 0 || n_pairs == 0) return 0;
  int page_shift = 4;
  while ((1 << page_shift) < page_size) ++page_shift;
  dim3 grid(static_cast<unsigned>(n_pairs) * heads);
  const float scale_log2 = scale * 1.4426950408889634f;
#define CASE(NB2)                                                                                                    \
  case NB2:                                                                                                          \
    hipLaunchKernelGGL((attn_prefill128_kernel<NB2>), grid, dim3(512), 0, stream, (const __bf16*)q,                  \
                       (const __bf16*)k_cache, (const __bf16*)v_cache, block_table, tile_seq, tile_q0, tile_rows,    \
                       pair_a, pair_b, positions, (__bf16*)out, part_o, part_ml, n_splits, heads, kv_heads, page_size, \
                       max_blocks, scale_log2, window, page_shift);                                                  \
    break;
  switch (head_dim / 32) { CASE(1) CASE(2) CASE(3) CASE(4) }
#undef CASE
  if (ix_check_launch("ix_attention_prefill128")) return 1;
  if (n_splits > 1) return ix_attention_combine(part_o, part_ml, out, tokens, heads, n_splits, head_dim, stream);
  return 0;
}
