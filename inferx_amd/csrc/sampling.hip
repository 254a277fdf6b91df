// Token selection on float32 logits [rows, vocab]: greedy, and temperature
// sampling with optional top-k / top-p / min-p cut-offs.
//
// Order of operations follows the reference's host sampler
// (src/engine/host_sampling.cc:50-110): temperature, softmax, cut-offs, one
// uniform draw scaled by the kept mass, walk of the cumulative sum.  The
// cut-offs keep exactly the prefix of the sorted order that the host sampler
// keeps (ties by index), found by histograms instead of a sort.  The walk is in
// index order, which samples the same truncated distribution.
#include "common.h"

#define SAMPLE_THREADS 1024

struct ArgPair {
  float v;
  int i;
};

__device__ __forceinline__ ArgPair better(ArgPair a, ArgPair b) {
  // larger value wins; equal values: lower index (reference: ArgmaxKernel, layers.cu:413-452)
  return (b.v > a.v || (b.v == a.v && b.i < a.i)) ? b : a;
}

__device__ ArgPair block_argmax(ArgPair p, ArgPair* red) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  ix_wave_argmax(p.v, p.i);
  __syncthreads();
  if (lane == 0) red[wave] = p;
  __syncthreads();
  ArgPair r = red[0];
  for (int w = 1; w < (int)(blockDim.x >> 6); ++w) r = better(r, red[w]);
  return r;
}

__global__ void __launch_bounds__(SAMPLE_THREADS)
argmax_kernel(const float* __restrict__ logits, int32_t* __restrict__ out, int64_t vocab) {
  __shared__ ArgPair red[16];
  const float* row = logits + blockIdx.x * vocab;
  ArgPair p{-INFINITY, 0x7fffffff};
  for (int64_t i = threadIdx.x; i < vocab; i += blockDim.x) {
    const float v = row[i];
    if (v > p.v) { p.v = v; p.i = (int)i; }
  }
  p = block_argmax(p, red);
  if (threadIdx.x == 0) out[blockIdx.x] = (p.i >= 0 && p.i < vocab) ? p.i : 0;
}

extern "C" int ix_argmax(const float* logits, int32_t* out, int64_t rows, int64_t vocab, hipStream_t stream) {
  IX_REQUIRE(rows >= 0 && vocab > 0 && vocab < (1ll << 31), "sizes must be positive");
  if (rows == 0) return 0;
  hipLaunchKernelGGL(argmax_kernel, dim3(rows), dim3(SAMPLE_THREADS), 0, stream, logits, out, vocab);
  return ix_check_launch("ix_argmax");
}

// 64-bit mix (splitmix64 finaliser) of key and counter -> uniform in [0, 1)
__device__ __forceinline__ float uniform_from(uint64_t key, uint64_t counter) {
  uint64_t z = key + 0x9e3779b97f4a7c15ull * (counter + 1ull);
  z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
  z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
  z = z ^ (z >> 31);
  return static_cast<float>(z >> 40) * (1.0f / 16777216.0f);
}

// One workgroup per row.  temperature <= 0 means greedy for that row.
//
// With u_i = max/t - l_i/t >= 0 the probabilities are p_i = exp(-u_i) (the most probable token has p = 1), and the
// order of the reference's sort -- falling p, rising index among equals -- is rising (u, index).  A cut-off keeps a
// prefix of that order, so all of them together keep the shortest prefix, up to and including one boundary token:
//   top-k    the token of rank k
//   min-p    the last token with u <= -ln(min_p)
//   top-p    the first token at which the running mass reaches top_p * total
// The boundary is found without sorting.  u is also taken as a 32-bit fixed-point number t = u * 2^27 (everything
// from u = 32 on, p < 1.3e-14, is the largest t).  A histogram over the upper 11 bits of t (bins of 1/64 in u; counts
// and masses as integers, so the order of the atomic additions does not matter and results repeat bit for bit)
// gives the bin the boundary lies in; if that bin holds more than 2,048 tokens, a histogram over its next 11 bits
// follows, then over the last 10; the tokens of the last bin are ranked exactly among themselves by (u, index).
// Only tokens that share all 32 bits of t with more than 2,048 others stay together.
// A pass over the row takes a workgroup about 25 us; a draw takes three to seven.
#define SAMPLE_BINS 2048
#define SAMPLE_LIST 2048
#define SAMPLE_MASS_ONE 1099511627776.0f  // 2^40: masses are summed as integers, p = 1 being 2^40

__device__ __forceinline__ float sample_u(float logit, float inv_t, float mx) {
  return fmaxf(fmaf(-logit, inv_t, mx), 0.f);  // formed the same way everywhere
}
__device__ __forceinline__ uint32_t sample_t(float u) {
  return u >= 32.f ? 0xffffffffu : (uint32_t)(u * 134217728.f);
}
__device__ __forceinline__ unsigned long long sample_q(float u) {
  return (unsigned long long)(expf(-u) * SAMPLE_MASS_ONE);
}

struct Cut {  // a token is kept if (t, u, index) <= (these) in that order
  uint32_t t;
  float u;
  int idx;
};
__device__ __forceinline__ bool kept(float u, int idx, Cut c) {
  const uint32_t t = sample_t(u);
  return t < c.t || (t == c.t && (u < c.u || (u == c.u && idx <= c.idx)));
}
__device__ __forceinline__ Cut stricter(Cut a, Cut b) {
  const bool b_first = b.t < a.t || (b.t == a.t && (b.u < a.u || (b.u == a.u && b.idx < a.idx)));
  return b_first ? b : a;
}

struct SampleShared {
  ArgPair ared[16];
  float red[16];
  uint32_t cnt[SAMPLE_BINS];
  unsigned long long mass[SAMPLE_BINS];
  float list_u[SAMPLE_LIST];
  int list_i[SAMPLE_LIST];
  unsigned long long list_q[SAMPLE_LIST];
  uint32_t list_n;
  int first_histogram_stands;   // cnt / mass still hold the histogram over the upper 11 bits of the whole row
  int bin;                      // the boundary's bin at the present level
  unsigned long long before;    // count or mass of the tokens before that bin
  unsigned long long all_mass;  // the whole row's mass
  Cut cut;
};

// The boundary token of one cut-off.  by_mass: the first token at which the running mass reaches `target` (in
// units of 2^-40); else the token of rank `target` (1-based).  A cut that keeps everything if there is none.
__device__ Cut sample_boundary(const float* __restrict__ row, int64_t vocab, float inv_t, float mx, bool by_mass,
                               unsigned long long target, SampleShared& sh) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const Cut keep_all{0xffffffffu, INFINITY, 0x7fffffff};
  const int shifts[3] = {21, 10, 0}, widths[3] = {11, 11, 10};
  unsigned long long before = 0;
  uint32_t prefix = 0;  // the bits of t above the present field, for the tokens still in question
  uint32_t in_bin = 0;
  int level = 0;
  for (;; ++level) {
    const int shift = shifts[level], width = widths[level];
    const int bins = 1 << width;
    if (!(level == 0 && sh.first_histogram_stands)) {
      __syncthreads();
      if (tid == 0) sh.first_histogram_stands = 0;
      for (int i = tid; i < SAMPLE_BINS; i += SAMPLE_THREADS) {
        sh.cnt[i] = 0;
        sh.mass[i] = 0;
      }
      __syncthreads();
      for (int64_t i = tid; i < vocab; i += SAMPLE_THREADS) {
        const float u = sample_u(row[i], inv_t, mx);
        const uint32_t t = sample_t(u);
        if (level > 0 && (t >> (shift + width)) != prefix) continue;
        const int bi = (int)((t >> shift) & (uint32_t)(bins - 1));
        atomicAdd(&sh.cnt[bi], 1u);
        if (by_mass) atomicAdd(&sh.mass[bi], sample_q(u));
      }
      __syncthreads();
    }
    // the bin in which the target is reached: the first wavefront, 32 bins per lane
    if (wave == 0) {
      unsigned long long mine = 0;
      for (int j = 0; j < SAMPLE_BINS / 64; ++j) {
        const int bi = lane * (SAMPLE_BINS / 64) + j;
        mine += by_mass ? sh.mass[bi] : (unsigned long long)sh.cnt[bi];
      }
      unsigned long long incl = mine;
#pragma unroll
      for (int off = 1; off < 64; off <<= 1) {
        const unsigned long long up = __shfl_up(incl, off, 64);
        if (lane >= off) incl += up;
      }
      const unsigned long long excl = before + incl - mine;
      const bool here = excl < target && target <= excl + mine;
      if (lane == 0) sh.bin = -1;  // stays if the target is never reached
      __builtin_amdgcn_wave_barrier();
      __threadfence_block();
      if (here) {
        unsigned long long run = excl;
        for (int j = 0; j < SAMPLE_BINS / 64; ++j) {
          const int bi = lane * (SAMPLE_BINS / 64) + j;
          const unsigned long long v = by_mass ? sh.mass[bi] : (unsigned long long)sh.cnt[bi];
          if (run + v >= target) {
            sh.bin = bi;
            sh.before = run;
            break;
          }
          run += v;
        }
      }
    }
    __syncthreads();
    const int b = sh.bin;
    if (b < 0) return keep_all;
    before = sh.before;
    in_bin = sh.cnt[b];
    prefix = (prefix << width) | (uint32_t)b;
    if (in_bin <= SAMPLE_LIST || level == 2) break;
  }
  const int shift = shifts[level];
  if (in_bin > SAMPLE_LIST) return Cut{prefix, INFINITY, 0x7fffffff};  // (level 2: the prefix is all of t)
  // the bin's tokens, ranked exactly among themselves
  __syncthreads();
  if (tid == 0) {
    sh.list_n = 0;
    sh.cut = keep_all;
  }
  __syncthreads();
  for (int64_t i = tid; i < vocab; i += SAMPLE_THREADS) {
    const float u = sample_u(row[i], inv_t, mx);
    if ((sample_t(u) >> shift) != prefix) continue;
    const uint32_t at = atomicAdd(&sh.list_n, 1u);
    if (at < SAMPLE_LIST) {
      sh.list_u[at] = u;
      sh.list_i[at] = (int)i;
      sh.list_q[at] = by_mass ? sample_q(u) : 1ull;
    }
  }
  __syncthreads();
  const int n = min((int)sh.list_n, SAMPLE_LIST);
  for (int e = tid; e < n; e += SAMPLE_THREADS) {
    const float ue = sh.list_u[e];
    const int ie = sh.list_i[e];
    unsigned long long upto = 0;  // count or mass of the bin's tokens up to and including this one
    for (int j = 0; j < n; ++j) {
      const float uj = sh.list_u[j];
      if (uj < ue || (uj == ue && sh.list_i[j] <= ie)) upto += sh.list_q[j];
    }
    // the boundary: the target is reached with this token and was not before it (exactly one token says so)
    if (before + upto >= target && before + upto - sh.list_q[e] < target) sh.cut = Cut{sample_t(ue), ue, ie};
  }
  __syncthreads();
  return sh.cut;
}

__global__ void __launch_bounds__(SAMPLE_THREADS)
sample_kernel(const float* __restrict__ logits, int32_t* __restrict__ out, const float* __restrict__ temperature,
              const float* __restrict__ top_p, const int32_t* __restrict__ top_k, const float* __restrict__ min_p,
              const uint64_t* __restrict__ rng_key, uint64_t* rng_counter, int advance, int64_t vocab) {
  __shared__ SampleShared sh;
  const int r = blockIdx.x, tid = threadIdx.x;
  const float* row = logits + static_cast<int64_t>(r) * vocab;
  const float temp = temperature[r];
  // The row's draw is number `draw` of its request.  With `advance` the counter is left at the next draw, so that
  // the parameters of a batch that stays together need not be brought to the device again step after step.
  const uint64_t draw = rng_counter[r];
  __syncthreads();
  if (advance && tid == 0) rng_counter[r] = draw + 1;

  ArgPair best{-INFINITY, 0x7fffffff};
  for (int64_t i = tid; i < vocab; i += SAMPLE_THREADS) {
    const float v = row[i];
    if (v > best.v) { best.v = v; best.i = (int)i; }
  }
  best = block_argmax(best, sh.ared);
  if (best.i < 0 || best.i >= vocab) best.i = 0;
  if (temp <= 0.f) {
    if (tid == 0) out[r] = best.i;
    return;
  }
  const float inv_t = 1.0f / temp;
  const float mx = best.v * inv_t;

  Cut cut{0xffffffffu, INFINITY, 0x7fffffff};  // keeps every token
  const float mp = min_p[r];
  if (mp > 0.f) {  // p >= min_p * p_max
    const float u_max = -logf(fminf(mp, 1.0f));
    cut = stricter(cut, Cut{sample_t(u_max), u_max, 0x7fffffff});
  }
  const int kk = top_k[r];
  const float tp = top_p[r];
  const bool by_rank = kk > 0 && kk < vocab, by_mass = tp < 1.0f;
  if (by_rank || by_mass) {
    // the first histogram serves both cut-offs
    for (int i = tid; i < SAMPLE_BINS; i += SAMPLE_THREADS) {
      sh.cnt[i] = 0;
      sh.mass[i] = 0;
    }
    if (tid == 0) {
      sh.all_mass = 0;
      sh.first_histogram_stands = 1;
    }
    __syncthreads();
    unsigned long long mine = 0;
    for (int64_t i = tid; i < vocab; i += SAMPLE_THREADS) {
      const float u = sample_u(row[i], inv_t, mx);
      const int bi = (int)(sample_t(u) >> 21);
      atomicAdd(&sh.cnt[bi], 1u);
      if (by_mass) {
        const unsigned long long q = sample_q(u);
        atomicAdd(&sh.mass[bi], q);
        mine += q;
      }
    }
    if (by_mass) atomicAdd(&sh.all_mass, mine);
    __syncthreads();
    if (by_rank) cut = stricter(cut, sample_boundary(row, vocab, inv_t, mx, false, (unsigned long long)kk, sh));
    if (by_mass) {
      unsigned long long want = (unsigned long long)ceil((double)tp * (double)sh.all_mass);
      if (want < 1) want = 1;
      cut = stricter(cut, sample_boundary(row, vocab, inv_t, mx, true, want, sh));
    }
  }

  // The kept mass of stretches of 64 G consecutive tokens (G such that there are at most 4,096 stretches; for a
  // vocabulary of up to 262,144 a stretch is 64 tokens, one load of a wavefront), each summed by one wavefront
  // in a fixed order.  The sums take the place of the histogram's masses, which are no longer needed.
  float* stretch = reinterpret_cast<float*>(sh.mass);
  static_assert(sizeof(sh.mass) >= 4096 * sizeof(float), "room for the sums of 4,096 stretches");
  const int lane = tid & 63, wave = tid >> 6;
  const int64_t units = (vocab + 63) / 64;
  const int G = static_cast<int>((units + 4095) / 4096);
  const int n_stretch = static_cast<int>((units + G - 1) / G);
  __syncthreads();
  for (int e = wave; e < n_stretch; e += SAMPLE_THREADS / 64) {
    float acc = 0.f;
    for (int gi = 0; gi < G; ++gi) {
      const int64_t i = (static_cast<int64_t>(e) * G + gi) * 64 + lane;
      if (i < vocab) {
        const float u = sample_u(row[i], inv_t, mx);
        acc += kept(u, (int)i, cut) ? expf(-u) : 0.f;
      }
    }
    acc = ix_wave_sum(acc);
    if (lane == 0) stretch[e] = acc;
  }
  __syncthreads();
  if (wave != 0) return;
  // The first wavefront finds the stretch in which the running mass passes the drawn point, then walks it 64
  // tokens at a time.  Sums are formed in a fixed order (a lane's stretches in turn, lanes by a scan).
  auto scan = [&](float v) {  // inclusive sums over the lanes
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const float up = __shfl_up(v, off, 64);
      if (lane >= off) v += up;
    }
    return v;
  };
  const int per_lane = (n_stretch + 63) / 64;
  float part = 0.f;
  for (int j = 0; j < per_lane; ++j)
    if (per_lane * lane + j < n_stretch) part += stretch[per_lane * lane + j];
  const float incl = scan(part);
  const float mass = __shfl(incl, 63, 64);
  const float target = uniform_from(rng_key[r], draw) * mass;
  const unsigned long long passes = __ballot(incl > target);
  const int at_lane = passes ? __builtin_ctzll(passes) : 63;
  float run = __shfl(incl - part, at_lane, 64);  // the mass before that lane's stretches
  int at = min(per_lane * at_lane, n_stretch - 1);
  for (int j = 0; j < per_lane - 1 && at + 1 < n_stretch; ++j) {  // every lane walks the same stretches: LDS broadcasts
    const float v = stretch[at];
    if (run + v > target) break;
    run += v;
    ++at;
  }
  const int64_t sb = static_cast<int64_t>(at) * G * 64, se = min<int64_t>(sb + static_cast<int64_t>(G) * 64, vocab);
  int pick = best.i;  // falls back to the most probable token
  for (int64_t c = sb; c < se; c += 64) {
    const int64_t i = c + lane;
    const bool valid = i < se;
    const float u = valid ? sample_u(row[i], inv_t, mx) : 0.f;
    const bool k = valid && kept(u, (int)i, cut);
    const float upto = scan(k ? expf(-u) : 0.f);
    const unsigned long long hit = __ballot(k && run + upto > target);
    if (hit) {
      pick = (int)(c + __builtin_ctzll(hit));
      break;
    }
    const unsigned long long any = __ballot(k);
    if (any) pick = (int)(c + 63 - __builtin_clzll(any));  // the last kept token so far
    run += __shfl(upto, 63, 64);
  }
  if (lane == 0) out[r] = pick;
}

extern "C" int ix_sample(const float* logits, int32_t* out, const float* temperature, const float* top_p,
                         const int32_t* top_k, const float* min_p, const uint64_t* rng_key,
                         uint64_t* rng_counter, int advance, int64_t rows, int64_t vocab, hipStream_t stream) {
  IX_REQUIRE(rows >= 0 && vocab > 0 && vocab < (1ll << 31), "sizes must be positive");
  if (rows == 0) return 0;
  hipLaunchKernelGGL(sample_kernel, dim3(rows), dim3(SAMPLE_THREADS), 0, stream, logits, out, temperature, top_p,
                     top_k, min_p, rng_key, rng_counter, advance, vocab);
  return ix_check_launch("ix_sample");
}

// ---------------------------------------------------------------------------
// Penalties and masks on the logits, before selection (reference:
// ApplyPenaltiesKernel layers.cu:1310-1345; host_sampling.cc:21-48).  Row r's
// history is ids[hist_begin[r] .. hist_begin[r+1]) with counts; for each id:
//   v = v > 0 ? v / repetition : v * repetition;  v -= presence;  v -= frequency * count
// and its masked ids mask_ids[mask_begin[r] .. mask_begin[r+1]) are set to -inf.
__global__ void penalties_kernel(float* __restrict__ logits, const int32_t* __restrict__ hist_begin,
                                 const int32_t* __restrict__ hist_ids, const int32_t* __restrict__ hist_counts,
                                 const float* __restrict__ presence, const float* __restrict__ frequency,
                                 const float* __restrict__ repetition, const int32_t* __restrict__ mask_begin,
                                 const int32_t* __restrict__ mask_ids, int64_t vocab) {
  const int r = blockIdx.x;
  float* row = logits + static_cast<int64_t>(r) * vocab;
  const float rep = repetition[r], pres = presence[r], freq = frequency[r];
  for (int i = hist_begin[r] + threadIdx.x; i < hist_begin[r + 1]; i += blockDim.x) {
    const int id = hist_ids[i];  // ids are distinct within a row
    if (id < 0 || id >= vocab) continue;
    float v = row[id];
    if (rep != 1.0f) v = v > 0.f ? v / rep : v * rep;
    v -= pres;
    v -= freq * static_cast<float>(hist_counts[i]);
    row[id] = v;
  }
  __syncthreads();
  for (int i = mask_begin[r] + threadIdx.x; i < mask_begin[r + 1]; i += blockDim.x) {
    const int id = mask_ids[i];
    if (id >= 0 && id < vocab) row[id] = -INFINITY;
  }
}

extern "C" int ix_apply_penalties(float* logits, const int32_t* hist_begin, const int32_t* hist_ids,
                                  const int32_t* hist_counts, const float* presence, const float* frequency,
                                  const float* repetition, const int32_t* mask_begin, const int32_t* mask_ids,
                                  int64_t rows, int64_t vocab, hipStream_t stream) {
  IX_REQUIRE(rows >= 0 && vocab > 0, "sizes must be positive");
  if (rows == 0) return 0;
  hipLaunchKernelGGL(penalties_kernel, dim3(rows), dim3(256), 0, stream, logits, hist_begin, hist_ids, hist_counts,
                     presence, frequency, repetition, mask_begin, mask_ids, vocab);
  return ix_check_launch("ix_apply_penalties");
}

// ---------------------------------------------------------------------------
// Greedy choice over a large vocabulary in two stages, so that a handful of rows still fills the machine:
// every workgroup finds the first maximum of one chunk of one row, a second kernel picks among the chunks
// (chunks ascend, ties go to the lower index: the result equals ix_argmax's).
#define ARGMAX_CHUNK 4096
__global__ void __launch_bounds__(256)
argmax_chunks_kernel(const float* __restrict__ logits, float* __restrict__ part_v, int32_t* __restrict__ part_i,
                     int64_t vocab, int chunks) {
  __shared__ ArgPair red[16];
  const int64_t r = blockIdx.x;
  const int c = blockIdx.y;
  const float* row = logits + r * vocab;
  const int64_t b = static_cast<int64_t>(c) * ARGMAX_CHUNK, e = min<int64_t>(b + ARGMAX_CHUNK, vocab);
  ArgPair p{-INFINITY, 0x7fffffff};
  for (int64_t i = b + threadIdx.x; i < e; i += blockDim.x) {
    const float v = row[i];
    if (v > p.v) { p.v = v; p.i = (int)i; }
  }
  p = block_argmax(p, red);
  if (threadIdx.x == 0) {
    part_v[r * chunks + c] = p.v;
    part_i[r * chunks + c] = p.i;
  }
}

__global__ void __launch_bounds__(256)
argmax_final_kernel(const float* __restrict__ part_v, const int32_t* __restrict__ part_i, int32_t* __restrict__ out,
                    int64_t vocab, int chunks) {
  __shared__ ArgPair red[16];
  const int64_t r = blockIdx.x;
  ArgPair p{-INFINITY, 0x7fffffff};
  for (int c = threadIdx.x; c < chunks; c += blockDim.x) {
    ArgPair o{part_v[r * chunks + c], part_i[r * chunks + c]};
    p = better(p, o);
  }
  p = block_argmax(p, red);
  if (threadIdx.x == 0) out[r] = (p.i >= 0 && p.i < vocab) ? p.i : 0;
}

// part_v / part_i: scratch with rows * ceil(vocab / 4096) entries each.
extern "C" int ix_argmax_two_stage(const float* logits, int32_t* out, float* part_v, int32_t* part_i, int64_t rows,
                                   int64_t vocab, hipStream_t stream) {
  IX_REQUIRE(rows >= 0 && vocab > 0 && vocab < (1ll << 31), "sizes must be positive");
  if (rows == 0) return 0;
  const int chunks = static_cast<int>((vocab + ARGMAX_CHUNK - 1) / ARGMAX_CHUNK);
  IX_REQUIRE(chunks <= 65535, "vocabulary too large");
  hipLaunchKernelGGL(argmax_chunks_kernel, dim3(rows, chunks), dim3(256), 0, stream, logits, part_v, part_i, vocab,
                     chunks);
  hipLaunchKernelGGL(argmax_final_kernel, dim3(rows), dim3(256), 0, stream, part_v, part_i, out, vocab, chunks);
  return ix_check_launch("ix_argmax_two_stage");
}

// ---------------------------------------------------------------------------
// Log-probabilities of the chosen token and of the `n_top` most probable ones, from the logits as they
// were sampled from (after penalties and masks): logprob_i = l_i - (max + log sum exp(l - max))
// (reference: ComputeLogprobsKernel layers.cu:1351-1458; host_sampling.cc:113-141; ties by lower index).
#define LOGPROB_MAX_TOP 20
__global__ void __launch_bounds__(SAMPLE_THREADS)
logprobs_kernel(const float* __restrict__ logits, const int32_t* __restrict__ chosen, float* __restrict__ chosen_lp,
                int32_t* __restrict__ top_ids, float* __restrict__ top_lp, int64_t vocab, int n_top) {
  __shared__ ArgPair ared[16];
  __shared__ float red[16];
  __shared__ int32_t taken[LOGPROB_MAX_TOP];
  const int r = blockIdx.x, tid = threadIdx.x;
  const float* row = logits + static_cast<int64_t>(r) * vocab;
  float mx = -INFINITY;
  for (int64_t i = tid; i < vocab; i += SAMPLE_THREADS) mx = fmaxf(mx, row[i]);
  mx = ix_block_max(mx, red);
  float s = 0.f;
  for (int64_t i = tid; i < vocab; i += SAMPLE_THREADS) s += expf(row[i] - mx);
  s = ix_block_sum(s, red);
  const float log_z = mx + logf(s);
  if (tid == 0) chosen_lp[r] = row[chosen[r]] - log_z;
  for (int n = 0; n < n_top; ++n) {
    ArgPair p{-INFINITY, 0x7fffffff};
    for (int64_t i = tid; i < vocab; i += SAMPLE_THREADS) {
      bool used = false;
      for (int j = 0; j < n; ++j) used |= (taken[j] == (int)i);
      const float v = row[i];
      if (!used && v > p.v) { p.v = v; p.i = (int)i; }
    }
    p = block_argmax(p, ared);
    if (tid == 0) {
      const int id = (p.i >= 0 && p.i < vocab) ? p.i : 0;
      taken[n] = id;
      top_ids[r * n_top + n] = id;
      top_lp[r * n_top + n] = row[id] - log_z;
    }
    __syncthreads();
  }
}

extern "C" int ix_logprobs(const float* logits, const int32_t* chosen, float* chosen_lp, int32_t* top_ids,
                           float* top_lp, int64_t rows, int64_t vocab, int n_top, hipStream_t stream) {
  IX_REQUIRE(rows >= 0 && vocab > 0 && vocab < (1ll << 31), "sizes must be positive");
  IX_REQUIRE(n_top >= 0 && n_top <= LOGPROB_MAX_TOP && n_top <= vocab, "at most 20 top log-probabilities");
  if (rows == 0) return 0;
  hipLaunchKernelGGL(logprobs_kernel, dim3(rows), dim3(SAMPLE_THREADS), 0, stream, logits, chosen, chosen_lp, top_ids,
                     top_lp, vocab, n_top);
  return ix_check_launch("ix_logprobs");
}
