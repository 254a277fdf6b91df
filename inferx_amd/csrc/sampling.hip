// Token selection on float32 logits [rows, vocab]: greedy, and temperature
// sampling with optional top-k / top-p / min-p cut-offs.
//
// Order of operations follows the reference's host sampler
// (src/engine/host_sampling.cc:50-110): temperature, softmax, cut-offs, one
// uniform draw scaled by the kept mass, walk of the cumulative sum.  Cut-offs
// are found as probability thresholds by bisection, the reference's device
// variant (layers.cu:1142-1302), so tokens tied at a threshold stay together.
// The walk is in index order, which samples the same truncated distribution.
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
__global__ void __launch_bounds__(SAMPLE_THREADS)
sample_kernel(const float* __restrict__ logits, int32_t* __restrict__ out, const float* __restrict__ temperature,
              const float* __restrict__ top_p, const int32_t* __restrict__ top_k, const float* __restrict__ min_p,
              const uint64_t* __restrict__ rng_key, const uint64_t* __restrict__ rng_counter, int64_t vocab) {
  __shared__ ArgPair ared[16];
  __shared__ float red[16];
  __shared__ float seg[SAMPLE_THREADS];
  const int r = blockIdx.x, tid = threadIdx.x;
  const float* row = logits + static_cast<int64_t>(r) * vocab;
  const float temp = temperature[r];

  ArgPair best{-INFINITY, 0x7fffffff};
  for (int64_t i = tid; i < vocab; i += SAMPLE_THREADS) {
    const float v = row[i];
    if (v > best.v) { best.v = v; best.i = (int)i; }
  }
  best = block_argmax(best, ared);
  if (best.i < 0 || best.i >= vocab) best.i = 0;
  if (temp <= 0.f) {
    if (tid == 0) out[r] = best.i;
    return;
  }
  const float inv_t = 1.0f / temp;
  const float mx = best.v * inv_t;
  // p_i = exp(l_i / t - max) in (0, 1], p_max = 1; total = sum p_i
  float s = 0.f;
  for (int64_t i = tid; i < vocab; i += SAMPLE_THREADS) s += expf(row[i] * inv_t - mx);
  const float total = ix_block_sum(s, red);

  // threshold on p: keep p >= thr
  float thr = 0.f;
  const float mp = min_p[r];
  if (mp > 0.f) thr = fmaxf(thr, fminf(mp, 1.0f));
  const int kk = top_k[r];
  if (kk > 0 && kk < vocab) {
    // largest threshold that still keeps at least kk tokens
    float lo = 0.f, hi = 1.0f;  // count(p >= lo) >= kk always; p_max = 1
    for (int it = 0; it < 32; ++it) {
      const float mid = 0.5f * (lo + hi);
      float c = 0.f;
      for (int64_t i = tid; i < vocab; i += SAMPLE_THREADS) c += (expf(row[i] * inv_t - mx) >= mid) ? 1.f : 0.f;
      c = ix_block_sum(c, red);
      if (c >= (float)kk) lo = mid; else hi = mid;
    }
    thr = fmaxf(thr, lo);
  }
  const float tp = top_p[r];
  if (tp < 1.0f) {
    // largest threshold whose kept mass still reaches top_p
    float lo = 0.f, hi = 1.0f;
    for (int it = 0; it < 32; ++it) {
      const float mid = 0.5f * (lo + hi);
      float msum = 0.f;
      for (int64_t i = tid; i < vocab; i += SAMPLE_THREADS) {
        const float p = expf(row[i] * inv_t - mx);
        msum += (p >= mid) ? p : 0.f;
      }
      msum = ix_block_sum(msum, red);
      if (msum >= tp * total) lo = mid; else hi = mid;
    }
    thr = fmaxf(thr, lo);
  }
  thr = fminf(thr, 1.0f);  // the most probable token always stays

  // contiguous segment per thread, kept mass per segment
  const int64_t per = (vocab + SAMPLE_THREADS - 1) / SAMPLE_THREADS;
  const int64_t b = min<int64_t>(tid * per, vocab), e = min<int64_t>(b + per, vocab);
  float mine = 0.f;
  for (int64_t i = b; i < e; ++i) {
    const float p = expf(row[i] * inv_t - mx);
    mine += (p >= thr) ? p : 0.f;
  }
  seg[tid] = mine;
  __syncthreads();
  if (tid == 0) {
    float mass = 0.f;
    for (int i = 0; i < SAMPLE_THREADS; ++i) mass += seg[i];
    const float target = uniform_from(rng_key[r], rng_counter[r]) * mass;
    float run = 0.f;
    int s_idx = 0;
    for (; s_idx < SAMPLE_THREADS - 1; ++s_idx) {
      if (run + seg[s_idx] > target) break;
      run += seg[s_idx];
    }
    // walk the chosen segment; fall back to the most probable token
    const int64_t sb = min<int64_t>((int64_t)s_idx * per, vocab), se = min<int64_t>(sb + per, vocab);
    int pick = best.i;
    for (int64_t i = sb; i < se; ++i) {
      const float p = expf(row[i] * inv_t - mx);
      if (p >= thr) {
        run += p;
        pick = (int)i;
        if (run > target) break;
      }
    }
    out[r] = pick;
  }
}

extern "C" int ix_sample(const float* logits, int32_t* out, const float* temperature, const float* top_p,
                         const int32_t* top_k, const float* min_p, const uint64_t* rng_key,
                         const uint64_t* rng_counter, int64_t rows, int64_t vocab, hipStream_t stream) {
  IX_REQUIRE(rows >= 0 && vocab > 0 && vocab < (1ll << 31), "sizes must be positive");
  if (rows == 0) return 0;
  hipLaunchKernelGGL(sample_kernel, dim3(rows), dim3(SAMPLE_THREADS), 0, stream, logits, out, temperature, top_p,
                     top_k, min_p, rng_key, rng_counter, vocab);
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
