// Paged attention, the plain kernel: one workgroup per (query token, query
// head), keys taken through the request's block table, softmax kept online in
// float32 over chunks of 256 keys.  It serves every element type, head size and
// page size; the float32 run uses it throughout, the bfloat16 run where the
// matrix-core kernels do not take a shape.
//
// A query at position p reads keys [start, p], start = 0 or, with a window W,
// max(0, p + 1 - W) (reference: PagedAttentionWithLseKernel, layers.cu:329-407;
// window rule :346-354).  Query head h reads kv head h / (heads / kv_heads).
// Key j of a request lives in page table[j / page_size] at offset j % page_size;
// keys are stored [page][kv_head][offset][d], values [page][kv_head][d][offset].
#include "common.h"

#define ATTN_PLAIN_THREADS 256

template <typename T>
__global__ void __launch_bounds__(ATTN_PLAIN_THREADS)
attn_plain_kernel(const T* __restrict__ q, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
                  const int32_t* __restrict__ block_table, const int32_t* __restrict__ seq_of_token,
                  const int32_t* __restrict__ positions, T* __restrict__ out, int heads, int kv_heads, int head_dim,
                  int page_size, int max_blocks, float scale, int window) {
  __shared__ float qs[256];
  __shared__ float sc[ATTN_PLAIN_THREADS];
  __shared__ int32_t pg[ATTN_PLAIN_THREADS];
  __shared__ float red[16];

  const int64_t t = blockIdx.x;
  const int head = blockIdx.y;
  const int g = head / (heads / kv_heads);
  const int tid = threadIdx.x;
  const int64_t seq = seq_of_token[t];
  const int pos = positions[t];
  const int start = (window > 0 && pos + 1 > window) ? pos + 1 - window : 0;
  const int32_t* table = block_table + seq * max_blocks;

  if (tid < head_dim) qs[tid] = ix_load(q + (t * heads + head) * head_dim + tid);
  __syncthreads();

  float m = -INFINITY, l = 0.f, acc = 0.f;
  for (int base = start; base <= pos; base += ATTN_PLAIN_THREADS) {
    const int j = base + tid;
    const bool live = j <= pos;
    float s = -INFINITY;
    int32_t page = 0;
    if (live) {
      page = table[j / page_size];
      const T* kr = k_cache + ((static_cast<int64_t>(page) * kv_heads + g) * page_size + j % page_size) * head_dim;
      float dot = 0.f;
      for (int i = 0; i < head_dim; ++i) dot += qs[i] * ix_load(kr + i);
      s = dot * scale;
    }
    pg[tid] = page;
    const float m_new = fmaxf(m, ix_block_max(s, red));
    const float p = live ? expf(s - m_new) : 0.f;
    sc[tid] = p;
    const float chunk_sum = ix_block_sum(p, red);  // has the barriers that publish sc and pg
    const float alpha = expf(m - m_new);           // exp(-inf) = 0 on the first chunk
    l = l * alpha + chunk_sum;
    m = m_new;
    if (tid < head_dim) {
      acc *= alpha;
      const int n = min(ATTN_PLAIN_THREADS, pos + 1 - base);
      for (int jj = 0; jj < n; ++jj) {
        const int key = base + jj;
        const T* vr =
            v_cache + ((static_cast<int64_t>(pg[jj]) * kv_heads + g) * head_dim + tid) * page_size + key % page_size;
        acc += sc[jj] * ix_load(vr);
      }
    }
    __syncthreads();
  }
  if (tid < head_dim) ix_store(out + (t * heads + head) * head_dim + tid, acc / l);
}

extern "C" int ix_attention_plain(const void* q, const void* k_cache, const void* v_cache, int dtype,
                                  const int32_t* block_table, const int32_t* seq_of_token, const int32_t* positions,
                                  void* out, int64_t tokens, int heads, int kv_heads, int head_dim, int page_size,
                                  int max_blocks, float scale, int window, hipStream_t stream) {
  IX_REQUIRE(tokens >= 0 && heads > 0 && kv_heads > 0 && page_size > 0 && max_blocks > 0, "sizes must be positive");
  IX_REQUIRE(heads % kv_heads == 0, "heads must be a multiple of kv_heads");
  IX_REQUIRE(head_dim > 0 && head_dim <= 256, "head_dim must be between 1 and 256");
  IX_REQUIRE(window >= 0, "window must not be negative");
  if (tokens == 0) return 0;
  dim3 grid(tokens, heads), block(ATTN_PLAIN_THREADS);
  if (dtype == IX_F32)
    hipLaunchKernelGGL(attn_plain_kernel<float>, grid, block, 0, stream, (const float*)q, (const float*)k_cache,
                       (const float*)v_cache, block_table, seq_of_token, positions, (float*)out, heads, kv_heads,
                       head_dim, page_size, max_blocks, scale, window);
  else if (dtype == IX_BF16)
    hipLaunchKernelGGL(attn_plain_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)q, (const bf16_t*)k_cache,
                       (const bf16_t*)v_cache, block_table, seq_of_token, positions, (bf16_t*)out, heads, kv_heads,
                       head_dim, page_size, max_blocks, scale, window);
  else
    IX_REQUIRE(false, "dtype must be float32 or bfloat16");
  return ix_check_launch("ix_attention_plain");
}
