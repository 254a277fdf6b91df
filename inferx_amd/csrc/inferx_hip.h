// Entry points of libinferx_hip.so that callers outside the Python face may want to link against or load by
// name.  Every entry point returns 0 on success; otherwise `ix_last_error()` holds the reason for the calling
// thread.  All pointers are device pointers on the current device unless said otherwise; work is queued on
// `stream` and the call returns without waiting for it.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

const char* ix_last_error();
int ix_abi_version();

// Paged attention on the matrix cores (bfloat16), keys cut into `n_splits` slices per query tile.
//   q, out        [tokens, heads, head_dim]
//   k_cache       [pages, kv_heads, page_size, head_dim]
//   v_cache       [pages, kv_heads, head_dim, page_size]  (transposed within a page)
//   block_table   int32 [requests, max_blocks]
//   tile_seq / tile_q0 / tile_rows   int32 [n_tiles]: request, first token row, rows (<= tile_queries) of a tile
//   positions     int32 [tokens]
//   part_o        float32 [tokens * heads * n_splits * head_dim], part_ml float32 [tokens * heads * n_splits * 2]:
//                 the slices' partial results, needed when n_splits > 1 (the caller's workspace)
int ix_attention_mfma(const void* q, const void* k_cache, const void* v_cache, const int32_t* block_table,
                      const int32_t* tile_seq, const int32_t* tile_q0, const int32_t* tile_rows,
                      const int32_t* positions, void* out, float* part_o, float* part_ml, int64_t tokens, int n_tiles,
                      int tile_queries, int n_splits, int heads, int kv_heads, int head_dim, int page_size,
                      int max_blocks, float scale, int window, int prefetch, int grouped, hipStream_t stream);

// The same operation for callers that cannot allocate device memory: code under HIP graph capture, tight
// serving loops that must not call hipMalloc, harnesses that forbid it.  It has no counterpart in the reference,
// whose attention kernels take their workspace from the caller's allocator.
//
// The slices' partial results go to a buffer that lives inside the library, IX_ATTENTION_SCRATCH_BYTES per
// device, held from the library's load until the process ends.  The call allocates and frees nothing.  It
// refuses (returns 1, with a message) when tokens * heads * n_splits * (head_dim + 2) floats do not fit.
//
// All calls on one device share that buffer, which keeps the last call's contents: two calls whose work overlaps
// on one device (different streams, or different threads on different streams) race and give wrong results;
// calls queued on one stream are safe.  Nothing in the buffer has to start at zero: every slice of every tile
// writes its part before the combining pass reads it.  Token rows that no tile covers are combined from whatever
// the buffer held, as they are from an uninitialised workspace in `ix_attention_mfma`.
//
// The first call on a device looks the buffer's address up once (not to be made while a graph is captured);
// later calls on that device only launch.
#define IX_ATTENTION_SCRATCH_BYTES (16 << 20)
int ix_attention_mfma_noalloc(const void* q, const void* k_cache, const void* v_cache, const int32_t* block_table,
                              const int32_t* tile_seq, const int32_t* tile_q0, const int32_t* tile_rows,
                              const int32_t* positions, void* out, int64_t tokens, int n_tiles, int tile_queries,
                              int n_splits, int heads, int kv_heads, int head_dim, int page_size, int max_blocks,
                              float scale, int window, int prefetch, int grouped, hipStream_t stream);

#ifdef __cplusplus
}
#endif
