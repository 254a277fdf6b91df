// The weighted sum of the routed experts' outputs, the shared expert, the
// residual add and the RMSNorm that follows, in one pass over a token's row:
//   v = h[row] + sum_s topk_w[row, s] * y[dest[row, s]] + gate[row] * shared[row]
//   h[row] = v (unless rows are picked);  out = v * rsqrt(mean(v^2) + eps) * w
// Arithmetic and order of additions are those of ix_moe_combine followed by
// ix_add_rmsnorm, except that the feed-forward's sum is not rounded to the
// activations' type before it joins the float32 residual stream.
#include "common.h"

template <typename T>
__global__ void moe_combine_add_rmsnorm_kernel(float* __restrict__ h, const T* __restrict__ y,
                                               const int32_t* __restrict__ dest, const float* __restrict__ topk_w,
                                               const T* __restrict__ shared, const float* __restrict__ shared_gate,
                                               const void* __restrict__ w, int w_dtype, T* __restrict__ out,
                                               const int32_t* __restrict__ rows, int64_t width, int k, float eps) {
  extern __shared__ __align__(16) float vrow[];  // [width]
  __shared__ float red[16];
  __shared__ float sw[32];
  __shared__ int32_t sd[32];
  const int64_t r = blockIdx.x;
  const int64_t row = rows ? rows[r] : r;
  if (threadIdx.x < k) {
    sw[threadIdx.x] = topk_w[row * k + threadIdx.x];
    sd[threadIdx.x] = dest[row * k + threadIdx.x];
  }
  __syncthreads();
  const float sg = shared ? (shared_gate ? shared_gate[row] : 1.0f) : 0.f;
  float* hr = h + row * width;
  float sumsq = 0.f;
  for (int64_t c = threadIdx.x; c < width; c += blockDim.x) {
    float acc = 0.f;
    for (int s = 0; s < k; ++s) acc += sw[s] * ix_load(y + static_cast<int64_t>(sd[s]) * width + c);
    if (shared) acc += sg * ix_load(shared + row * width + c);
    const float v = hr[c] + acc;
    if (!rows) hr[c] = v;
    vrow[c] = v;
    sumsq += v * v;
  }
  sumsq = ix_block_sum(sumsq, red);
  const float inv = 1.0f / sqrtf(sumsq / static_cast<float>(width) + eps);
  T* outr = out + r * width;
  for (int64_t c = threadIdx.x; c < width; c += blockDim.x) ix_store(outr + c, vrow[c] * inv * ix_load_rt(w, w_dtype, c));
}

extern "C" int ix_moe_combine_add_rmsnorm(void* h, const void* y, int dtype, const int32_t* dest,
                                          const float* topk_w, const void* shared, const float* shared_gate,
                                          const void* w, int w_dtype, void* out, const int32_t* rows,
                                          int64_t n_out_rows, int64_t width, int k, float eps, hipStream_t stream) {
  IX_REQUIRE(n_out_rows >= 0 && width > 0, "sizes must be positive");
  IX_REQUIRE(k > 0 && k <= 32, "top_k must be between 1 and 32");
  IX_REQUIRE(width * sizeof(float) <= 60 * 1024, "hidden width too large for the fused kernel (limit 15360)");
  IX_REQUIRE(w_dtype == IX_F32 || w_dtype == IX_BF16, "weight dtype must be float32 or bfloat16");
  if (n_out_rows == 0) return 0;
  dim3 grid(n_out_rows), block(width >= 4096 ? 1024 : (width >= 1024 ? 512 : 256));
  const size_t smem = width * sizeof(float);
  if (dtype == IX_F32)
    hipLaunchKernelGGL(moe_combine_add_rmsnorm_kernel<float>, grid, block, smem, stream, (float*)h, (const float*)y,
                       dest, topk_w, (const float*)shared, shared_gate, w, w_dtype, (float*)out, rows, width, k, eps);
  else if (dtype == IX_BF16)
    hipLaunchKernelGGL(moe_combine_add_rmsnorm_kernel<bf16_t>, grid, block, smem, stream, (float*)h,
                       (const bf16_t*)y, dest, topk_w, (const bf16_t*)shared, shared_gate, w, w_dtype, (bf16_t*)out,
                       rows, width, k, eps);
  else
    IX_REQUIRE(false, "dtype must be float32 or bfloat16");
  return ix_check_launch("ix_moe_combine_add_rmsnorm");
}
