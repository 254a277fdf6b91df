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

// bfloat16 with a width that is a multiple of 4: four columns per thread (8-byte loads of the experts' rows,
// 16-byte ones of the residual stream); the same additions in the same order as above.
__device__ __forceinline__ void bf16x4_to_f32(uint2 p, float (&f)[4]) {
  f[0] = __uint_as_float(p.x << 16);
  f[1] = __uint_as_float(p.x & 0xffff0000u);
  f[2] = __uint_as_float(p.y << 16);
  f[3] = __uint_as_float(p.y & 0xffff0000u);
}

__global__ void moe_combine_add_rmsnorm_vec4_kernel(float* __restrict__ h, const uint16_t* __restrict__ y,
                                                    const int32_t* __restrict__ dest,
                                                    const float* __restrict__ topk_w,
                                                    const uint16_t* __restrict__ shared,
                                                    const float* __restrict__ shared_gate, const void* __restrict__ w,
                                                    int w_dtype, uint16_t* __restrict__ out,
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
  for (int64_t c = 4 * threadIdx.x; c < width; c += 4 * blockDim.x) {
    float acc[4] = {0.f, 0.f, 0.f, 0.f}, f[4];
    for (int s = 0; s < k; ++s) {
      bf16x4_to_f32(*reinterpret_cast<const uint2*>(y + static_cast<int64_t>(sd[s]) * width + c), f);
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[i] += sw[s] * f[i];
    }
    if (shared) {
      bf16x4_to_f32(*reinterpret_cast<const uint2*>(shared + row * width + c), f);
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[i] += sg * f[i];
    }
    float4 v = *reinterpret_cast<const float4*>(hr + c);
    v.x += acc[0]; v.y += acc[1]; v.z += acc[2]; v.w += acc[3];
    if (!rows) *reinterpret_cast<float4*>(hr + c) = v;
    *reinterpret_cast<float4*>(vrow + c) = v;
    sumsq += v.x * v.x;
    sumsq += v.y * v.y;
    sumsq += v.z * v.z;
    sumsq += v.w * v.w;
  }
  sumsq = ix_block_sum(sumsq, red);
  const float inv = 1.0f / sqrtf(sumsq / static_cast<float>(width) + eps);
  uint16_t* outr = out + r * width;
  for (int64_t c = 4 * threadIdx.x; c < width; c += 4 * blockDim.x) {
    const float4 v = *reinterpret_cast<const float4*>(vrow + c);
    uint2 o;
    o.x = ix_f32_to_bf16(v.x * inv * ix_load_rt(w, w_dtype, c)) |
          static_cast<uint32_t>(ix_f32_to_bf16(v.y * inv * ix_load_rt(w, w_dtype, c + 1))) << 16;
    o.y = ix_f32_to_bf16(v.z * inv * ix_load_rt(w, w_dtype, c + 2)) |
          static_cast<uint32_t>(ix_f32_to_bf16(v.w * inv * ix_load_rt(w, w_dtype, c + 3))) << 16;
    *reinterpret_cast<uint2*>(outr + c) = o;
  }
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
  else if (dtype == IX_BF16 && width % 4 == 0 &&
           ((reinterpret_cast<uintptr_t>(h) | reinterpret_cast<uintptr_t>(y) | reinterpret_cast<uintptr_t>(shared) |
             reinterpret_cast<uintptr_t>(out)) & 15) == 0)
    hipLaunchKernelGGL(moe_combine_add_rmsnorm_vec4_kernel, grid, dim3(width >= 4096 ? 1024 : (width >= 2048 ? 512 : 256)),
                       smem, stream, (float*)h, (const uint16_t*)y, dest, topk_w, (const uint16_t*)shared, shared_gate, w,
                       w_dtype, (uint16_t*)out, rows, width, k, eps);
  else if (dtype == IX_BF16)
    hipLaunchKernelGGL(moe_combine_add_rmsnorm_kernel<bf16_t>, grid, block, smem, stream, (float*)h,
                       (const bf16_t*)y, dest, topk_w, (const bf16_t*)shared, shared_gate, w, w_dtype, (bf16_t*)out,
                       rows, width, k, eps);
  else
    IX_REQUIRE(false, "dtype must be float32 or bfloat16");
  return ix_check_launch("ix_moe_combine_add_rmsnorm");
}
