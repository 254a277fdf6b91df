// Shared helpers for the gfx950 kernels: element types, conversions, wave and
// block reductions, error reporting.  Wavefronts are 64 lanes wide everywhere.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#define IX_WAVE 64

// dtype codes shared with the Python side
enum IxDtype { IX_F32 = 0, IX_BF16 = 1 };

struct bf16_t {
  uint16_t bits;
};

__device__ __forceinline__ float ix_bf16_to_f32(uint16_t b) {
  return __uint_as_float(static_cast<uint32_t>(b) << 16);
}

// round to nearest even; NaN stays NaN
__device__ __forceinline__ uint16_t ix_f32_to_bf16(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return static_cast<uint16_t>((u >> 16) | 0x40u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return static_cast<uint16_t>(u >> 16);
}

__device__ __forceinline__ float ix_load(const float* p) { return *p; }
__device__ __forceinline__ float ix_load(const bf16_t* p) { return ix_bf16_to_f32(p->bits); }
__device__ __forceinline__ void ix_store(float* p, float v) { *p = v; }
__device__ __forceinline__ void ix_store(bf16_t* p, float v) { p->bits = ix_f32_to_bf16(v); }

// element `i` of an array whose type is only known at run time (small tensors:
// norm weights, biases, router rows)
__device__ __forceinline__ float ix_load_rt(const void* base, int dtype, int64_t i) {
  return dtype == IX_F32 ? static_cast<const float*>(base)[i]
                         : ix_bf16_to_f32(static_cast<const uint16_t*>(base)[i]);
}

__device__ __forceinline__ float ix_wave_sum(float v) {
#pragma unroll
  for (int off = IX_WAVE / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, IX_WAVE);
  return v;
}

__device__ __forceinline__ float ix_wave_max(float v) {
#pragma unroll
  for (int off = IX_WAVE / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, IX_WAVE));
  return v;
}

// Block-wide sum/max, result in every thread.  `red` holds one float per wave
// (at most 16).  The order of additions is fixed, so results repeat bit for bit.
__device__ __forceinline__ float ix_block_sum(float v, float* red) {
  const int lane = threadIdx.x & (IX_WAVE - 1), wave = threadIdx.x / IX_WAVE;
  const int nwaves = (blockDim.x + IX_WAVE - 1) / IX_WAVE;
  v = ix_wave_sum(v);
  __syncthreads();
  if (lane == 0) red[wave] = v;
  __syncthreads();
  float total = 0.f;
  for (int w = 0; w < nwaves; ++w) total += red[w];
  return total;
}

__device__ __forceinline__ float ix_block_max(float v, float* red) {
  const int lane = threadIdx.x & (IX_WAVE - 1), wave = threadIdx.x / IX_WAVE;
  const int nwaves = (blockDim.x + IX_WAVE - 1) / IX_WAVE;
  v = ix_wave_max(v);
  __syncthreads();
  if (lane == 0) red[wave] = v;
  __syncthreads();
  float total = -INFINITY;
  for (int w = 0; w < nwaves; ++w) total = fmaxf(total, red[w]);
  return total;
}

// ---- host side -------------------------------------------------------------
#include <algorithm>
#include <string>
void ix_set_error(const std::string& msg);
int ix_check_launch(const char* what);
#define IX_REQUIRE(cond, msg)                          \
  do {                                                 \
    if (!(cond)) {                                     \
      ix_set_error(std::string(__func__) + ": " + msg); \
      return 1;                                        \
    }                                                  \
  } while (0)
