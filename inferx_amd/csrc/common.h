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

// Sum / maximum over the 64 lanes, result in every lane.  Within a row of 16 lanes the partners come through
// DPP (lanes ^1, ^2, then the half row and the row mirrored: no LDS round trip), across rows through two
// exchanges.  The order of the additions is fixed.
template <int CTRL>
__device__ __forceinline__ float ix_dpp(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
template <int CTRL>
__device__ __forceinline__ int ix_dpp(int v) {
  return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xf, 0xf, true);
}
#define IX_DPP_XOR1 0xB1         // quad_perm [1, 0, 3, 2]
#define IX_DPP_XOR2 0x4E         // quad_perm [2, 3, 0, 1]
#define IX_DPP_HALF_MIRROR 0x141  // lane i of 8 <-> lane 7 - i
#define IX_DPP_MIRROR 0x140       // lane i of 16 <-> lane 15 - i

__device__ __forceinline__ float ix_wave_sum(float v) {
  v += ix_dpp<IX_DPP_XOR1>(v);
  v += ix_dpp<IX_DPP_XOR2>(v);
  v += ix_dpp<IX_DPP_HALF_MIRROR>(v);
  v += ix_dpp<IX_DPP_MIRROR>(v);
  v += __shfl_xor(v, 16, IX_WAVE);
  v += __shfl_xor(v, 32, IX_WAVE);
  return v;
}

__device__ __forceinline__ float ix_wave_max(float v) {
  v = fmaxf(v, ix_dpp<IX_DPP_XOR1>(v));
  v = fmaxf(v, ix_dpp<IX_DPP_XOR2>(v));
  v = fmaxf(v, ix_dpp<IX_DPP_HALF_MIRROR>(v));
  v = fmaxf(v, ix_dpp<IX_DPP_MIRROR>(v));
  v = fmaxf(v, __shfl_xor(v, 16, IX_WAVE));
  v = fmaxf(v, __shfl_xor(v, 32, IX_WAVE));
  return v;
}

// The largest value over the 64 lanes and, among equals, the smallest index that comes with it; in every lane.
__device__ __forceinline__ void ix_wave_argmax(float& v, int& idx) {
#define IX_ARGMAX_STEP(OV, OI)                               \
  {                                                          \
    const float ov = (OV);                                   \
    const int oi = (OI);                                     \
    if (ov > v || (ov == v && oi < idx)) {                   \
      v = ov;                                                \
      idx = oi;                                              \
    }                                                        \
  }
  IX_ARGMAX_STEP(ix_dpp<IX_DPP_XOR1>(v), ix_dpp<IX_DPP_XOR1>(idx))
  IX_ARGMAX_STEP(ix_dpp<IX_DPP_XOR2>(v), ix_dpp<IX_DPP_XOR2>(idx))
  IX_ARGMAX_STEP(ix_dpp<IX_DPP_HALF_MIRROR>(v), ix_dpp<IX_DPP_HALF_MIRROR>(idx))
  IX_ARGMAX_STEP(ix_dpp<IX_DPP_MIRROR>(v), ix_dpp<IX_DPP_MIRROR>(idx))
  IX_ARGMAX_STEP(__shfl_xor(v, 16, IX_WAVE), __shfl_xor(idx, 16, IX_WAVE))
  IX_ARGMAX_STEP(__shfl_xor(v, 32, IX_WAVE), __shfl_xor(idx, 32, IX_WAVE))
#undef IX_ARGMAX_STEP
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
// out[t, h, :] from the parts that kernels which cut keys into slices leave (attention_mfma.hip)
int ix_attention_combine(const float* part_o, const float* part_ml, void* out, int64_t tokens, int heads,
                         int n_splits, int head_dim, hipStream_t stream);
int ix_check_launch(const char* what);
#define IX_REQUIRE(cond, msg)                          \
  do {                                                 \
    if (!(cond)) {                                     \
      ix_set_error(std::string(__func__) + ": " + msg); \
      return 1;                                        \
    }                                                  \
  } while (0)
