// Two probes of the machine the engine runs on: what a kernel that does nothing but read memory gets out of
// HBM, and what a kernel that does nothing but matrix-core products gets out of the matrix cores.  The
// benchmark prices its results against these measured ceilings beside the published ones.  (The reference's
// benchmark notes ask for both, docs/ARCHITECTURE.md:595-603; it has no such kernels itself.)
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

// Every workgroup reads its share of `n16` 16-byte pieces, sixteen loads in flight per thread, pieces of a
// wavefront side by side; what it read is folded into one number per workgroup so that no load can be dropped.
__global__ void __launch_bounds__(256) probe_read_kernel(const u32x4* __restrict__ src, int64_t n16,
                                                         unsigned int* __restrict__ out) {
  constexpr int UNROLL = 16;
  const int64_t per_block = (n16 + gridDim.x - 1) / gridDim.x;
  const int64_t begin = per_block * blockIdx.x, end = min(n16, begin + per_block);
  u32x4 acc = {0u, 0u, 0u, 0u};
  int64_t i = begin + threadIdx.x;
  for (; i + static_cast<int64_t>(UNROLL - 1) * 256 < end; i += static_cast<int64_t>(UNROLL) * 256) {
    u32x4 v[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) v[u] = __builtin_nontemporal_load(src + i + static_cast<int64_t>(u) * 256);
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) acc ^= v[u];
  }
  for (; i < end; i += 256) acc ^= src[i];
  unsigned int folded = acc[0] ^ acc[1] ^ acc[2] ^ acc[3];
  folded ^= __shfl_xor(folded, 32, 64);
  folded ^= __shfl_xor(folded, 16, 64);
  if ((threadIdx.x & 15) == 0) atomicXor(out + (blockIdx.x & 1023), folded);
}

// Every wavefront issues `iters` rounds of four independent v_mfma_f32_32x32x16_bf16 on operands it keeps in
// registers: 4 * 32 * 32 * 16 * 2 flops per round and wavefront.  (This is the shape that reaches the published
// rate on MI355X, 2.46 PFLOP/s measured with two wavefronts per SIMD; v_mfma_f32_16x16x32_bf16 measured 1.3 to 1.44.)
typedef float f32x16 __attribute__((ext_vector_type(16)));
__global__ void __launch_bounds__(256) probe_mfma_kernel(int iters, float* __restrict__ out) {
  bf16x8 a, b;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    a[j] = (__bf16)(0.001f * static_cast<float>((threadIdx.x + j) & 7));
    b[j] = (__bf16)(0.002f * static_cast<float>((threadIdx.x * 3 + j) & 7));
  }
  f32x16 acc[4];
#pragma unroll
  for (int u = 0; u < 4; ++u)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[u][i] = 0.f;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int u = 0; u < 4; ++u) acc[u] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[u], 0, 0, 0);
  }
  float s = 0.f;
#pragma unroll
  for (int u = 0; u < 4; ++u) s += acc[u][0] + acc[u][5] + acc[u][10] + acc[u][15];
  if (s == 12345.678f) out[0] = s;  // never true: keeps the products alive
}

// Queues `repeats` passes over `bytes` of device memory at `src` (a multiple of 16, and large beside every cache:
// gigabytes).  `out`: 1024 uint32 of scratch.
extern "C" int ix_probe_read(const void* src, int64_t bytes, void* out, int blocks, int repeats, hipStream_t stream) {
  IX_REQUIRE(src && out && bytes >= 16 && bytes % 16 == 0, "a buffer of a multiple of 16 bytes is needed");
  IX_REQUIRE(blocks > 0 && blocks <= (1 << 20) && repeats > 0, "blocks and repeats must be positive");
  for (int r = 0; r < repeats; ++r)
    hipLaunchKernelGGL(probe_read_kernel, dim3(blocks), dim3(256), 0, stream, static_cast<const u32x4*>(src),
                       bytes / 16, static_cast<unsigned int*>(out));
  return ix_check_launch("ix_probe_read");
}

// Queues one launch of `blocks` workgroups of four wavefronts, `iters` rounds each; returns the flops it does
// through `flops` (host memory).  `out`: one float of scratch.
extern "C" int ix_probe_mfma(int blocks, int iters, float* out, double* flops, hipStream_t stream) {
  IX_REQUIRE(out && flops && blocks > 0 && blocks <= (1 << 20) && iters > 0, "sizes must be positive");
  hipLaunchKernelGGL(probe_mfma_kernel, dim3(blocks), dim3(256), 0, stream, iters, out);
  *flops = static_cast<double>(blocks) * 4.0 * iters * 4.0 * (32.0 * 32.0 * 16.0 * 2.0);
  return ix_check_launch("ix_probe_mfma");
}
