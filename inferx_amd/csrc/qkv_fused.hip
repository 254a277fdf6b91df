// Decoding (at most 32 tokens): the fused q/k/v product with its epilogue in one kernel, bfloat16:
//   qkv = x . Wqkv^T + bias;  rotate q and k (half-split pairs);  q -> q_out,  k, v -> cache pages.
// What moe_mfma.hip's streaming kernel and elementwise.hip's qkv_rope_append do one after the other
// (reference: src/model/qwen2.cc:920-969), with one launch less.
//
// A workgroup owns, for one head, 16 features of the low half and the 16 of the high half that pair
// with them; its four wavefronts split the reduction and add up through LDS in a fixed order.  The
// product is formed transposed (A = weight rows, B = token rows), so lane l ends up with features
// 4*(l/16)+i of token l%16: four consecutive numbers of one output row.  NT: sixteens of tokens (1 or 2); the
// weights are read once for both.
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

template <int NT>
__global__ void __launch_bounds__(256)
qkv_rope_skinny_kernel(const __bf16* x, const __bf16* w, const void* __restrict__ bias,
                       int bias_dtype, const float2* __restrict__ cs, const int32_t* __restrict__ slots,
                       __bf16* __restrict__ q_out, __bf16* __restrict__ k_cache, __bf16* __restrict__ v_cache,
                       int tokens, int width, int heads, int kv_heads, int head_dim, int page_size,
                       int64_t total_slots) {
  __shared__ float red[3 * 64 * 8 * NT];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int m = lane & 15, g = lane >> 4;
  const int half = head_dim / 2, per_head = half / 16;
  const int head = blockIdx.x / per_head, jt = blockIdx.x - head * per_head;
  const int row_lo = head * head_dim + 16 * jt + m;  // weight row (= output feature) of the low half

  const int kper = (((width + 3) / 4) + 127) & ~127;
  const int kbegin = wave * kper, kend = min(width, kbegin + kper);
  const __bf16* wl = w + static_cast<int64_t>(row_lo) * width;
  const __bf16* wh = wl + static_cast<int64_t>(half) * width;
  const __bf16* xr[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) xr[t] = x + static_cast<int64_t>(min(16 * t + m, tokens - 1)) * width;

  const bf16x8 zero = {(__bf16)0.f, (__bf16)0.f, (__bf16)0.f, (__bf16)0.f,
                       (__bf16)0.f, (__bf16)0.f, (__bf16)0.f, (__bf16)0.f};
  f32x4 acc[NT][2];
#pragma unroll
  for (int t = 0; t < NT; ++t) acc[t][0] = acc[t][1] = f32x4{0.f, 0.f, 0.f, 0.f};
  // Steps of 128 of the reduction in two register sets: the loads of the next step are on their way while this
  // one is multiplied.  Every load is unconditional (a piece past the end of a ragged last round is read from
  // the range's first piece instead, and its token values are replaced by zeros when they are used), so that
  // the loop is one straight line and the compiler lets the younger loads stay in flight at each wait.
  struct Step { bf16x8 fl[4], fh[4], fx[NT][4]; };
  Step one, two;
  auto fetch = [&](int k0, Step& st) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      int kk = k0 + 32 * j + 8 * g;  // the four lane groups cover 64 contiguous bytes of a row
      kk = kk < kend ? kk : kbegin;  // (past the end: the range's first piece, which exists and was read before)
      st.fl[j] = *reinterpret_cast<const bf16x8*>(wl + kk);
      st.fh[j] = *reinterpret_cast<const bf16x8*>(wh + kk);
#pragma unroll
      for (int t = 0; t < NT; ++t) st.fx[t][j] = *reinterpret_cast<const bf16x8*>(xr[t] + kk);
    }
  };
  auto multiply = [&](int k0, const Step& st) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const bool ok = k0 + 32 * j + 8 * g < kend;
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        const bf16x8 xv = ok ? st.fx[t][j] : zero;
        acc[t][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(st.fl[j], xv, acc[t][0], 0, 0, 0);
        acc[t][1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(st.fh[j], xv, acc[t][1], 0, 0, 0);
      }
    }
  };
  // What the first wavefront needs after the products is asked for now, so that it is there by then.
  const int j0 = 16 * jt + 4 * g, col = head * head_dim + j0;
  const bool is_v = head >= heads + kv_heads;
  float4 blo = make_float4(0.f, 0.f, 0.f, 0.f), bhi = blo, cs01[NT], cs23[NT];
  uint2 blo16 = make_uint2(0u, 0u), bhi16 = blo16;
  int slot_of[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    cs01[t] = cs23[t] = blo;
    slot_of[t] = -1;
  }
  if (wave == 0) {
    if (bias) {
      if (bias_dtype == IX_BF16) {
        blo16 = *reinterpret_cast<const uint2*>(static_cast<const uint16_t*>(bias) + col);
        bhi16 = *reinterpret_cast<const uint2*>(static_cast<const uint16_t*>(bias) + col + half);
      } else {
        blo = *reinterpret_cast<const float4*>(static_cast<const float*>(bias) + col);
        bhi = *reinterpret_cast<const float4*>(static_cast<const float*>(bias) + col + half);
      }
    }
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      const int tok = 16 * t + m;
      if (tok >= tokens) continue;
      if (!is_v && cs) {
        const float4* c = reinterpret_cast<const float4*>(cs + static_cast<int64_t>(tok) * half + j0);
        cs01[t] = c[0];
        cs23[t] = c[1];
      }
      if (slots) slot_of[t] = slots[tok];
    }
  }
  // rounds in pairs; the loop runs while both rounds of a turn are followed by another one and has no way out of
  // its middle, the last one or two rounds come after it
  const int rounds = kbegin < kend ? (kend - kbegin + 127) >> 7 : 0;
  if (rounds > 0) {
    fetch(kbegin, one);
    int k0 = kbegin, left = rounds;
    for (; left > 2; left -= 2, k0 += 256) {
      fetch(k0 + 128, two);
      __builtin_amdgcn_sched_barrier(0);
      multiply(k0, one);
      __builtin_amdgcn_sched_barrier(0);
      fetch(k0 + 256, one);
      __builtin_amdgcn_sched_barrier(0);
      multiply(k0 + 128, two);
      __builtin_amdgcn_sched_barrier(0);
    }
    if (left == 2) {
      fetch(k0 + 128, two);
      __builtin_amdgcn_sched_barrier(0);
      multiply(k0, one);
      multiply(k0 + 128, two);
    } else {
      multiply(k0, one);
    }
  }
  if (wave > 0) {
    float* dst = red + ((wave - 1) * 64 + lane) * 8 * NT;
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int i = 0; i < 4; ++i) dst[(t * 2 + u) * 4 + i] = acc[t][u][i];
  }
  __syncthreads();
  if (wave > 0) return;
#pragma unroll
  for (int s = 0; s < 3; ++s) {
    const float* src = red + (s * 64 + lane) * 8 * NT;
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[t][u][i] += src[(t * 2 + u) * 4 + i];
  }

  // lane holds features j = 16 jt + 4 g + i (low) and j + half (high) of tokens m and (NT = 2) 16 + m
  if (bias && bias_dtype == IX_BF16) {
    blo = make_float4(__uint_as_float(blo16.x << 16), __uint_as_float(blo16.x & 0xffff0000u),
                      __uint_as_float(blo16.y << 16), __uint_as_float(blo16.y & 0xffff0000u));
    bhi = make_float4(__uint_as_float(bhi16.x << 16), __uint_as_float(bhi16.x & 0xffff0000u),
                      __uint_as_float(bhi16.y << 16), __uint_as_float(bhi16.y & 0xffff0000u));
  }
  const float bl[4] = {blo.x, blo.y, blo.z, blo.w}, bh[4] = {bhi.x, bhi.y, bhi.z, bhi.w};
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const int tok = 16 * t + m;
    if (tok >= tokens) continue;
    const float2 rot[4] = {make_float2(cs01[t].x, cs01[t].y), make_float2(cs01[t].z, cs01[t].w),
                           make_float2(cs23[t].x, cs23[t].y), make_float2(cs23[t].z, cs23[t].w)};
    float lo[4], hi[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      // the product is rounded to bfloat16 before the bias joins it, as when the two kernels run one after the other
      lo[i] = ix_bf16_to_f32(ix_f32_to_bf16(acc[t][0][i]));
      hi[i] = ix_bf16_to_f32(ix_f32_to_bf16(acc[t][1][i]));
      if (bias) {
        lo[i] += bl[i];
        hi[i] += bh[i];
      }
    }
    if (!is_v && cs) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float2 c = rot[i];
        const float rlo = lo[i] * c.x - hi[i] * c.y;
        const float rhi = hi[i] * c.x + lo[i] * c.y;
        lo[i] = rlo;
        hi[i] = rhi;
      }
    }
    const int slot_t = slot_of[t];
    const bool cache_ok = k_cache != nullptr && slot_t >= 0 && slot_t < total_slots;
    const int64_t page = cache_ok ? slot_t / page_size : 0;  // (slots are 32-bit: a short division)
    const int off = cache_ok ? slot_t - static_cast<int>(page) * page_size : 0;
    if (is_v) {
      if (!cache_ok) continue;
      __bf16* dst = v_cache + ((page * kv_heads + (head - heads - kv_heads)) * head_dim + j0) * page_size + off;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        dst[static_cast<int64_t>(i) * page_size] = (__bf16)lo[i];
        dst[static_cast<int64_t>(half + i) * page_size] = (__bf16)hi[i];
      }
      continue;
    }
    __bf16* dst = nullptr;
    if (head < heads) dst = q_out + (static_cast<int64_t>(tok) * heads + head) * head_dim + j0;
    else if (cache_ok) dst = k_cache + ((page * kv_heads + (head - heads)) * page_size + off) * head_dim + j0;
    if (dst) {
      bf16x4 a = {(__bf16)lo[0], (__bf16)lo[1], (__bf16)lo[2], (__bf16)lo[3]};
      bf16x4 b = {(__bf16)hi[0], (__bf16)hi[1], (__bf16)hi[2], (__bf16)hi[3]};
      *reinterpret_cast<bf16x4*>(dst) = a;
      *reinterpret_cast<bf16x4*>(dst + half) = b;
    }
  }
}

// x [tokens <= 32, width], w [(heads + 2 kv_heads) * head_dim, width]; head_dim a multiple of 32, width of 8.
extern "C" int ix_qkv_rope_skinny(const void* x, const void* w, const void* bias, int bias_dtype, const void* cs,
                                  const int32_t* slots, void* q_out, void* k_cache, void* v_cache, int tokens,
                                  int64_t width, int heads, int kv_heads, int head_dim, int page_size,
                                  int64_t total_slots, hipStream_t stream) {
  IX_REQUIRE(tokens > 0 && tokens <= 32, "between 1 and 32 tokens");
  IX_REQUIRE(heads > 0 && kv_heads > 0 && page_size > 0 && width > 0, "sizes must be positive");
  IX_REQUIRE(head_dim % 32 == 0 && head_dim <= 256, "head_dim must be a multiple of 32 up to 256");
  IX_REQUIRE(width % 8 == 0 && width < (1 << 30), "the reduction width must be a multiple of 8");
  IX_REQUIRE((k_cache == nullptr) == (v_cache == nullptr), "give both caches or neither");
  IX_REQUIRE(bias == nullptr || bias_dtype == IX_F32 || bias_dtype == IX_BF16, "the bias must be float32 or bfloat16");
  IX_REQUIRE(((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(w) | reinterpret_cast<uintptr_t>(bias) |
               reinterpret_cast<uintptr_t>(cs)) & 15) == 0, "operands must be aligned to 16 bytes");
  dim3 grid((heads + 2 * kv_heads) * (head_dim / 32)), block(256);
#define LAUNCH(NT)                                                                                                  \
  hipLaunchKernelGGL(qkv_rope_skinny_kernel<NT>, grid, block, 0, stream, (const __bf16*)x, (const __bf16*)w, bias,  \
                     bias_dtype, (const float2*)cs, slots, (__bf16*)q_out, (__bf16*)k_cache, (__bf16*)v_cache,      \
                     tokens, (int)width, heads, kv_heads, head_dim, page_size, total_slots)
  if (tokens <= 16) LAUNCH(1);
  else LAUNCH(2);
#undef LAUNCH
  return ix_check_launch("ix_qkv_rope_skinny");
}
