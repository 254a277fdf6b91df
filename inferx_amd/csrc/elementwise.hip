// Embedding gather, residual-add + RMSNorm, SwiGLU product, rotary table,
// and the fused bias + rotation + cache-append that follows the q/k/v product.
//
// The residual stream `h` is float32 in every run; activations that feed
// matrix products have the run's type (float32 or bfloat16).  Sums of squares,
// the reciprocal root, rotation angles and the bias add are float32.
#include "common.h"

// ---------------------------------------------------------------------------
// h[t, :] = table[ids[t], :] * scale   (reference: EmbeddingKernel, layers.cu:465-481, which has no scale;
// an id outside the table gives a zero row here instead of row 0 -- the host
// rejects such ids before any launch)
template <typename TW>
__global__ void embed_kernel(float* __restrict__ h, const TW* __restrict__ table,
                             const int32_t* __restrict__ ids, int64_t width, int64_t vocab, float scale) {
  const int64_t t = blockIdx.x;
  const int64_t id = ids[t];
  const bool ok = id >= 0 && id < vocab;
  const TW* row = table + (ok ? id : 0) * width;
  for (int64_t i = threadIdx.x; i < width; i += blockDim.x) h[t * width + i] = ok ? ix_load(row + i) * scale : 0.f;
}

extern "C" int ix_embed(void* h, const void* table, int table_dtype, const int32_t* ids, int64_t tokens,
                        int64_t width, int64_t vocab, float scale, hipStream_t stream) {
  IX_REQUIRE(tokens >= 0 && width > 0 && vocab > 0, "sizes must be positive");
  if (tokens == 0) return 0;
  dim3 grid(tokens), block(256);
  if (table_dtype == IX_F32)
    hipLaunchKernelGGL(embed_kernel<float>, grid, block, 0, stream, (float*)h, (const float*)table, ids, width, vocab,
                       scale);
  else if (table_dtype == IX_BF16)
    hipLaunchKernelGGL(embed_kernel<bf16_t>, grid, block, 0, stream, (float*)h, (const bf16_t*)table, ids, width,
                       vocab, scale);
  else
    IX_REQUIRE(false, "table dtype must be float32 or bfloat16");
  return ix_check_launch("ix_embed");
}

// ---------------------------------------------------------------------------
// v = h[row] (+ delta[row]);  out[r] = v * rsqrt(mean(v^2) + eps) * w
// (reference: RmsNormKernel, layers.cu:50-76: one reciprocal root per row, the
// product x*inv*w formed in float32 and rounded once).
// With `rows` == null every row r is normalised in place order and h is
// updated with the sum; with `rows` given, out[r] comes from row rows[r] and h
// is left alone (a row may be asked for twice).
template <typename TD, typename TO>
__global__ void add_rmsnorm_kernel(float* __restrict__ h, const TD* __restrict__ delta, const void* __restrict__ w,
                                   int w_dtype, TO* __restrict__ out, const int32_t* __restrict__ rows,
                                   int64_t width, float eps) {
  __shared__ float red[16];
  const int64_t r = blockIdx.x;
  const int64_t row = rows ? rows[r] : r;
  float* hr = h + row * width;
  const TD* dr = delta ? delta + row * width : nullptr;
  const bool write_back = (rows == nullptr) && (dr != nullptr);
  float sumsq = 0.f;
  for (int64_t i = threadIdx.x; i < width; i += blockDim.x) {
    float v = hr[i];
    if (dr) v += ix_load(dr + i);
    if (write_back) hr[i] = v;
    sumsq += v * v;
  }
  sumsq = ix_block_sum(sumsq, red);
  const float inv = 1.0f / sqrtf(sumsq / static_cast<float>(width) + eps);
  TO* outr = out + r * width;
  for (int64_t i = threadIdx.x; i < width; i += blockDim.x) {
    float v = hr[i];
    if (dr && !write_back) v += ix_load(dr + i);
    ix_store(outr + i, v * inv * ix_load_rt(w, w_dtype, i));
  }
}

// bfloat16 delta and output with a width that is a multiple of 4: four columns per thread
__global__ void add_rmsnorm_vec4_kernel(float* __restrict__ h, const uint16_t* __restrict__ delta,
                                        const void* __restrict__ w, int w_dtype, uint16_t* __restrict__ out,
                                        const int32_t* __restrict__ rows, int64_t width, float eps) {
  __shared__ float red[16];
  const int64_t r = blockIdx.x;
  const int64_t row = rows ? rows[r] : r;
  float* hr = h + row * width;
  const uint16_t* dr = delta ? delta + row * width : nullptr;
  const bool write_back = (rows == nullptr) && (dr != nullptr);
  auto value = [&](int64_t c) {
    float4 v = *reinterpret_cast<const float4*>(hr + c);
    if (dr) {
      const uint2 d = *reinterpret_cast<const uint2*>(dr + c);
      v.x += __uint_as_float(d.x << 16);
      v.y += __uint_as_float(d.x & 0xffff0000u);
      v.z += __uint_as_float(d.y << 16);
      v.w += __uint_as_float(d.y & 0xffff0000u);
    }
    return v;
  };
  float sumsq = 0.f;
  for (int64_t c = 4 * threadIdx.x; c < width; c += 4 * blockDim.x) {
    const float4 v = value(c);
    sumsq += v.x * v.x;
    sumsq += v.y * v.y;
    sumsq += v.z * v.z;
    sumsq += v.w * v.w;
  }
  sumsq = ix_block_sum(sumsq, red);
  const float inv = 1.0f / sqrtf(sumsq / static_cast<float>(width) + eps);
  uint16_t* outr = out + r * width;
  for (int64_t c = 4 * threadIdx.x; c < width; c += 4 * blockDim.x) {
    const float4 v = value(c);  // h is still as it was: it is written here, after its last reading
    if (write_back) *reinterpret_cast<float4*>(hr + c) = v;
    uint2 o;
    o.x = ix_f32_to_bf16(v.x * inv * ix_load_rt(w, w_dtype, c)) |
          static_cast<uint32_t>(ix_f32_to_bf16(v.y * inv * ix_load_rt(w, w_dtype, c + 1))) << 16;
    o.y = ix_f32_to_bf16(v.z * inv * ix_load_rt(w, w_dtype, c + 2)) |
          static_cast<uint32_t>(ix_f32_to_bf16(v.w * inv * ix_load_rt(w, w_dtype, c + 3))) << 16;
    *reinterpret_cast<uint2*>(outr + c) = o;
  }
}

extern "C" int ix_add_rmsnorm(void* h, const void* delta, int delta_dtype, const void* w, int w_dtype, void* out,
                              int out_dtype, const int32_t* rows, int64_t n_out_rows, int64_t width, float eps,
                              hipStream_t stream) {
  IX_REQUIRE(width > 0 && n_out_rows >= 0, "sizes must be positive");
  IX_REQUIRE(w_dtype == IX_F32 || w_dtype == IX_BF16, "weight dtype must be float32 or bfloat16");
  if (n_out_rows == 0) return 0;
  dim3 grid(n_out_rows), block(width >= 4096 ? 1024 : (width >= 1024 ? 512 : 256));
#define LAUNCH(TD, TO)                                                                                          \
  hipLaunchKernelGGL((add_rmsnorm_kernel<TD, TO>), grid, block, 0, stream, (float*)h, (const TD*)delta, w, w_dtype, \
                     (TO*)out, rows, width, eps)
  if (out_dtype == IX_BF16 && (delta == nullptr || delta_dtype == IX_BF16) && width % 4 == 0 &&
      ((reinterpret_cast<uintptr_t>(h) | reinterpret_cast<uintptr_t>(delta) | reinterpret_cast<uintptr_t>(out)) & 15) == 0) {
    hipLaunchKernelGGL(add_rmsnorm_vec4_kernel, grid, dim3(width >= 4096 ? 1024 : (width >= 2048 ? 512 : 256)), 0, stream,
                       (float*)h, (const uint16_t*)delta, w, w_dtype, (uint16_t*)out, rows, width, eps);
    return ix_check_launch("ix_add_rmsnorm");
  }
  if (delta_dtype == IX_F32 && out_dtype == IX_F32) LAUNCH(float, float);
  else if (delta_dtype == IX_F32 && out_dtype == IX_BF16) LAUNCH(float, bf16_t);
  else if (delta_dtype == IX_BF16 && out_dtype == IX_F32) LAUNCH(bf16_t, float);
  else if (delta_dtype == IX_BF16 && out_dtype == IX_BF16) LAUNCH(bf16_t, bf16_t);
  else IX_REQUIRE(false, "dtypes must be float32 or bfloat16");
#undef LAUNCH
  return ix_check_launch("ix_add_rmsnorm");
}

// ---------------------------------------------------------------------------
// out[t, i] = silu(gu[t, i]) * gu[t, width + i],  silu(g) = g / (1 + exp(-g))
// (reference: SiluMulFusedKernel, layers.cu:512-529)
template <typename T>
__global__ void silu_mul_kernel(const T* __restrict__ gu, T* __restrict__ out, int64_t tokens, int64_t width) {
  const int64_t n = tokens * width;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    const int64_t t = i / width, c = i - t * width;
    const float g = ix_load(gu + t * 2 * width + c);
    const float u = ix_load(gu + t * 2 * width + width + c);
    ix_store(out + i, g / (1.0f + expf(-g)) * u);
  }
}

// bfloat16 with a width that is a multiple of 8: eight numbers per thread, 16-byte loads and stores
__global__ void __launch_bounds__(256)
silu_mul_vec8_kernel(const uint16_t* __restrict__ gu, uint16_t* __restrict__ out, int64_t tokens, int64_t width) {
  const int64_t per_row = width / 8, n = tokens * per_row;
  for (int64_t p = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; p < n;
       p += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    const int64_t t = p / per_row, c = (p - t * per_row) * 8;
    const uint4 g4 = *reinterpret_cast<const uint4*>(gu + t * 2 * width + c);
    const uint4 u4 = *reinterpret_cast<const uint4*>(gu + t * 2 * width + width + c);
    const uint32_t gw[4] = {g4.x, g4.y, g4.z, g4.w}, uw[4] = {u4.x, u4.y, u4.z, u4.w};
    uint32_t o[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float g0 = __uint_as_float(gw[i] << 16), g1 = __uint_as_float(gw[i] & 0xffff0000u);
      const float u0 = __uint_as_float(uw[i] << 16), u1 = __uint_as_float(uw[i] & 0xffff0000u);
      o[i] = ix_f32_to_bf16(g0 / (1.0f + expf(-g0)) * u0) |
             static_cast<uint32_t>(ix_f32_to_bf16(g1 / (1.0f + expf(-g1)) * u1)) << 16;
    }
    *reinterpret_cast<uint4*>(out + t * width + c) = make_uint4(o[0], o[1], o[2], o[3]);
  }
}

extern "C" int ix_silu_mul(const void* gu, void* out, int dtype, int64_t tokens, int64_t width, hipStream_t stream) {
  IX_REQUIRE(tokens >= 0 && width > 0, "sizes must be positive");
  if (tokens == 0) return 0;
  const int64_t n = tokens * width;
  dim3 grid(static_cast<unsigned>(std::min<int64_t>((n + 255) / 256, 65536))), block(256);
  if (dtype == IX_F32)
    hipLaunchKernelGGL(silu_mul_kernel<float>, grid, block, 0, stream, (const float*)gu, (float*)out, tokens, width);
  else if (dtype == IX_BF16 && width % 8 == 0 &&
           ((reinterpret_cast<uintptr_t>(gu) | reinterpret_cast<uintptr_t>(out)) & 15) == 0) {
    dim3 grid8(static_cast<unsigned>(std::min<int64_t>((n / 8 + 255) / 256, 65536)));
    hipLaunchKernelGGL(silu_mul_vec8_kernel, grid8, block, 0, stream, (const uint16_t*)gu, (uint16_t*)out, tokens,
                       width);
  } else if (dtype == IX_BF16)
    hipLaunchKernelGGL(silu_mul_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)gu, (bf16_t*)out, tokens,
                       width);
  else
    IX_REQUIRE(false, "dtype must be float32 or bfloat16");
  return ix_check_launch("ix_silu_mul");
}

// ---------------------------------------------------------------------------
// y[t, c] += bias[c]  (a product's bias where no kernel after it takes it along; the sum is formed in float32
// and rounded to y's type)
template <typename T>
__global__ void add_bias_kernel(T* __restrict__ y, const void* __restrict__ bias, int bias_dtype, int64_t n,
                                int64_t width) {
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x)
    ix_store(y + i, ix_load(y + i) + ix_load_rt(bias, bias_dtype, i % width));
}

extern "C" int ix_add_bias(void* y, int dtype, const void* bias, int bias_dtype, int64_t tokens, int64_t width,
                           hipStream_t stream) {
  IX_REQUIRE(tokens >= 0 && width > 0, "sizes must be positive");
  IX_REQUIRE(bias_dtype == IX_F32 || bias_dtype == IX_BF16, "the bias must be float32 or bfloat16");
  if (tokens == 0) return 0;
  const int64_t n = tokens * width;
  dim3 grid(static_cast<unsigned>(std::min<int64_t>((n + 255) / 256, 65536))), block(256);
  if (dtype == IX_F32)
    hipLaunchKernelGGL(add_bias_kernel<float>, grid, block, 0, stream, (float*)y, bias, bias_dtype, n, width);
  else if (dtype == IX_BF16)
    hipLaunchKernelGGL(add_bias_kernel<bf16_t>, grid, block, 0, stream, (bf16_t*)y, bias, bias_dtype, n, width);
  else
    IX_REQUIRE(false, "dtype must be float32 or bfloat16");
  return ix_check_launch("ix_add_bias");
}

// ---------------------------------------------------------------------------
// cs[t, j] = (cos a, sin a),  a = float(pos[t]) * inv_freq[j],  j < half
// (reference: RopeKernel, layers.cu:80-115, which recomputes the angle per head
// with fast intrinsics; here it is computed once per step with sincosf)
__global__ void rope_table_kernel(float2* __restrict__ cs, const int32_t* __restrict__ positions,
                                  const float* __restrict__ inv_freq, int64_t tokens, int half) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= tokens * half) return;
  const int64_t t = i / half;
  const int j = static_cast<int>(i - t * half);
  const float a = static_cast<float>(positions[t]) * inv_freq[j];
  float s, c;
  sincosf(a, &s, &c);
  cs[i] = make_float2(c, s);
}

extern "C" int ix_rope_table(void* cs, const int32_t* positions, const float* inv_freq, int64_t tokens, int half,
                             hipStream_t stream) {
  IX_REQUIRE(tokens >= 0 && half > 0, "sizes must be positive");
  if (tokens == 0) return 0;
  const int64_t n = tokens * half;
  hipLaunchKernelGGL(rope_table_kernel, dim3((n + 255) / 256), dim3(256), 0, stream, (float2*)cs, positions, inv_freq,
                     tokens, half);
  return ix_check_launch("ix_rope_table");
}

// ---------------------------------------------------------------------------
// After the fused q/k/v product: add the bias, rotate q and k (half-split
// pairs (j, j + d/2): x'_j = x_j cos - x_{j+d/2} sin, x'_{j+d/2} = x_{j+d/2} cos
// + x_j sin; reference RopeKernel layers.cu:80-115), write q to its own buffer
// and k, v into the cache page of the token's slot (rotated keys are what the
// cache holds; reference AppendKvKernel layers.cu:195-219, SplitQkvKernel :485-510).
// Cache layout per layer: keys [page][kv_head][offset in page][head_dim],
// values transposed [page][kv_head][head_dim][offset in page] (so that eight
// consecutive keys of one value column are 16 contiguous bytes for the
// matrix-core kernel).  A negative slot, or null caches, writes nothing.
// Rotation of a part of each head: the rot_dim elements from rot_begin on are rotated (pairs (j, j + rot_dim / 2)
// within that part, table [T, rot_dim / 2]), the others pass through (the reference rotates the trailing part of a
// head in the same pairing, src/backends/cuda/ops/mla.cu:24-46).  This general kernel takes that; the faster ones
// below rotate whole heads only.
template <typename T>
__global__ void qkv_rope_append_kernel(const T* __restrict__ qkv, const void* __restrict__ bias, int bias_dtype,
                                       const float2* __restrict__ cs, const int32_t* __restrict__ slots,
                                       T* __restrict__ q_out, T* __restrict__ k_cache, T* __restrict__ v_cache,
                                       int heads, int kv_heads, int head_dim, int page_size, int64_t total_slots,
                                       int rot_begin, int rot_dim) {
  const int64_t t = blockIdx.x;
  const int half = head_dim / 2, rot_half = rot_dim / 2;
  const int items = (heads + 2 * kv_heads) * half;
  const int64_t in_width = static_cast<int64_t>(heads + 2 * kv_heads) * head_dim;
  const T* in = qkv + t * in_width;
  const int64_t slot = slots ? slots[t] : -1;
  const bool cache_ok = k_cache != nullptr && slot >= 0 && slot < total_slots;
  const int64_t page = cache_ok ? slot / page_size : 0;
  const int off = cache_ok ? static_cast<int>(slot % page_size) : 0;
  for (int p = blockIdx.y * blockDim.x + threadIdx.x; p < items; p += gridDim.y * blockDim.x) {
    const int head = p / half, j = p - head * half;
    // the two elements of the head that this item takes: a pair of the rotated part, or two that pass through
    int ja, jb;
    const bool pair = j < rot_half;
    if (pair) {
      ja = rot_begin + j;
      jb = ja + rot_half;
    } else {
      const int u = 2 * (j - rot_half);  // the u-th and (u + 1)-th of the elements outside the rotated part
      ja = u < rot_begin ? u : u + rot_dim;
      jb = u + 1 < rot_begin ? u + 1 : u + 1 + rot_dim;
    }
    const int col = head * head_dim;
    float lo = ix_load(in + col + ja), hi = ix_load(in + col + jb);
    if (bias) {
      lo += ix_load_rt(bias, bias_dtype, col + ja);
      hi += ix_load_rt(bias, bias_dtype, col + jb);
    }
    const bool is_v = head >= heads + kv_heads;
    if (!is_v && cs && pair) {
      const float2 c = cs[t * rot_half + j];
      const float rlo = lo * c.x - hi * c.y;
      const float rhi = hi * c.x + lo * c.y;
      lo = rlo;
      hi = rhi;
    }
    if (head < heads) {
      T* dst = q_out + (t * heads + head) * head_dim;
      ix_store(dst + ja, lo);
      ix_store(dst + jb, hi);
    } else if (cache_ok) {
      if (is_v) {
        const int g = head - heads - kv_heads;
        T* dst = v_cache + (page * kv_heads + g) * head_dim * page_size + off;
        ix_store(dst + static_cast<int64_t>(ja) * page_size, lo);
        ix_store(dst + static_cast<int64_t>(jb) * page_size, hi);
      } else {
        const int g = head - heads;
        T* dst = k_cache + ((page * kv_heads + g) * page_size + off) * head_dim;
        ix_store(dst + ja, lo);
        ix_store(dst + jb, hi);
      }
    }
  }
}

// The same for bfloat16 with head_dim a multiple of 16: a thread takes eight consecutive elements of the
// low half of a head and the eight of the high half that pair with them (16-byte loads and stores).
// (`t`: the token; `part` of `parts` workgroups share its elements)
__device__ __forceinline__ void
qkv_rope_append_vec8_body(int64_t t, int part, int parts, const uint16_t* __restrict__ qkv,
                          const void* __restrict__ bias, int bias_dtype, const float2* __restrict__ cs,
                          const int32_t* __restrict__ slots, uint16_t* __restrict__ q_out,
                          uint16_t* __restrict__ k_cache, uint16_t* __restrict__ v_cache, int heads, int kv_heads,
                          int head_dim, int page_size, int64_t total_slots, int skip_v) {
  const int half = head_dim / 2, per_head = half / 8;
  const int items = (heads + (skip_v ? 1 : 2) * kv_heads) * per_head;  // values may be left to the kernel below
  const int64_t in_width = static_cast<int64_t>(heads + 2 * kv_heads) * head_dim;
  const uint16_t* in = qkv + t * in_width;
  const int64_t slot = slots ? slots[t] : -1;
  const bool cache_ok = k_cache != nullptr && slot >= 0 && slot < total_slots;
  const int64_t page = cache_ok ? slot / page_size : 0;
  const int off = cache_ok ? static_cast<int>(slot % page_size) : 0;
  // eight bias values from column c on (c is a multiple of 8): one or two 16-byte loads where the bias allows it
  const bool bias_vec = (reinterpret_cast<uintptr_t>(bias) & 15) == 0;
  auto add_bias8 = [&](float (&v)[8], int c) {
    if (bias_vec && bias_dtype == IX_BF16) {
      const uint4 b = *reinterpret_cast<const uint4*>(static_cast<const uint16_t*>(bias) + c);
      const uint32_t w[4] = {b.x, b.y, b.z, b.w};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        v[2 * i] += __uint_as_float(w[i] << 16);
        v[2 * i + 1] += __uint_as_float(w[i] & 0xffff0000u);
      }
    } else if (bias_vec && bias_dtype == IX_F32) {
      const float4 a = *reinterpret_cast<const float4*>(static_cast<const float*>(bias) + c);
      const float4 b = *reinterpret_cast<const float4*>(static_cast<const float*>(bias) + c + 4);
      v[0] += a.x; v[1] += a.y; v[2] += a.z; v[3] += a.w;
      v[4] += b.x; v[5] += b.y; v[6] += b.z; v[7] += b.w;
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) v[i] += ix_load_rt(bias, bias_dtype, c + i);
    }
  };
  for (int p = part * blockDim.x + threadIdx.x; p < items; p += parts * blockDim.x) {
    const int head = p / per_head, j = (p - head * per_head) * 8;
    const int col = head * head_dim + j;
    const uint4 lo4 = *reinterpret_cast<const uint4*>(in + col);
    const uint4 hi4 = *reinterpret_cast<const uint4*>(in + col + half);
    const uint32_t lw[4] = {lo4.x, lo4.y, lo4.z, lo4.w}, hw[4] = {hi4.x, hi4.y, hi4.z, hi4.w};
    float lo[8], hi[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      lo[2 * i] = __uint_as_float(lw[i] << 16);
      lo[2 * i + 1] = __uint_as_float(lw[i] & 0xffff0000u);
      hi[2 * i] = __uint_as_float(hw[i] << 16);
      hi[2 * i + 1] = __uint_as_float(hw[i] & 0xffff0000u);
    }
    if (bias) {
      add_bias8(lo, col);
      add_bias8(hi, col + half);
    }
    const bool is_v = head >= heads + kv_heads;
    if (!is_v && cs) {
      // eight (cos, sin) pairs are 64 contiguous bytes (the table is float32 [T, half, 2], a row a multiple of 64 bytes)
      const float4* c4 = reinterpret_cast<const float4*>(cs + t * half + j);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float4 c = c4[i];
        const float l0 = lo[2 * i], h0 = hi[2 * i], l1 = lo[2 * i + 1], h1 = hi[2 * i + 1];
        lo[2 * i] = l0 * c.x - h0 * c.y;
        hi[2 * i] = h0 * c.x + l0 * c.y;
        lo[2 * i + 1] = l1 * c.z - h1 * c.w;
        hi[2 * i + 1] = h1 * c.z + l1 * c.w;
      }
    }
    uint16_t lb[8], hb[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      lb[i] = ix_f32_to_bf16(lo[i]);
      hb[i] = ix_f32_to_bf16(hi[i]);
    }
    if (is_v) {
      if (cache_ok) {
        const int g = head - heads - kv_heads;
        uint16_t* dst = v_cache + ((page * kv_heads + g) * head_dim + j) * page_size + off;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          dst[static_cast<int64_t>(i) * page_size] = lb[i];
          dst[static_cast<int64_t>(half + i) * page_size] = hb[i];
        }
      }
    } else {
      uint16_t* dst = nullptr;
      if (head < heads) dst = q_out + (t * heads + head) * head_dim + j;
      else if (cache_ok) dst = k_cache + ((page * kv_heads + (head - heads)) * page_size + off) * head_dim + j;
      if (dst) {
        uint4 a, b;
        a.x = lb[0] | (uint32_t)lb[1] << 16; a.y = lb[2] | (uint32_t)lb[3] << 16;
        a.z = lb[4] | (uint32_t)lb[5] << 16; a.w = lb[6] | (uint32_t)lb[7] << 16;
        b.x = hb[0] | (uint32_t)hb[1] << 16; b.y = hb[2] | (uint32_t)hb[3] << 16;
        b.z = hb[4] | (uint32_t)hb[5] << 16; b.w = hb[6] | (uint32_t)hb[7] << 16;
        *reinterpret_cast<uint4*>(dst) = a;
        *reinterpret_cast<uint4*>(dst + half) = b;
      }
    }
  }
}

__global__ void __launch_bounds__(256)
qkv_rope_append_vec8_kernel(const uint16_t* __restrict__ qkv, const void* __restrict__ bias, int bias_dtype,
                            const float2* __restrict__ cs, const int32_t* __restrict__ slots,
                            uint16_t* __restrict__ q_out, uint16_t* __restrict__ k_cache,
                            uint16_t* __restrict__ v_cache, int heads, int kv_heads, int head_dim, int page_size,
                            int64_t total_slots, int skip_v) {
  qkv_rope_append_vec8_body(blockIdx.x, blockIdx.y, gridDim.y, qkv, bias, bias_dtype, cs, slots, q_out, k_cache, v_cache,
                            heads, kv_heads, head_dim, page_size, total_slots, skip_v);
}

// Values of many tokens (bfloat16): the cache keeps them transposed, so a token's values are head_dim separate
// 2-byte stores.  A workgroup takes 32 tokens of one kv head, turns the tile in LDS and stores with neighbouring
// lanes on neighbouring tokens: tokens of one request have consecutive slots, so 32 lanes fill 64 contiguous bytes.
#define V_TILE_TOKENS 32
__device__ __forceinline__ void
v_append_tile_body(int64_t tile, int g, uint16_t* v_tile, const uint16_t* __restrict__ qkv,
                   const void* __restrict__ bias, int bias_dtype, const int32_t* __restrict__ slots,
                   uint16_t* __restrict__ v_cache, int64_t tokens, int heads, int kv_heads, int head_dim, int page_size,
                   int64_t total_slots) {
  const int stride = head_dim + 2;  // v_tile is [32][head_dim + 2]
  const int64_t t0 = tile * V_TILE_TOKENS;
  const int tid = threadIdx.x;
  const int64_t in_width = static_cast<int64_t>(heads + 2 * kv_heads) * head_dim;
  const int col0 = (heads + kv_heads + g) * head_dim;
  const int pieces = head_dim / 8;
  for (int item = tid; item < V_TILE_TOKENS * pieces; item += 256) {
    const int i = item / pieces, d0 = (item - i * pieces) * 8;
    if (t0 + i >= tokens) continue;
    const uint4 v4 = *reinterpret_cast<const uint4*>(qkv + (t0 + i) * in_width + col0 + d0);
    const uint32_t vw[4] = {v4.x, v4.y, v4.z, v4.w};
    uint32_t* dst = reinterpret_cast<uint32_t*>(v_tile + i * stride + d0);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      float a = __uint_as_float(vw[j] << 16), b = __uint_as_float(vw[j] & 0xffff0000u);
      if (bias) {
        a += ix_load_rt(bias, bias_dtype, col0 + d0 + 2 * j);
        b += ix_load_rt(bias, bias_dtype, col0 + d0 + 2 * j + 1);
      }
      dst[j] = ix_f32_to_bf16(a) | static_cast<uint32_t>(ix_f32_to_bf16(b)) << 16;
    }
  }
  __syncthreads();
  const int i = tid & (V_TILE_TOKENS - 1);
  if (t0 + i >= tokens) return;
  const int64_t slot = slots[t0 + i];
  if (slot < 0 || slot >= total_slots) return;
  const int64_t page = slot / page_size;
  const int off = static_cast<int>(slot % page_size);
  uint16_t* dst = v_cache + (page * kv_heads + g) * head_dim * page_size + off;
  for (int d = tid / V_TILE_TOKENS; d < head_dim; d += 256 / V_TILE_TOKENS)
    dst[static_cast<int64_t>(d) * page_size] = v_tile[i * stride + d];
}

// One launch for both: the first `rope_blocks` workgroups (`parts` per token) add the bias, rotate and store
// queries and keys; the others turn tiles of values.  Neither half waits for the other, and a prompt portion
// pays one launch instead of two.
__global__ void __launch_bounds__(256)
qkv_rope_append_tiles_kernel(const uint16_t* __restrict__ qkv, const void* __restrict__ bias, int bias_dtype,
                             const float2* __restrict__ cs, const int32_t* __restrict__ slots,
                             uint16_t* __restrict__ q_out, uint16_t* __restrict__ k_cache,
                             uint16_t* __restrict__ v_cache, int64_t tokens, int heads, int kv_heads, int head_dim,
                             int page_size, int64_t total_slots, int parts, int64_t rope_blocks) {
  extern __shared__ __align__(16) uint16_t v_tile[];
  const int64_t b = blockIdx.x;
  if (b < rope_blocks) {
    qkv_rope_append_vec8_body(b / parts, static_cast<int>(b % parts), parts, qkv, bias, bias_dtype, cs, slots, q_out,
                              k_cache, v_cache, heads, kv_heads, head_dim, page_size, total_slots, 1);
  } else {
    const int64_t v = b - rope_blocks;
    v_append_tile_body(v / kv_heads, static_cast<int>(v % kv_heads), v_tile, qkv, bias, bias_dtype, slots, v_cache,
                       tokens, heads, kv_heads, head_dim, page_size, total_slots);
  }
}

// cs float32 [tokens, rot_dim / 2, 2] (cosine, sine) or null; elements [rot_begin, rot_begin + rot_dim) of every
// head of q and k are rotated.
extern "C" int ix_qkv_rope_append(const void* qkv, int dtype, const void* bias, int bias_dtype, const void* cs,
                                  const int32_t* slots, void* q_out, void* k_cache, void* v_cache, int64_t tokens,
                                  int heads, int kv_heads, int head_dim, int page_size, int64_t total_slots,
                                  int rot_begin, int rot_dim, hipStream_t stream) {
  IX_REQUIRE(tokens >= 0 && heads > 0 && kv_heads > 0 && head_dim > 0 && page_size > 0, "sizes must be positive");
  IX_REQUIRE(head_dim % 2 == 0, "head_dim must be even");
  IX_REQUIRE((k_cache == nullptr) == (v_cache == nullptr), "give both caches or neither");
  IX_REQUIRE(rot_begin >= 0 && rot_dim >= 0 && rot_dim % 2 == 0 && rot_begin + rot_dim <= head_dim,
             "the rotated part must be an even number of elements within the head");
  if (tokens == 0) return 0;
  const bool whole = cs == nullptr || (rot_begin == 0 && rot_dim == head_dim);
  if (cs == nullptr) rot_begin = 0, rot_dim = head_dim;
  const int items = (heads + 2 * kv_heads) * (head_dim / 2);
  dim3 grid(tokens, std::min((items + 255) / 256, 8)), block(256);
  if (dtype == IX_F32)
    hipLaunchKernelGGL(qkv_rope_append_kernel<float>, grid, block, 0, stream, (const float*)qkv, bias, bias_dtype,
                       (const float2*)cs, slots, (float*)q_out, (float*)k_cache, (float*)v_cache, heads, kv_heads,
                       head_dim, page_size, total_slots, rot_begin, rot_dim);
  else if (dtype == IX_BF16 && whole && head_dim % 16 == 0 && (reinterpret_cast<uintptr_t>(cs) & 15) == 0) {
    // from a few dozen tokens on, the values go through the kernel that turns tiles of them
    const int skip_v = (tokens >= 2 * V_TILE_TOKENS && v_cache != nullptr && slots != nullptr) ? 1 : 0;
    const int items8 = (heads + (skip_v ? 1 : 2) * kv_heads) * (head_dim / 16);
    const int parts = std::min((items8 + 255) / 256, 8);
    if (skip_v) {
      const int64_t rope_blocks = tokens * parts;
      const int64_t tile_blocks = (tokens + V_TILE_TOKENS - 1) / V_TILE_TOKENS * kv_heads;
      IX_REQUIRE(rope_blocks + tile_blocks < (int64_t(1) << 31), "too many tokens for one launch");
      const size_t lds = static_cast<size_t>(V_TILE_TOKENS) * (head_dim + 2) * sizeof(uint16_t);
      hipLaunchKernelGGL(qkv_rope_append_tiles_kernel, dim3(static_cast<unsigned>(rope_blocks + tile_blocks)), block, lds,
                         stream, (const uint16_t*)qkv, bias, bias_dtype, (const float2*)cs, slots, (uint16_t*)q_out,
                         (uint16_t*)k_cache, (uint16_t*)v_cache, tokens, heads, kv_heads, head_dim, page_size,
                         total_slots, parts, rope_blocks);
    } else {
      hipLaunchKernelGGL(qkv_rope_append_vec8_kernel, dim3(tokens, parts), block, 0, stream, (const uint16_t*)qkv, bias,
                         bias_dtype, (const float2*)cs, slots, (uint16_t*)q_out, (uint16_t*)k_cache,
                         (uint16_t*)v_cache, heads, kv_heads, head_dim, page_size, total_slots, 0);
    }
  } else if (dtype == IX_BF16)
    hipLaunchKernelGGL(qkv_rope_append_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)qkv, bias, bias_dtype,
                       (const float2*)cs, slots, (bf16_t*)q_out, (bf16_t*)k_cache, (bf16_t*)v_cache, heads, kv_heads,
                       head_dim, page_size, total_slots, rot_begin, rot_dim);
  else
    IX_REQUIRE(false, "dtype must be float32 or bfloat16");
  return ix_check_launch("ix_qkv_rope_append");
}
