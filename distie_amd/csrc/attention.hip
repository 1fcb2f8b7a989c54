// Attention over the paged cache for one head size (compile with -DDISTIE_HEAD_DIM=<multiple of 16>).
//
// out[t, h] = softmax_j(q[t, h] . k[j, h / G] * scale) v[j, h / G] over the keys j that token t may see:
// first(t) <= j <= position(t), first = 0, or position - window + 1 on a windowed layer. Keys and values
// are read through the block table of the token's request: key j lives in page table[j / P] at offset
// j % P of a cache laid out [pages, kv_heads, P, D]. The new tokens of the step are already in the cache
// (the reference writes before it reads too: worker/src/inference/qwen2/paged_attn.py:389-397), so
// prefill, portions of prompts and decoded tokens are the same computation.
// Formula: worker/src/inference/qwen2/model.py:154-161; softmax and all sums in float32.
//
//  * attn_generic: one wave per (token, head); any types; the true 32-bit path and the fallback.

#include "common.h"

#ifndef DISTIE_HEAD_DIM
#error "compile with -DDISTIE_HEAD_DIM=<head size>"
#endif
#if DISTIE_HEAD_DIM % 16 != 0 || DISTIE_HEAD_DIM < 16 || DISTIE_HEAD_DIM > 256
#error "head size must be a multiple of 16 between 16 and 256"
#endif

constexpr int D = DISTIE_HEAD_DIM;
constexpr int DIMS_PER_LANE = (D + DISTIE_WAVE - 1) / DISTIE_WAVE;

extern "C" int distie_attention_head_dim() { return D; }

template <typename C>
__device__ __forceinline__ float dot_row(const float* q, const C* k);

template <>
__device__ __forceinline__ float dot_row<float>(const float* q, const float* k) {
  float s = 0.f;
#pragma unroll
  for (int d = 0; d < D; d += 4) {
    const float4 v = *reinterpret_cast<const float4*>(k + d);
    s = fmaf(q[d], v.x, s);
    s = fmaf(q[d + 1], v.y, s);
    s = fmaf(q[d + 2], v.z, s);
    s = fmaf(q[d + 3], v.w, s);
  }
  return s;
}

template <>
__device__ __forceinline__ float dot_row<bf16_t>(const float* q, const bf16_t* k) {
  float s = 0.f;
#pragma unroll
  for (int d = 0; d < D; d += 8) {
    const uint4 raw = *reinterpret_cast<const uint4*>(k + d);
    const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      s = fmaf(q[d + 2 * i], __uint_as_float(w[i] << 16), s);
      s = fmaf(q[d + 2 * i + 1], __uint_as_float(w[i] & 0xffff0000u), s);
    }
  }
  return s;
}

template <typename T, typename C>
__global__ __launch_bounds__(DISTIE_WAVE) void attn_generic_kernel(
    const T* __restrict__ qkv, int64_t q_stride, const C* __restrict__ k_cache, const C* __restrict__ v_cache,
    const int32_t* __restrict__ positions, const int32_t* __restrict__ token_request,
    const int32_t* __restrict__ block_table, int table_width, T* __restrict__ out, int heads, int kv_heads,
    int block_size, float scale, int window) {
  __shared__ float q_s[D];
  __shared__ float p_s[DISTIE_WAVE];
  __shared__ int64_t at_s[DISTIE_WAVE];
  const int lane = threadIdx.x;
  const int64_t t = blockIdx.x;
  const int h = blockIdx.y;
  const int kh = h / (heads / kv_heads);
  const int q_pos = positions[t];
  const int32_t* table = block_table + static_cast<int64_t>(token_request[t]) * table_width;
  const T* q = qkv + t * q_stride + static_cast<int64_t>(h) * D;
  for (int d = lane; d < D; d += DISTIE_WAVE) q_s[d] = to_float(q[d]);
  __syncthreads();

  const int first = window > 0 ? max(0, q_pos - window + 1) : 0;
  const int last = q_pos;   // inclusive
  float m = -INFINITY, l = 0.f;
  float acc[DIMS_PER_LANE];
#pragma unroll
  for (int i = 0; i < DIMS_PER_LANE; ++i) acc[i] = 0.f;

  for (int c = first; c <= last; c += DISTIE_WAVE) {
    const int key = c + lane;
    const bool valid = key <= last;
    float s = -INFINITY;
    int64_t at = 0;
    if (valid) {
      const int page = table[key / block_size];
      at = ((static_cast<int64_t>(page) * kv_heads + kh) * block_size + key % block_size) * D;
      s = dot_row<C>(q_s, k_cache + at) * scale;
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float alpha = expf(m - m_new);          // 0 on the first chunk (m = -inf)
    const float p = valid ? expf(s - m_new) : 0.f;
    l = l * alpha + wave_sum(p);
    m = m_new;
    __syncthreads();
    p_s[lane] = p;
    at_s[lane] = at;
    __syncthreads();
    const int n = min(DISTIE_WAVE, last - c + 1);
#pragma unroll
    for (int i = 0; i < DIMS_PER_LANE; ++i) {
      const int d = lane + i * DISTIE_WAVE;
      if (d < D) {
        float a = acc[i] * alpha;
        for (int j = 0; j < n; ++j) a = fmaf(p_s[j], to_float(v_cache[at_s[j] + d]), a);
        acc[i] = a;
      }
    }
  }
  T* o = out + (t * heads + h) * D;
  const float inv = 1.f / l;
#pragma unroll
  for (int i = 0; i < DIMS_PER_LANE; ++i) {
    const int d = lane + i * DISTIE_WAVE;
    if (d < D) o[d] = from_float<T>(acc[i] * inv);
  }
}

// qkv: [T, q_stride] with q of head h at columns h*D; out: [T, heads*D]. window = 0: every earlier key.
extern "C" int distie_attention_generic(const void* qkv, int dtype, int64_t q_stride, const void* k_cache,
                                        const void* v_cache, int cache_dtype, const int32_t* positions,
                                        const int32_t* token_request, const int32_t* block_table,
                                        int table_width, void* out, int tokens, int heads, int kv_heads,
                                        int block_size, float scale, int window, hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (heads < 1 || kv_heads < 1 || heads % kv_heads != 0 || block_size < 1 || table_width < 1 || window < 0)
    return DISTIE_BAD_ARGUMENT;
  if (heads > 65535) return DISTIE_BAD_ARGUMENT;
  dim3 grid(tokens, heads);
  DISTIE_DISPATCH(dtype, T, DISTIE_DISPATCH(cache_dtype, C,
      attn_generic_kernel<T, C><<<grid, DISTIE_WAVE, 0, stream>>>(
          static_cast<const T*>(qkv), q_stride, static_cast<const C*>(k_cache), static_cast<const C*>(v_cache),
          positions, token_request, block_table, table_width, static_cast<T*>(out), heads, kv_heads, block_size,
          scale, window)));
  return launch_status();
}
