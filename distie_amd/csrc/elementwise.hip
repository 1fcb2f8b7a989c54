// Memory-bound kernels of a step: embedding rows, RMS norm (alone and fused with the residual
// sum), rotation + cache write, gated activation, row gather.
//
// Reference formulas (paths in the reference checkout):
//   RMS norm   worker/src/inference/qwen2/model.py:85-90
//   rotation   worker/src/inference/qwen2/model.py:98-117
//   cache slot worker/src/inference/qwen2/paged_attn.py:341, 360-371
//   SwiGLU     worker/src/inference/qwen2/model.py:236
// Statistics, angles, trigonometry and the residual sum are float32 whatever the storage type.

#include "common.h"

// ---------------------------------------------------------------- embedding
template <typename W>
__global__ void embed_kernel(const int32_t* __restrict__ ids, const W* __restrict__ table,
                             float* __restrict__ out, int width, int vocab) {
  const int64_t t = blockIdx.x;
  int64_t id = ids[t];
  if (id < 0 || id >= vocab) id = 0;  // ids are validated on the host; never read outside the table
  const W* row = table + id * width;
  float* dst = out + t * width;
  for (int i = threadIdx.x; i < width; i += blockDim.x) dst[i] = to_float(row[i]);
}

extern "C" int distie_embed(const int32_t* ids, const void* table, int table_dtype, float* out,
                            int tokens, int width, int vocab, hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (width <= 0 || vocab <= 0) return DISTIE_BAD_ARGUMENT;
  const int threads = width >= 1024 ? 256 : 64;
  DISTIE_DISPATCH(table_dtype, W,
                  embed_kernel<W><<<tokens, threads, 0, stream>>>(ids, static_cast<const W*>(table), out, width, vocab));
  return launch_status();
}

// ---------------------------------------------------------------- RMS norm
// One block per row. With `delta`, the row of the residual stream is first updated
// (residual += delta, float32) and then normed: one pass less over the activations. `delta` may be
// `slices` partial sums laid side by side (`slice_stride` elements apart); they are added in order.
template <typename D, typename W, typename O>
__global__ void rmsnorm_kernel(float* __restrict__ residual, const D* __restrict__ delta, int slices,
                               int64_t slice_stride, const W* __restrict__ weight, O* __restrict__ out,
                               int width, float eps) {
  __shared__ float scratch[16];
  const int64_t row = blockIdx.x;
  float* x = residual + row * width;
  O* y = out + row * width;
  const D* d = delta != nullptr ? delta + row * width : nullptr;
  constexpr int KEEP = 4;                       // elements a thread keeps in registers between the passes
  if (width <= KEEP * static_cast<int>(blockDim.x)) {
    float v[KEEP];
    float ss = 0.f;
#pragma unroll
    for (int e = 0; e < KEEP; ++e) {
      const int i = threadIdx.x + e * blockDim.x;
      v[e] = 0.f;
      if (i < width) {
        v[e] = x[i];
        if (d != nullptr) {
          v[e] += sum_strided(d + i, slices, slice_stride);
          x[i] = v[e];
        }
        ss += v[e] * v[e];
      }
    }
    const float scale = rsqrtf(block_sum(ss, scratch) / static_cast<float>(width) + eps);
#pragma unroll
    for (int e = 0; e < KEEP; ++e) {
      const int i = threadIdx.x + e * blockDim.x;
      if (i < width) y[i] = from_float<O>(v[e] * scale * to_float(weight[i]));
    }
    return;
  }
  float ss = 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    float v = x[i];
    if (d != nullptr) {
      v += sum_strided(d + i, slices, slice_stride);
      x[i] = v;
    }
    ss += v * v;
  }
  const float scale = rsqrtf(block_sum(ss, scratch) / static_cast<float>(width) + eps);
  // each thread re-reads what it wrote itself
  for (int i = threadIdx.x; i < width; i += blockDim.x) y[i] = from_float<O>(x[i] * scale * to_float(weight[i]));
}

// The same for rows of whole float4s and float32 (or no) delta: a thread owns NV groups of four
// consecutive elements, every load of the row (residual, all slices, weights) is in flight before the
// first sum, and nothing is read twice.
static __device__ __forceinline__ float4 load_weights4(const float* w) { return *reinterpret_cast<const float4*>(w); }
static __device__ __forceinline__ float4 load_weights4(const bf16_t* w) {
  const uint2 raw = *reinterpret_cast<const uint2*>(w);
  return float4{__uint_as_float(raw.x << 16), __uint_as_float(raw.x & 0xffff0000u), __uint_as_float(raw.y << 16),
                __uint_as_float(raw.y & 0xffff0000u)};
}
static __device__ __forceinline__ void store4(float* p, const float4& v) { *reinterpret_cast<float4*>(p) = v; }
static __device__ __forceinline__ void store4(bf16_t* p, const float4& v) {
  const uint32_t a = __builtin_bit_cast(uint16_t, static_cast<bf16_t>(v.x));
  const uint32_t b = __builtin_bit_cast(uint16_t, static_cast<bf16_t>(v.y));
  const uint32_t c = __builtin_bit_cast(uint16_t, static_cast<bf16_t>(v.z));
  const uint32_t d = __builtin_bit_cast(uint16_t, static_cast<bf16_t>(v.w));
  *reinterpret_cast<uint2*>(p) = uint2{a | (b << 16), c | (d << 16)};
}

template <typename D, typename W, typename O, int NV>
__global__ __launch_bounds__(1024) void rmsnorm_vec_kernel(float* __restrict__ residual, const D* __restrict__ delta,
                                                           int slices, int64_t slice_stride,
                                                           const W* __restrict__ weight, O* __restrict__ out, int width,
                                                           float eps) {
  __shared__ float scratch[16];
  constexpr int GROUP = 8;                     // slices loaded together (16 changes nothing: 4.2 us at 14 slices)
  const int64_t row = blockIdx.x;
  const int quads = width / 4;
  float4 v[NV], wq[NV];
  float ss = 0.f;
#pragma unroll
  for (int e = 0; e < NV; ++e) {
    const int q = threadIdx.x + e * blockDim.x;
    const bool in = q < quads;
    const int64_t at = row * width + 4 * static_cast<int64_t>(in ? q : 0);
    const float4 x4 = *reinterpret_cast<const float4*>(residual + at);
    wq[e] = load_weights4(weight + 4 * (in ? q : 0));
    float4 sum = {0.f, 0.f, 0.f, 0.f};
    if (delta != nullptr && slices == 1) {
      sum = load_weights4(delta + at);
    } else if (delta != nullptr) {
      const int last = slices - 1;
      for (int s0 = 0; s0 < slices; s0 += GROUP) {
        float4 part[GROUP];
#pragma unroll
        for (int u = 0; u < GROUP; ++u)
          part[u] = load_weights4(delta + min(s0 + u, last) * slice_stride + at);
#pragma unroll
        for (int u = 0; u < GROUP; ++u) {
          if (s0 + u <= last) {
            sum.x += part[u].x;
            sum.y += part[u].y;
            sum.z += part[u].z;
            sum.w += part[u].w;
          }
        }
      }
    }
    v[e] = float4{x4.x + sum.x, x4.y + sum.y, x4.z + sum.z, x4.w + sum.w};
    if (!in) v[e] = float4{0.f, 0.f, 0.f, 0.f};
    if (in && delta != nullptr) *reinterpret_cast<float4*>(residual + at) = v[e];
    ss += v[e].x * v[e].x + v[e].y * v[e].y + v[e].z * v[e].z + v[e].w * v[e].w;
  }
  const float scale = rsqrtf(block_sum(ss, scratch) / static_cast<float>(width) + eps);
#pragma unroll
  for (int e = 0; e < NV; ++e) {
    const int q = threadIdx.x + e * blockDim.x;
    if (q >= quads) continue;
    store4(out + row * width + 4 * static_cast<int64_t>(q),
           float4{v[e].x * scale * wq[e].x, v[e].y * scale * wq[e].y, v[e].z * scale * wq[e].z, v[e].w * scale * wq[e].w});
  }
}

static inline bool aligned16(const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; }

template <typename D, typename W>
static int rmsnorm_launch_out(float* residual, const D* delta, int slices, const W* weight, void* out,
                              int out_dtype, int rows, int width, float eps, hipStream_t stream) {
  const int64_t slice_stride = static_cast<int64_t>(rows) * width;
  {
    if (width % 4 == 0 && width <= 8192 && aligned16(residual) && aligned16(delta) && aligned16(weight) &&
        aligned16(out)) {
      const int quads = width / 4;
      int threads = (quads + 63) / 64 * 64;
      // two groups of four a thread for rows beyond 4,096 elements, and when one group a thread would make
      // more waves than the chip holds at once (256 compute units x 32): the rows then fit in one round
      const int nv = (threads > 1024 || (quads > 64 && static_cast<int64_t>(rows) * (threads / 64) > 8192)) ? 2 : 1;
      if (nv == 2) threads = ((quads + 1) / 2 + 63) / 64 * 64;
      if (nv == 1) {
        DISTIE_DISPATCH(out_dtype, O, (rmsnorm_vec_kernel<D, W, O, 1><<<rows, threads, 0, stream>>>(
                                          residual, delta, slices, slice_stride, weight, static_cast<O*>(out), width, eps)));
      } else {
        DISTIE_DISPATCH(out_dtype, O, (rmsnorm_vec_kernel<D, W, O, 2><<<rows, threads, 0, stream>>>(
                                          residual, delta, slices, slice_stride, weight, static_cast<O*>(out), width, eps)));
      }
      return launch_status();
    }
  }
  // a thread's work is a chain of loads: about two elements a thread, so that a row stays in registers
  // between the two passes
  int threads = (width / 2 + 63) / 64 * 64;
  threads = threads < 64 ? 64 : (threads > 1024 ? 1024 : threads);
  DISTIE_DISPATCH(out_dtype, O,
                  rmsnorm_kernel<D, W, O><<<rows, threads, 0, stream>>>(
                      residual, delta, slices, slice_stride, weight, static_cast<O*>(out), width, eps));
  return launch_status();
}

// delta: null, or [slices, rows, width] of delta_dtype
extern "C" int distie_rmsnorm(float* residual, const void* delta, int delta_dtype, int slices, const void* weight,
                              int weight_dtype, void* out, int out_dtype, int rows, int width, float eps,
                              hipStream_t stream) {
  if (rows <= 0) return 0;
  if (width <= 0 || slices < 1) return DISTIE_BAD_ARGUMENT;
  DISTIE_DISPATCH(weight_dtype, W, DISTIE_DISPATCH(delta_dtype, D, return rmsnorm_launch_out<D, W>(
      residual, static_cast<const D*>(delta), slices, static_cast<const W*>(weight), out, out_dtype, rows, width, eps,
      stream)));
  return DISTIE_BAD_ARGUMENT;
}

// ---------------------------------------------------------------- rotation + cache write
// in: [slices, T, (H + 2 KH) * D] (partial sums of the q/k/v product, added in order; one slice for a
// finished product), out: [T, (H + 2 KH) * D], which may be `in` itself. One block per token. Pair
// (j, j + R/2) of every q and k head is turned by angle = float(position) * inv_freq[j] (R = 2 * pairs <= D
// is the rotated width). The turned k and the v of the token go to the cache at the token's slot
// (slot = page * P + offset): k into [pages, KH, P, D], v transposed into [pages, KH, D, P].
// cos and sin of every (token, pair), once per step: all layers of a step turn by the same angles
__global__ void rope_table_kernel(const int32_t* __restrict__ positions, const float* __restrict__ inv_freq,
                                  float2* __restrict__ table, int pairs) {
  const int64_t t = blockIdx.x;
  const float pos = static_cast<float>(positions[t]);
  for (int j = threadIdx.x; j < pairs; j += blockDim.x) {
    float sn, cs;
    sincosf(pos * inv_freq[j], &sn, &cs);
    table[t * pairs + j] = float2{cs, sn};
  }
}

extern "C" int distie_rope_table(const int32_t* positions, const float* inv_freq, void* table, int tokens, int pairs,
                                 hipStream_t stream) {
  if (tokens <= 0 || pairs <= 0) return 0;
  rope_table_kernel<<<tokens, 64, 0, stream>>>(positions, inv_freq, static_cast<float2*>(table), pairs);
  return launch_status();
}

template <typename I, typename T, typename C>
__global__ void rope_kv_write_kernel(const I* in, int slices, int64_t slice_stride, T* out,
                                     const float2* __restrict__ table,
                                     const int32_t* __restrict__ positions, const int32_t* __restrict__ slots,
                                     C* __restrict__ k_cache, C* __restrict__ v_cache,
                                     const float* __restrict__ inv_freq, int pairs, int heads, int kv_heads, int dim,
                                     int block_size, int write) {
  const int64_t t = blockIdx.x;
  const int64_t width = static_cast<int64_t>(heads + 2 * kv_heads) * dim;
  const I* src = in + t * width;
  T* row = out + t * width;
  const float pos = static_cast<float>(positions[t]);
  const int64_t slot = write ? slots[t] : 0;
  const int64_t page = slot / block_size;
  const int offset = static_cast<int>(slot % block_size);
  auto value = [&](int64_t i) { return sum_strided(src + i, slices, slice_stride); };
  // q and k heads: every thread owns whole pairs, so `out` may alias `in`. A thread that turns a pair of a k
  // head, or copies a value of a v head, also stores it into the cache.
  const int rotated_heads = heads + kv_heads;
  const int half = dim / 2;
  const int rot = 2 * pairs;
  for (int i = threadIdx.x; i < rotated_heads * pairs; i += blockDim.x) {
    const int head = i / pairs;
    const int j = i % pairs;
    const int64_t lo = static_cast<int64_t>(head) * dim + j;
    const float x0 = value(lo), x1 = value(lo + pairs);
    float sn, cs;
    if (table != nullptr) {
      const float2 e = table[t * pairs + j];
      cs = e.x;
      sn = e.y;
    } else {
      sincosf(pos * inv_freq[j], &sn, &cs);
    }
    const T a = from_float<T>(x0 * cs - x1 * sn);
    const T b = from_float<T>(x1 * cs + x0 * sn);
    row[lo] = a;
    row[lo + pairs] = b;
    if (write && head >= heads) {
      const int64_t at = ((page * kv_heads + (head - heads)) * block_size + offset) * dim;
      k_cache[at + j] = from_float<C>(to_float(a));
      k_cache[at + j + pairs] = from_float<C>(to_float(b));
    }
  }
  (void)half;
  // columns of q and k beyond the rotated width, and v: copied
  for (int64_t i = threadIdx.x; i < width; i += blockDim.x) {
    const int head = static_cast<int>(i / dim);
    const int d = static_cast<int>(i % dim);
    if (head < rotated_heads && d < rot) continue;
    const T v = from_float<T>(value(i));
    row[i] = v;
    if (!write || head < heads) continue;
    if (head < rotated_heads) {
      k_cache[((page * kv_heads + (head - heads)) * block_size + offset) * dim + d] = from_float<C>(to_float(v));
    } else {
      v_cache[(page * kv_heads + (head - rotated_heads)) * block_size * dim + static_cast<int64_t>(d) * block_size + offset] =
          from_float<C>(to_float(v));
    }
  }
}

// The same for a finished bfloat16 product (one slice), a bfloat16 cache, the whole head rotated and a head
// size that is a multiple of 16: a thread turns eight pairs at a time with 16-byte loads and stores.
static __device__ __forceinline__ void unpack8(const uint4& raw, float v[8]) {
  const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    v[2 * e] = __uint_as_float(w[e] << 16);
    v[2 * e + 1] = __uint_as_float(w[e] & 0xffff0000u);
  }
}
static __device__ __forceinline__ uint4 pack8(const float v[8]) {
  uint32_t w[4];
#pragma unroll
  for (int e = 0; e < 4; ++e)
    w[e] = static_cast<uint32_t>(__builtin_bit_cast(uint16_t, static_cast<bf16_t>(v[2 * e]))) |
           (static_cast<uint32_t>(__builtin_bit_cast(uint16_t, static_cast<bf16_t>(v[2 * e + 1]))) << 16);
  return uint4{w[0], w[1], w[2], w[3]};
}

// Blocks 0 .. tokens - 1 turn q and k of one token each and write k into the cache; the blocks behind them write v
// into the cache for 16 tokens each: the cache keeps v with the key index innermost, so one token's values lie
// block_size elements apart, and 16 tokens that follow one another inside a page fill 32 bytes in a row, written
// by one thread as two 16-byte stores instead of 16 stores of 2 bytes from 16 blocks.
constexpr int V_GROUP = 16;

__global__ void rope_kv_write_bf16_kernel(const bf16_t* in, bf16_t* out, const float2* __restrict__ table,
                                          const int32_t* __restrict__ slots, bf16_t* __restrict__ k_cache,
                                          bf16_t* __restrict__ v_cache, int tokens, int heads, int kv_heads, int dim,
                                          int block_size, int write) {
  const int64_t width = static_cast<int64_t>(heads + 2 * kv_heads) * dim;
  if (static_cast<int>(blockIdx.x) >= tokens) {
    const int t0 = (static_cast<int>(blockIdx.x) - tokens) * V_GROUP;
    const int n = min(V_GROUP, tokens - t0);
    const int64_t slot0 = slots[t0];
    // one run inside a page, a whole group, at a place where 16-byte stores are aligned?
    bool together = n == V_GROUP && block_size % 8 == 0 && slot0 % block_size % 8 == 0 &&
                    slot0 % block_size + V_GROUP <= block_size;
#pragma unroll
    for (int i = 1; i < V_GROUP; ++i) together = together && slots[min(t0 + i, tokens - 1)] == slot0 + i;
    const uint16_t* src = reinterpret_cast<const uint16_t*>(in) + static_cast<int64_t>(heads + kv_heads) * dim;
    uint16_t* cache = reinterpret_cast<uint16_t*>(v_cache);
    for (int item = threadIdx.x; item < kv_heads * dim; item += blockDim.x) {
      const int head = item / dim;
      const int d = item % dim;
      uint32_t v[V_GROUP];
#pragma unroll
      for (int i = 0; i < V_GROUP; ++i) v[i] = src[min(t0 + i, tokens - 1) * width + item];
      if (together) {
        const int64_t page = slot0 / block_size;
        uint16_t* dst = cache + ((page * kv_heads + head) * dim + d) * block_size + slot0 % block_size;
        *reinterpret_cast<uint4*>(dst) = uint4{v[0] | (v[1] << 16), v[2] | (v[3] << 16), v[4] | (v[5] << 16), v[6] | (v[7] << 16)};
        *reinterpret_cast<uint4*>(dst + 8) =
            uint4{v[8] | (v[9] << 16), v[10] | (v[11] << 16), v[12] | (v[13] << 16), v[14] | (v[15] << 16)};
      } else {
#pragma unroll
        for (int i = 0; i < V_GROUP; ++i) {
          if (i >= n) break;
          const int64_t slot = slots[t0 + i];
          const int64_t page = slot / block_size;
          cache[((page * kv_heads + head) * dim + d) * block_size + slot % block_size] = static_cast<uint16_t>(v[i]);
        }
      }
    }
    return;
  }
  const int64_t t = blockIdx.x;
  const bf16_t* src = in + t * width;
  bf16_t* row = out + t * width;
  const int64_t slot = write ? slots[t] : 0;
  const int64_t page = slot / block_size;
  const int offset = static_cast<int>(slot % block_size);
  const int half = dim / 2;
  const int per_head = half / 8;
  const int rotated_heads = heads + kv_heads;
  for (int i = threadIdx.x; i < rotated_heads * per_head; i += blockDim.x) {
    const int head = i / per_head;
    const int j0 = 8 * (i % per_head);
    const int64_t lo = static_cast<int64_t>(head) * dim + j0;
    const uint4 raw0 = *reinterpret_cast<const uint4*>(src + lo);
    const uint4 raw1 = *reinterpret_cast<const uint4*>(src + lo + half);
    const float4* angles = reinterpret_cast<const float4*>(table + t * half + j0);      // (cos, sin) x 8
    float4 cs[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) cs[e] = angles[e];
    float x0[8], x1[8], a[8], b[8];
    unpack8(raw0, x0);
    unpack8(raw1, x1);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      a[2 * e] = x0[2 * e] * cs[e].x - x1[2 * e] * cs[e].y;
      b[2 * e] = x1[2 * e] * cs[e].x + x0[2 * e] * cs[e].y;
      a[2 * e + 1] = x0[2 * e + 1] * cs[e].z - x1[2 * e + 1] * cs[e].w;
      b[2 * e + 1] = x1[2 * e + 1] * cs[e].z + x0[2 * e + 1] * cs[e].w;
    }
    const uint4 pa = pack8(a), pb = pack8(b);
    *reinterpret_cast<uint4*>(row + lo) = pa;
    *reinterpret_cast<uint4*>(row + lo + half) = pb;
    if (write && head >= heads) {
      bf16_t* at = k_cache + ((page * kv_heads + (head - heads)) * block_size + offset) * dim + j0;
      *reinterpret_cast<uint4*>(at) = pa;
      *reinterpret_cast<uint4*>(at + half) = pb;
    }
  }
  // v: copied (nothing to do in place); the blocks behind the tokens' write it into the cache
  if (row == src) return;
  const int v_items = kv_heads * (dim / 8);
  for (int i = threadIdx.x; i < v_items; i += blockDim.x) {
    const int64_t at = static_cast<int64_t>(rotated_heads) * dim + 8 * i;
    *reinterpret_cast<uint4*>(row + at) = *reinterpret_cast<const uint4*>(src + at);
  }
}

extern "C" int distie_rope_kv_write(const void* in, int in_dtype, int slices, void* out, int dtype, const void* table,
                                    const int32_t* positions, const int32_t* slots, void* k_cache, void* v_cache,
                                    int cache_dtype, const float* inv_freq, int pairs, int tokens, int heads,
                                    int kv_heads, int dim, int block_size, int write, hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (heads < 1 || kv_heads < 1 || dim < 1 || block_size < 1 || 2 * pairs > dim || pairs < 0 || slices < 1)
    return DISTIE_BAD_ARGUMENT;
  if (pairs > 0 && inv_freq == nullptr) return DISTIE_BAD_ARGUMENT;
  if (in == out && (slices != 1 || in_dtype != dtype)) return DISTIE_BAD_ARGUMENT;
  if (slices == 1 && in_dtype == DISTIE_BF16 && dtype == DISTIE_BF16 && cache_dtype == DISTIE_BF16 && dim % 16 == 0 &&
      2 * pairs == dim && table != nullptr && reinterpret_cast<uintptr_t>(in) % 16 == 0 &&
      reinterpret_cast<uintptr_t>(out) % 16 == 0 && reinterpret_cast<uintptr_t>(k_cache) % 16 == 0 &&
      reinterpret_cast<uintptr_t>(v_cache) % 16 == 0 &&
      reinterpret_cast<uintptr_t>(table) % 16 == 0) {
    const int items = (heads + kv_heads) * (dim / 16) + kv_heads * (dim / 8);
    const int threads = items >= 256 ? 256 : (items >= 128 ? 128 : 64);
    rope_kv_write_bf16_kernel<<<tokens + (write ? (tokens + V_GROUP - 1) / V_GROUP : 0), threads, 0, stream>>>(
        static_cast<const bf16_t*>(in), static_cast<bf16_t*>(out), static_cast<const float2*>(table), slots,
        static_cast<bf16_t*>(k_cache), static_cast<bf16_t*>(v_cache), tokens, heads, kv_heads, dim, block_size, write);
    return launch_status();
  }
  const int work = (heads + kv_heads) * dim / 2;
  int threads = work >= 512 ? 256 : (work >= 128 ? 128 : 64);
  if (slices > 1 && work >= 512) threads = work >= 1024 ? 1024 : 512;
  const int64_t stride = static_cast<int64_t>(tokens) * (heads + 2 * kv_heads) * dim;
  DISTIE_DISPATCH(in_dtype, I, DISTIE_DISPATCH(dtype, T, DISTIE_DISPATCH(cache_dtype, C,
      rope_kv_write_kernel<I, T, C><<<tokens, threads, 0, stream>>>(
          static_cast<const I*>(in), slices, stride, static_cast<T*>(out), static_cast<const float2*>(table),
          positions, slots,
          static_cast<C*>(k_cache), static_cast<C*>(v_cache), inv_freq, pairs, heads, kv_heads, dim, block_size,
          write))));
  return launch_status();
}

// ---------------------------------------------------------------- gated activation
// gate_up: [slices, rows, 2 * inter] (partial sums added in order) -> out [rows, inter]
template <typename I, typename T>
__global__ void silu_mul_kernel(const I* __restrict__ gate_up, int slices, int64_t slice_stride, T* __restrict__ out,
                                int64_t rows, int inter) {
  const int64_t total = rows * inter;
  for (int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; i < total;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    const int64_t r = i / inter;
    const int c = static_cast<int>(i % inter);
    const I* p = gate_up + r * 2 * inter + c;
    const float g = sum_strided(p, slices, slice_stride);
    const float u = sum_strided(p + inter, slices, slice_stride);
    out[i] = from_float<T>(g / (1.f + expf(-g)) * u);
  }
}

// bfloat16 in and out, one slice, inter a multiple of 8: 16-byte loads and stores
__global__ void silu_mul_bf16x8_kernel(const uint4* __restrict__ gate_up, uint4* __restrict__ out, int64_t rows,
                                       int inter8) {
  const int64_t total = rows * inter8;
  for (int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; i < total;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    const int64_t r = i / inter8;
    const int c = static_cast<int>(i % inter8);
    const uint4 g4 = gate_up[r * 2 * inter8 + c];
    const uint4 u4 = gate_up[r * 2 * inter8 + inter8 + c];
    const uint32_t gw[4] = {g4.x, g4.y, g4.z, g4.w}, uw[4] = {u4.x, u4.y, u4.z, u4.w};
    uint32_t ow[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float g0 = __uint_as_float(gw[e] << 16), g1 = __uint_as_float(gw[e] & 0xffff0000u);
      const float u0 = __uint_as_float(uw[e] << 16), u1 = __uint_as_float(uw[e] & 0xffff0000u);
      const bf16_t lo = static_cast<bf16_t>(g0 / (1.f + expf(-g0)) * u0);
      const bf16_t hi = static_cast<bf16_t>(g1 / (1.f + expf(-g1)) * u1);
      ow[e] = static_cast<uint32_t>(__builtin_bit_cast(uint16_t, lo)) |
              (static_cast<uint32_t>(__builtin_bit_cast(uint16_t, hi)) << 16);
    }
    out[i] = uint4{ow[0], ow[1], ow[2], ow[3]};
  }
}

extern "C" int distie_silu_mul(const void* gate_up, int in_dtype, int slices, void* out, int dtype, int rows,
                               int inter, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (inter <= 0 || slices < 1) return DISTIE_BAD_ARGUMENT;
  if (in_dtype == DISTIE_BF16 && dtype == DISTIE_BF16 && slices == 1 && inter % 8 == 0) {
    const int64_t pieces = static_cast<int64_t>(rows) * (inter / 8);
    const int blocks8 = static_cast<int>(pieces / 256 + 1 < 16384 ? pieces / 256 + 1 : 16384);
    silu_mul_bf16x8_kernel<<<blocks8, 256, 0, stream>>>(static_cast<const uint4*>(gate_up), static_cast<uint4*>(out),
                                                        rows, inter / 8);
    return launch_status();
  }
  const int64_t total = static_cast<int64_t>(rows) * inter;
  const int threads = 256;
  const int blocks = static_cast<int>(total / threads + 1 < 16384 ? total / threads + 1 : 16384);
  DISTIE_DISPATCH(in_dtype, I, DISTIE_DISPATCH(dtype, T, silu_mul_kernel<I, T><<<blocks, threads, 0, stream>>>(
      static_cast<const I*>(gate_up), slices, 2 * total, static_cast<T*>(out), rows, inter)));
  return launch_status();
}

// ---------------------------------------------------------------- sum of partial slices
template <typename T>
__global__ void sum_slices_kernel(const float* __restrict__ in, int slices, int64_t count, T* __restrict__ out) {
  for (int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; i < count;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    out[i] = from_float<T>(sum_strided(in + i, slices, count));
  }
}

extern "C" int distie_sum_slices(const float* in, int slices, int64_t count, void* out, int dtype,
                                 hipStream_t stream) {
  if (count <= 0) return 0;
  if (slices < 1) return DISTIE_BAD_ARGUMENT;
  const int blocks = static_cast<int>(count / 256 + 1 < 8192 ? count / 256 + 1 : 8192);
  DISTIE_DISPATCH(dtype, T, sum_slices_kernel<T><<<blocks, 256, 0, stream>>>(in, slices, count, static_cast<T*>(out)));
  return launch_status();
}

// ---------------------------------------------------------------- row gather
__global__ void gather_rows_kernel(const uint8_t* __restrict__ src, const int32_t* __restrict__ rows,
                                   uint8_t* __restrict__ dst, int64_t row_bytes, int src_rows) {
  const int64_t r = blockIdx.x;
  int64_t from = rows[r];
  if (from < 0 || from >= src_rows) from = 0;
  const uint8_t* s = src + from * row_bytes;
  uint8_t* d = dst + r * row_bytes;
  if ((row_bytes & 3) == 0) {
    const uint32_t* s4 = reinterpret_cast<const uint32_t*>(s);
    uint32_t* d4 = reinterpret_cast<uint32_t*>(d);
    for (int64_t i = threadIdx.x; i < row_bytes / 4; i += blockDim.x) d4[i] = s4[i];
  } else {
    for (int64_t i = threadIdx.x; i < row_bytes; i += blockDim.x) d[i] = s[i];
  }
}

extern "C" int distie_gather_rows(const void* src, const int32_t* rows, void* dst, int count, int64_t row_bytes,
                                  int src_rows, hipStream_t stream) {
  if (count <= 0) return 0;
  if (row_bytes <= 0 || src_rows <= 0) return DISTIE_BAD_ARGUMENT;
  gather_rows_kernel<<<count, 256, 0, stream>>>(static_cast<const uint8_t*>(src), rows,
                                                static_cast<uint8_t*>(dst), row_bytes, src_rows);
  return launch_status();
}

// ---------------------------------------------------------------- scattered int32 writes
// table[index[i]] = value[i]: how the block tables on the device follow the host's book-keeping (a step
// brings only the entries that changed since the step before). The indexes of one call are distinct.
__global__ void scatter_i32_kernel(int32_t* __restrict__ table, const int32_t* __restrict__ index,
                                   const int32_t* __restrict__ value, int count, int64_t size) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= count) return;
  const int64_t at = index[i];
  if (at >= 0 && at < size) table[at] = value[i];
}

extern "C" int distie_scatter_i32(int32_t* table, const int32_t* index, const int32_t* value, int count, int64_t size,
                                  hipStream_t stream) {
  if (count <= 0) return 0;
  if (size <= 0) return DISTIE_BAD_ARGUMENT;
  scatter_i32_kernel<<<(count + 255) / 256, 256, 0, stream>>>(table, index, value, count, size);
  return launch_status();
}
