// Attention over the paged cache for one head size (compile with -DDISTIE_HEAD_DIM=<even size up to 256>; the
// matrix-core kernels exist for multiples of 16 only, the wave-per-token kernel for every even size).
//
// out[t, h] = softmax_j(q[t, h] . k[j, h / G] * scale) v[j, h / G] over the keys j that token t may see:
// first(t) <= j <= position(t), first = 0, or position - window + 1 on a windowed layer. Keys and values
// are read through the block table of the token's request (row table_rows[request] of block_table, or row
// `request` itself when table_rows is null): key j lives in page table[j / P] at offset
// j % P of a cache laid out k [pages, kv_heads, P, D], v [pages, kv_heads, D, P]. The new tokens of the step are
// already in the cache
// (the reference writes before it reads too: worker/src/inference/qwen2/paged_attn.py:389-397), so
// prefill, portions of prompts and decoded tokens are the same computation.
// Formula: worker/src/inference/qwen2/model.py:154-161; softmax and all sums in float32.
//
//  * attn_generic: one wave per (token, head); any types; the true 32-bit path and the fallback.
//  * attn_decode + attn_reduce, attn_prefill: bfloat16 on the matrix cores (described further down).

#include "common.h"

#ifndef DISTIE_HEAD_DIM
#error "compile with -DDISTIE_HEAD_DIM=<head size>"
#endif
#if DISTIE_HEAD_DIM % 2 != 0 || DISTIE_HEAD_DIM < 2 || DISTIE_HEAD_DIM > 256
#error "head size must be even and at most 256"
#endif
#define DISTIE_MATRIX_CORE_ATTENTION (DISTIE_HEAD_DIM % 16 == 0)

constexpr int D = DISTIE_HEAD_DIM;
constexpr int DIMS_PER_LANE = (D + DISTIE_WAVE - 1) / DISTIE_WAVE;

extern "C" int distie_attention_head_dim() { return D; }

template <typename C>
__device__ __forceinline__ float dot_row(const float* q, const C* k);

template <>
__device__ __forceinline__ float dot_row<float>(const float* q, const float* k) {
  float s = 0.f;
  if constexpr (D % 4 != 0) {                  // rows are not 16-byte aligned: element by element
#pragma unroll
    for (int d = 0; d < D; ++d) s = fmaf(q[d], k[d], s);
    return s;
  }
#pragma unroll
  for (int d = 0; d + 4 <= D; d += 4) {
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
  if constexpr (D % 8 != 0) {
#pragma unroll
    for (int d = 0; d < D; ++d) s = fmaf(q[d], to_float(k[d]), s);
    return s;
  }
#pragma unroll
  for (int d = 0; d + 8 <= D; d += 8) {
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

// four consecutive values of a page's row of V^T as floats
__device__ __forceinline__ void load4(const float* p, float v[4]) {
  const float4 a = *reinterpret_cast<const float4*>(p);
  v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
}
__device__ __forceinline__ void load4(const bf16_t* p, float v[4]) {
  const uint2 raw = *reinterpret_cast<const uint2*>(p);
  v[0] = __uint_as_float(raw.x << 16); v[1] = __uint_as_float(raw.x & 0xffff0000u);
  v[2] = __uint_as_float(raw.y << 16); v[3] = __uint_as_float(raw.y & 0xffff0000u);
}

// One workgroup of WAVES waves per (token, head). The keys are taken in chunks of 64 that begin at multiples of
// 64; the chunks are dealt to the waves in turn (a token that decodes over thousands of keys then has eight
// waves at work instead of one), every wave keeps its own running maximum, sum and output, and wave 0 puts them
// together at the end, in wave order. In a chunk a lane owns one key for the scores; for the output it owns
// the dimensions lane, lane + 64, ... and walks the chunk's keys: a page at a time with 16-byte loads of the
// page's row of V^T when pages divide 64 and hold a multiple of four tokens, else key by key.
template <typename T, typename C, int WAVES>
__global__ __launch_bounds__(DISTIE_WAVE * WAVES) void attn_generic_kernel(
    const T* __restrict__ qkv, int64_t q_stride, const C* __restrict__ k_cache, const C* __restrict__ v_cache,
    const int32_t* __restrict__ positions, const int32_t* __restrict__ token_request,
    const int32_t* __restrict__ block_table, int table_width, const int32_t* __restrict__ table_rows, T* __restrict__ out, int heads, int kv_heads,
    int block_size, float scale, int window, const float* __restrict__ head_slopes, float score_cap) {
  __shared__ float q_s[D];
  __shared__ float p_s[WAVES][DISTIE_WAVE];
  __shared__ int64_t base_s[WAVES][DISTIE_WAVE];
  __shared__ float m_s[WAVES], l_s[WAVES];
  __shared__ float acc_s[WAVES][D];
  const int lane = threadIdx.x % DISTIE_WAVE;
  const int wave = threadIdx.x / DISTIE_WAVE;
  const int64_t t = blockIdx.x;
  const int h = blockIdx.y;
  const int kh = h / (heads / kv_heads);
  const int q_pos = positions[t];
  const int request_of_token = token_request[t];
  const int32_t* table = block_table + static_cast<int64_t>(table_rows != nullptr ? table_rows[request_of_token] : request_of_token) * table_width;
  const T* q = qkv + t * q_stride + static_cast<int64_t>(h) * D;
  for (int d = threadIdx.x; d < D; d += DISTIE_WAVE * WAVES) q_s[d] = to_float(q[d]);
  __syncthreads();

  const int first = window > 0 ? max(0, q_pos - window + 1) : 0;
  const int last = q_pos;   // inclusive
  const bool by_page = block_size % 4 == 0 && DISTIE_WAVE % block_size == 0;
  const float slope = head_slopes != nullptr ? head_slopes[h] : 0.f;
  float m = -INFINITY, l = 0.f;
  float acc[DIMS_PER_LANE];
#pragma unroll
  for (int i = 0; i < DIMS_PER_LANE; ++i) acc[i] = 0.f;

  for (int c = first / DISTIE_WAVE * DISTIE_WAVE + wave * DISTIE_WAVE; c <= last; c += DISTIE_WAVE * WAVES) {
    const int key = c + lane;
    const bool valid = key >= first && key <= last;
    float s = -INFINITY;
    int64_t base = 0;
    if (valid) {
      const int page = table[key / block_size];
      base = (static_cast<int64_t>(page) * kv_heads + kh) * block_size * D;
      s = dot_row<C>(q_s, k_cache + base + static_cast<int64_t>(key % block_size) * D) * scale;
      // what a variant of attention adds to a score (both off for plain attention): a cap that bends large
      // scores, then a bias by the distance to the key with the head's own slope
      if (score_cap > 0.f) s = score_cap * tanhf(s / score_cap);
      s += slope * static_cast<float>(key - q_pos);
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float alpha = m_new == -INFINITY ? 0.f : expf(m - m_new);     // 0 on the first chunk with a key (m = -inf)
    const float p = valid ? expf(s - m_new) : 0.f;
    l = l * alpha + wave_sum(p);
    m = m_new;
    // what the lanes of this wave hand each other goes through the wave's own rows of LDS; the wave runs its
    // LDS traffic in order, so no barrier across waves is needed, only that the compiler keeps the order
    __builtin_amdgcn_wave_barrier();
    p_s[wave][lane] = p;
    base_s[wave][lane] = base;
    __builtin_amdgcn_wave_barrier();
    const int lo = max(first - c, 0);                                   // keys lo .. hi of the chunk count
    const int hi = min(DISTIE_WAVE - 1, last - c);
#pragma unroll
    for (int i = 0; i < DIMS_PER_LANE; ++i) {
      const int d = lane + i * DISTIE_WAVE;
      if (d >= D) continue;
      float a = acc[i] * alpha;
      if (by_page) {
        for (int j0 = lo / block_size * block_size; j0 <= hi; j0 += block_size) {
          // the page of keys j0 .. j0 + P - 1: its address from a key of it that counts
          const C* row = v_cache + base_s[wave][max(j0, lo)] + static_cast<int64_t>(d) * block_size;
          for (int jj = 0; jj < block_size; jj += 4) {
            float v[4];
            load4(row + jj, v);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const int j = j0 + jj + e;
              if (j >= lo && j <= hi) a = fmaf(p_s[wave][j], v[e], a);    // never a value of a key that does not count
            }
          }
        }
      } else {
        for (int j = lo; j <= hi; ++j)
          a = fmaf(p_s[wave][j], to_float(v_cache[base_s[wave][j] + static_cast<int64_t>(d) * block_size + (c + j) % block_size]), a);
      }
      acc[i] = a;
    }
  }
  T* o = out + (t * heads + h) * D;
  if constexpr (WAVES == 1) {
    const float inv = 1.f / l;
#pragma unroll
    for (int i = 0; i < DIMS_PER_LANE; ++i) {
      const int d = lane + i * DISTIE_WAVE;
      if (d < D) o[d] = from_float<T>(acc[i] * inv);
    }
  } else {
    if (lane == 0) {
      m_s[wave] = m;
      l_s[wave] = l;
    }
#pragma unroll
    for (int i = 0; i < DIMS_PER_LANE; ++i) {
      const int d = lane + i * DISTIE_WAVE;
      if (d < D) acc_s[wave][d] = acc[i];
    }
    __syncthreads();
    if (wave != 0) return;
    float top = -INFINITY;
    for (int w = 0; w < WAVES; ++w) top = fmaxf(top, m_s[w]);
    float total = 0.f;
    float weight[WAVES];
    for (int w = 0; w < WAVES; ++w) {
      weight[w] = m_s[w] == -INFINITY ? 0.f : expf(m_s[w] - top);       // a wave without keys counts nothing
      total += l_s[w] * weight[w];
    }
    const float inv = 1.f / total;
#pragma unroll
    for (int i = 0; i < DIMS_PER_LANE; ++i) {
      const int d = lane + i * DISTIE_WAVE;
      if (d >= D) continue;
      float sum = 0.f;
      for (int w = 0; w < WAVES; ++w) sum += acc_s[w][d] * weight[w];
      o[d] = from_float<T>(sum * inv);
    }
  }
}

// The same walk in float32 for requests that decode, with loads that cover whole rows: one workgroup per
// (token, kv head, part of up to G query heads of it). For the scores eight lanes share a key: each reads an
// eighth of the key's row of K (a run of D / 8 floats, so a wave's load covers eight whole rows; with a lane
// to a key every 16-byte load of a wave touched 64 lines) against its slices of the heads' queries, which it
// keeps in registers; the sums of the eight lanes are added by three exchanges. With G > 1 every row of K
// and every value of V^T is read once for G heads; the caller takes G as large as leaves enough workgroups.
constexpr bool GQ_FITS = D % 32 == 0;
constexpr int GQ_SLICE = GQ_FITS ? D / 8 : 4;

template <int G, int WAVES>
__global__ __launch_bounds__(DISTIE_WAVE * WAVES) void attn_grouped_f32_kernel(
    const float* __restrict__ qkv, int64_t q_stride, const float* __restrict__ k_cache, const float* __restrict__ v_cache,
    const int32_t* __restrict__ positions, const int32_t* __restrict__ token_request,
    const int32_t* __restrict__ block_table, int table_width, const int32_t* __restrict__ table_rows,
    float* __restrict__ out, int heads, int kv_heads, int parts, int block_size, float scale, int window) {
  __shared__ float p_s[WAVES][G][DISTIE_WAVE];
  __shared__ int64_t base_s[WAVES][DISTIE_WAVE];
  __shared__ float m_s[WAVES][G], l_s[WAVES][G];
  __shared__ float acc_s[WAVES][G][D];
  const int lane = threadIdx.x % DISTIE_WAVE;
  const int wave = threadIdx.x / DISTIE_WAVE;
  const int64_t t = blockIdx.x;
  const int group = heads / kv_heads;
  const int kh = blockIdx.y / parts;
  const int g0 = (blockIdx.y % parts) * G;
  const int n = min(G, group - g0);                        // heads of this part
  const int h0 = kh * group + g0;
  const int q_pos = positions[t];
  const int request_of_token = token_request[t];
  const int32_t* table = block_table + static_cast<int64_t>(table_rows != nullptr ? table_rows[request_of_token] : request_of_token) * table_width;
  const int sub = lane % 8;                                // which eighth of a row
  const int key_in_pass = lane / 8;
  float q_r[G][GQ_SLICE];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    const float* q = qkv + t * q_stride + static_cast<int64_t>(h0 + min(g, n - 1)) * D + sub * GQ_SLICE;
#pragma unroll
    for (int d = 0; d < GQ_SLICE; d += 4) {
      const float4 v = *reinterpret_cast<const float4*>(q + d);
      q_r[g][d] = v.x; q_r[g][d + 1] = v.y; q_r[g][d + 2] = v.z; q_r[g][d + 3] = v.w;
    }
  }
  const int first = window > 0 ? max(0, q_pos - window + 1) : 0;
  const int last = q_pos;   // inclusive
  float m[G], l[G];
  float acc[G][DIMS_PER_LANE];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    m[g] = -INFINITY;
    l[g] = 0.f;
#pragma unroll
    for (int i = 0; i < DIMS_PER_LANE; ++i) acc[g][i] = 0.f;
  }

  for (int c = first / DISTIE_WAVE * DISTIE_WAVE + wave * DISTIE_WAVE; c <= last; c += DISTIE_WAVE * WAVES) {
    // Every load of a phase is issued before its results are used (a chunk costs a few trips to memory, not one
    // for every pass and page): lane j looks up the page of key c + j, the addresses go from lane to lane.
    const int key = c + lane;
    const bool valid = key >= first && key <= last;
    int64_t base = 0, row = 0;                              // keys that do not count read the start of the cache
    if (valid) {
      const int page = table[key / block_size];
      base = (static_cast<int64_t>(page) * kv_heads + kh) * block_size * D;
      row = base + static_cast<int64_t>(key % block_size) * D;
    }
    // ---- scores: eight keys a pass, four passes of loads in flight; afterwards lane j holds the scores of key c + j
    float s[G];
#pragma unroll
    for (int g = 0; g < G; ++g) s[g] = 0.f;
    constexpr int ROUND = G == 1 ? 8 : 4;                 // passes whose loads are in flight together: what the registers allow
#pragma unroll
    for (int round = 0; round < 8 / ROUND; ++round) {
      float4 kk[ROUND][GQ_SLICE / 4];
#pragma unroll
      for (int ps = 0; ps < ROUND; ++ps) {
        const int64_t from = __shfl(row, 8 * (ROUND * round + ps) + key_in_pass, DISTIE_WAVE);
        const float* k = k_cache + from + sub * GQ_SLICE;
#pragma unroll
        for (int d = 0; d < GQ_SLICE / 4; ++d) kk[ps][d] = *reinterpret_cast<const float4*>(k + 4 * d);
      }
      __builtin_amdgcn_sched_barrier(0);                    // all of these loads are under way before the first is used
#pragma unroll
      for (int ps = 0; ps < ROUND; ++ps) {
        const int pass = ROUND * round + ps;
#pragma unroll
        for (int g = 0; g < G; ++g) {
          float v = 0.f;
#pragma unroll
          for (int d = 0; d < GQ_SLICE / 4; ++d) {
            v = fmaf(q_r[g][4 * d], kk[ps][d].x, v);
            v = fmaf(q_r[g][4 * d + 1], kk[ps][d].y, v);
            v = fmaf(q_r[g][4 * d + 2], kk[ps][d].z, v);
            v = fmaf(q_r[g][4 * d + 3], kk[ps][d].w, v);
          }
          v += __shfl_xor(v, 1, DISTIE_WAVE);
          v += __shfl_xor(v, 2, DISTIE_WAVE);
          v += __shfl_xor(v, 4, DISTIE_WAVE);
          // the lane that owns this key for the softmax is lane 8 pass + (the key's place in the pass)
          const float mine = __shfl(v, (lane % 8) * 8, DISTIE_WAVE);
          if (lane / 8 == pass) s[g] = mine;
        }
      }
    }
    float alpha[G];
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int g = 0; g < G; ++g) {
      const float sg = valid && g < n ? s[g] * scale : -INFINITY;
      const float m_new = fmaxf(m[g], wave_max(sg));
      alpha[g] = m_new == -INFINITY ? 0.f : expf(m[g] - m_new);     // 0 on the first chunk with a key (m = -inf)
      const float p = valid && g < n ? expf(sg - m_new) : 0.f;
      l[g] = l[g] * alpha[g] + wave_sum(p);
      m[g] = m_new;
      p_s[wave][g][lane] = p;
    }
    base_s[wave][lane] = base;
    __builtin_amdgcn_wave_barrier();
    // ---- output: the lane owns dimensions lane, lane + 64, ...; the chunk's values of a dimension are 16 pieces
    // of four keys (a piece lies in one page: pages hold a multiple of four tokens)
    const int lo = max(first - c, 0);                                   // keys lo .. hi of the chunk count
    const int hi = min(DISTIE_WAVE - 1, last - c);
#pragma unroll
    for (int i = 0; i < DIMS_PER_LANE; ++i) {
      const int d = lane + i * DISTIE_WAVE;
      if (d >= D) continue;
      float a[G];
#pragma unroll
      for (int g = 0; g < G; ++g) a[g] = acc[g][i] * alpha[g];
      constexpr int GQ_PIECES = G == 1 ? 16 : 8;            // 16-byte pieces of V^T whose loads are in flight together
#pragma unroll
      for (int part = 0; part < 16 / GQ_PIECES; ++part) {
        float4 vv[GQ_PIECES];
#pragma unroll
        for (int u = 0; u < GQ_PIECES; ++u) {
          const int q = part * GQ_PIECES + u;
          const int64_t page_base = base_s[wave][min(max(4 * q, lo), hi)];      // of a key that counts
          vv[u] = *reinterpret_cast<const float4*>(v_cache + page_base + static_cast<int64_t>(d) * block_size +
                                                   (c + 4 * q) % block_size);
        }
        __builtin_amdgcn_sched_barrier(0);                  // all of these loads are under way before the first is used
#pragma unroll
        for (int g = 0; g < G; ++g) {
#pragma unroll
          for (int u = 0; u < GQ_PIECES; ++u) {
            const int q = part * GQ_PIECES + u;
            const float4 pp = *reinterpret_cast<const float4*>(&p_s[wave][g][4 * q]);
            const float v[4] = {vv[u].x, vv[u].y, vv[u].z, vv[u].w};
            const float w[4] = {pp.x, pp.y, pp.z, pp.w};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const int j = 4 * q + e;
              // never a value of a key that does not count (a weight of zero times what lies there could be NaN)
              a[g] = fmaf(w[e], (j >= lo && j <= hi) ? v[e] : 0.f, a[g]);
            }
          }
        }
      }
#pragma unroll
      for (int g = 0; g < G; ++g) acc[g][i] = a[g];
    }
  }
  // ---- the waves' parts, put together by wave 0 in wave order
  if (lane == 0) {
#pragma unroll
    for (int g = 0; g < G; ++g) {
      m_s[wave][g] = m[g];
      l_s[wave][g] = l[g];
    }
  }
#pragma unroll
  for (int g = 0; g < G; ++g)
#pragma unroll
    for (int i = 0; i < DIMS_PER_LANE; ++i) {
      const int d = lane + i * DISTIE_WAVE;
      if (d < D) acc_s[wave][g][d] = acc[g][i];
    }
  __syncthreads();
  // wave w writes heads w, w + WAVES, ... of the part
  for (int g = wave; g < n; g += WAVES) {
    float top = -INFINITY;
    for (int w = 0; w < WAVES; ++w) top = fmaxf(top, m_s[w][g]);
    float total = 0.f;
    float weight[WAVES];
    for (int w = 0; w < WAVES; ++w) {
      weight[w] = m_s[w][g] == -INFINITY ? 0.f : expf(m_s[w][g] - top);    // a wave without keys counts nothing
      total += l_s[w][g] * weight[w];
    }
    const float inv = 1.f / total;
    float* o = out + (t * heads + h0 + g) * D;
#pragma unroll
    for (int i = 0; i < DIMS_PER_LANE; ++i) {
      const int d = lane + i * DISTIE_WAVE;
      if (d >= D) continue;
      float sum = 0.f;
      for (int w = 0; w < WAVES; ++w) sum += acc_s[w][g][d] * weight[w];
      o[d] = sum * inv;
    }
  }
}

// qkv: [T, q_stride] with q of head h at columns h*D; out: [T, heads*D]. window = 0: every earlier key.
// head_slopes (float32 [heads], may be null): score += slope[h] * (key - position); score_cap > 0: the scaled score
// goes through cap * tanh(score / cap) first. Only this kernel takes the two.
extern "C" int distie_attention_generic(const void* qkv, int dtype, int64_t q_stride, const void* k_cache,
                                        const void* v_cache, int cache_dtype, const int32_t* positions,
                                        const int32_t* token_request, const int32_t* block_table,
                                        int table_width, const int32_t* table_rows, void* out, int tokens, int heads, int kv_heads,
                                        int block_size, float scale, int window, const float* head_slopes,
                                        float score_cap, hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (heads < 1 || kv_heads < 1 || heads % kv_heads != 0 || block_size < 1 || table_width < 1 || window < 0 ||
      score_cap < 0.f)
    return DISTIE_BAD_ARGUMENT;
  const bool plain_scores = head_slopes == nullptr && score_cap == 0.f;
  if (heads > 65535) return DISTIE_BAD_ARGUMENT;
  dim3 grid(tokens, heads);
  const int group = heads / kv_heads;
  if (plain_scores && GQ_FITS && dtype == DISTIE_F32 && cache_dtype == DISTIE_F32 && q_stride % 4 == 0 && block_size % 4 == 0 &&
      DISTIE_WAVE % block_size == 0 && static_cast<int64_t>(tokens) * heads < 2048) {
    // requests that decode, float32: as many heads of a kv head to a workgroup as leaves a workgroup a compute unit
    int per = 1;
    for (int g : {2, 4})
      if (group >= g && static_cast<int64_t>(tokens) * kv_heads * ((group + g - 1) / g) >= 256) per = g;
    const int parts = (group + per - 1) / per;
    const dim3 grouped(tokens, kv_heads * parts);
#define DISTIE_GROUPED(G, WAVES)                                                                                   \
    attn_grouped_f32_kernel<G, WAVES><<<grouped, DISTIE_WAVE * WAVES, 0, stream>>>(                                  \
        static_cast<const float*>(qkv), q_stride, static_cast<const float*>(k_cache),                               \
        static_cast<const float*>(v_cache), positions, token_request, block_table, table_width, table_rows,         \
        static_cast<float*>(out), heads, kv_heads, parts, block_size, scale, window)
    if (per == 4) DISTIE_GROUPED(4, 8);
    else if (per == 2) DISTIE_GROUPED(2, 8);
    else DISTIE_GROUPED(1, 8);
#undef DISTIE_GROUPED
    return launch_status();
  }
  // few (token, head) pairs, as when requests decode: eight waves share each pair's keys
  if (static_cast<int64_t>(tokens) * heads < 2048) {
    DISTIE_DISPATCH(dtype, T, DISTIE_DISPATCH(cache_dtype, C,
        (attn_generic_kernel<T, C, 8><<<grid, DISTIE_WAVE * 8, 0, stream>>>(
            static_cast<const T*>(qkv), q_stride, static_cast<const C*>(k_cache), static_cast<const C*>(v_cache),
            positions, token_request, block_table, table_width, table_rows, static_cast<T*>(out), heads, kv_heads, block_size,
            scale, window, head_slopes, score_cap))));
  } else {
    DISTIE_DISPATCH(dtype, T, DISTIE_DISPATCH(cache_dtype, C,
        (attn_generic_kernel<T, C, 1><<<grid, DISTIE_WAVE, 0, stream>>>(
            static_cast<const T*>(qkv), q_stride, static_cast<const C*>(k_cache), static_cast<const C*>(v_cache),
            positions, token_request, block_table, table_width, table_rows, static_cast<T*>(out), heads, kv_heads, block_size,
            scale, window, head_slopes, score_cap))));
  }
  return launch_status();
}

#if DISTIE_MATRIX_CORE_ATTENTION
// ===================================================================================================
//  Matrix-core kernels (bfloat16, pages of a multiple of 16 tokens). The decode kernel works on 16-wide
//  blocks of "columns" against blocks of 16 keys with two products (the tiled kernel for portions of prompts
//  does the same with 32-wide blocks and is described where it stands):
//        S^T[key, col] = K[key, :] . q[col, :]        (v_mfma_f32_16x16x32_bf16, K rows as the A operand)
//        online softmax over keys, per column, in float32 (weights as 2^x: scores are scaled by log2 e)
//        O[col, d]  += P[col, key] . V^T[d, key]      (values are stored transposed inside a page, so the
//                                                      summed index, the key, is contiguous for the B operand)
//  A lane holds, of a 16 x 16 score tile, keys 4g..4g+3 of column r (r = lane % 16, g = lane / 16): exactly
//  the shape of the A operand of the second product if its 32 summed keys are taken in the order
//  (block 0: 4g..4g+3, block 1: 4g..4g+3); the values are read in the same order, so no data moves
//  between lanes except the maxima and the rescaling factors.
//
//  * attn_decode: requests that bring one token. Columns = the G query heads that share one kv head. The
//    keys of a request are cut into runs of equal length, one wave each (this is where the parallelism comes from when
//    few requests decode); a wave takes its run in chunks of DC_KEYS keys and issues every load of a chunk
//    (pages, K rows, V^T rows) before it computes, so a chunk costs one trip to memory. It writes
//    unnormalised partial results that attn_reduce combines.
// ===================================================================================================
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(short)))) short shortx4;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;
typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t uintx4;

// 2^x in one instruction (v_exp_f32; float32, about 1 ulp; -inf gives 0)
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

constexpr int DK32 = D / 32;            // full 32-wide steps of the q.k product
constexpr bool DK_TAIL = (D % 32) != 0; // one more step of 16
constexpr int DB16 = D / 16;            // 16-wide blocks of the output
constexpr int DC_BLOCKS = (D <= 128) ? 4 : 2;   // blocks of 16 keys whose loads are in flight together
constexpr int DC_KEYS = 16 * DC_BLOCKS;

// How one request's keys are cut into runs. The visible keys (all of them, or the window's), counted from the
// 64-key boundary at or before the first of them, are cut into at most `max_splits` runs of one length, a
// multiple of RUN_STEP: the request's own length decides, not the longest of the batch, so that every request
// keeps all of its waves busy whatever else the step holds. Both kernels derive the same numbers.
constexpr int RUN_STEP = 64;            // a multiple of DC_KEYS for every head size
struct KeyRuns {
  int first;      // first visible key
  int origin;     // where run 0 begins
  int length;     // keys per run
  int count;      // runs that hold a key
};
// run_len > 0: runs of this length for every request (`decode_run_len_kernel`), so that a long request gets more of them
// than a short one; the caller made it long enough for the longest request to fit max_splits runs.
__device__ __forceinline__ KeyRuns key_runs(int q_pos, int window, int max_splits, int run_len = 0) {
  KeyRuns runs;
  runs.first = window > 0 ? max(0, q_pos - window + 1) : 0;
  runs.origin = runs.first / RUN_STEP * RUN_STEP;
  const int span = q_pos - runs.origin + 1;
  const int step = max_splits * RUN_STEP;
  runs.length = run_len > 0 ? run_len : (span + step - 1) / step * RUN_STEP;        // ceil(span / max_splits), rounded up to RUN_STEP
  runs.count = (span + runs.length - 1) / runs.length;      // <= max_splits
  return runs;
}

// One run length for all requests of a step (no window): the shortest, in steps of 64 keys, with which the runs of
// all requests together are at most `budget` (the waves the caller wants at work, per kv head) and no request has
// more than `max_splits`. A long request then gets more runs than a short one; with every request cut into the
// same number of runs the runs of the longest end last, alone. The caller uses it where that same number would
// leave many of the waves unused (256 requests of 1,050 to 3,150 keys on 4 kv heads, one run each: 263 us, with one
// run length 245); requests of one length are cut exactly as without it. It is the same for every layer of a step,
// so one wave finds it once a step and the attention kernels read it beside their request's length (found by
// every wave of theirs it cost 3 to 10 us a call).
__global__ __launch_bounds__(DISTIE_WAVE) void decode_run_len_kernel(const int32_t* __restrict__ kv_len, int num_requests,
                                                                     int budget, int max_splits, int32_t* __restrict__ run_len) {
  const int lane = threadIdx.x;
  int most = 1;
  for (int i = lane; i < num_requests; i += DISTIE_WAVE) most = max(most, kv_len[i]);
#pragma unroll
  for (int o = DISTIE_WAVE / 2; o > 0; o >>= 1) most = max(most, __shfl_xor(most, o, DISTIE_WAVE));
  // in units of RUN_STEP keys: from what the longest request needs to fit max_splits runs, up to one run a request
  int lo = (most + max_splits * RUN_STEP - 1) / (max_splits * RUN_STEP);
  int hi = (most + RUN_STEP - 1) / RUN_STEP;
  while (lo < hi) {                                     // (the same in every lane)
    const int mid = (lo + hi) / 2;
    int runs = 0;
    for (int i = lane; i < num_requests; i += DISTIE_WAVE) runs += (kv_len[i] + mid * RUN_STEP - 1) / (mid * RUN_STEP);
#pragma unroll
    for (int o = DISTIE_WAVE / 2; o > 0; o >>= 1) runs += __shfl_xor(runs, o, DISTIE_WAVE);
    if (runs <= budget) {
      hi = mid;
    } else {
      lo = mid + 1;
    }
  }
  if (lane == 0) *run_len = lo * RUN_STEP;
}

// run_len: int32 [1], for a step of num_requests requests that bring one token each.
extern "C" int distie_attention_decode_run_len(const int32_t* kv_len, int num_requests, int budget, int max_splits,
                                               int32_t* run_len, hipStream_t stream) {
  if (num_requests < 1 || budget < 1 || max_splits < 1 || kv_len == nullptr || run_len == nullptr) return DISTIE_BAD_ARGUMENT;
  decode_run_len_kernel<<<1, DISTIE_WAVE, 0, stream>>>(kv_len, num_requests, budget, max_splits, run_len);
  return launch_status();
}

// Two waves a SIMD where the registers allow it without spilling (one block of query heads, head sizes up to 128:
// 234 registers; left to itself the compiler took a few more and one wave a SIMD). The chip then holds 2,048 waves
// instead of 1,024, and a batch whose runs are a few more than 1,024, or whose requests differ in length, no
// longer waits for the last waves to get a place: 7B shape's heads at 2,100 keys, 96 requests 91 -> 83 us a layer,
// 160 requests 165 -> 130; contexts of 1,050 to 3,150 keys, 96 requests 121 -> 96, 160 requests 222 -> 157.
template <int MB>
__global__ __launch_bounds__(DISTIE_WAVE, (MB == 1 && D <= 128 ? 2 : 1)) void attn_decode_kernel(
    const bf16_t* __restrict__ qkv, int64_t q_stride, const bf16_t* __restrict__ k_cache,
    const bf16_t* __restrict__ v_cache, const int32_t* __restrict__ kv_len, const int32_t* __restrict__ cu_q,
    const int32_t* __restrict__ block_table, int table_width, const int32_t* __restrict__ table_rows, float* __restrict__ part_o,
    float* __restrict__ part_ml, int heads, int kv_heads, int block_size, float scale, int window, int split_hint,
    int max_splits, int dense_rows, const int32_t* __restrict__ shared_run_len) {
  const int lane = threadIdx.x;
  const int r = lane % 16;
  const int g = lane / 16;
  const int group = heads / kv_heads;
  const float scale_log2 = scale * 1.4426950408889634f;
  // With a shared run length the run is the slowest index of the grid: the places past a request's last run, whose
  // waves leave at once, then come after all the others (in front of them they held the places on the SIMDs that
  // the working waves behind them were waiting for: 64 requests took 106 us instead of 54, at one wave a SIMD).
  const bool shared = shared_run_len != nullptr;
  const int run = shared ? blockIdx.z : blockIdx.x;
  const int request = shared ? blockIdx.y : blockIdx.z;
  const int kh = shared ? blockIdx.x : blockIdx.y;
  const int32_t* table = block_table + static_cast<int64_t>(table_rows != nullptr ? table_rows[request] : request) * table_width;
  // The pages of the run's first chunk are asked for before the request's length says where the run begins:
  // at the place it has if the runs are `split_hint` long and begin at key 0, which the host derives from the
  // longest request of the step (the entry is inside the table either way). Where the guess holds, which it
  // does when few requests of similar length decode, that is one trip to memory less on the way to the keys.
  const int guess_begin = run * split_hint;
  int pages[DC_BLOCKS];
#pragma unroll
  for (int b = 0; b < DC_BLOCKS; ++b) pages[b] = table[min((guess_begin + 16 * b) / block_size, table_width - 1)];
  // dense_rows: every request brings one token, so request i's token is row i
  const int run_len = shared ? *shared_run_len : 0;
  const int token = dense_rows ? request : cu_q[request];
  if (!dense_rows && cu_q[request + 1] - token != 1) return;        // a portion of a prompt: the tiled kernel's
  const int q_pos = kv_len[request] - 1;              // the new token is the last one cached
  const KeyRuns runs = key_runs(q_pos, window, max_splits, run_len);
  if (run >= runs.count) return;
  const int run_begin = runs.origin + run * runs.length;
  const int key_begin = max(runs.first, run_begin);
  const int key_end = min(q_pos, run_begin + runs.length - 1);

  // ---- the query of this lane's column (head kh * G + 16 mb + r; columns past the group repeat the last)
  bf16x8 q_reg[MB][DK32 > 0 ? DK32 : 1];
  shortx4 q_tail[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    const int col = min(16 * mb + r, group - 1);
    const bf16_t* q = qkv + token * q_stride + static_cast<int64_t>(kh * group + col) * D;
#pragma unroll
    for (int dk = 0; dk < DK32; ++dk) q_reg[mb][dk] = *reinterpret_cast<const bf16x8*>(q + 32 * dk + 8 * g);
    if (DK_TAIL) q_tail[mb] = *reinterpret_cast<const shortx4*>(q + (D - 16) + 4 * g);
  }
  floatx4 o_acc[MB][DB16];
  float m_run[MB], l_run[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    m_run[mb] = -INFINITY;
    l_run[mb] = 0.f;
#pragma unroll
    for (int db = 0; db < DB16; ++db) o_acc[mb][db] = floatx4{0.f, 0.f, 0.f, 0.f};
  }

  // every chunk of the walk holds at least one visible key (the running maximum is then finite): under a
  // window the walk starts at the chunk of the first visible key, whose pages are asked for now
  const int chunk_begin = max(run_begin, key_begin / DC_KEYS * DC_KEYS);      // runs begin at multiples of DC_KEYS
  if (chunk_begin != guess_begin) {
#pragma unroll
    for (int b = 0; b < DC_BLOCKS; ++b) pages[b] = table[min((chunk_begin + 16 * b) / block_size, table_width - 1)];
  }
  for (int chunk = chunk_begin; chunk <= key_end; chunk += DC_KEYS) {
    // ---- every load of the chunk first
    bool live[DC_BLOCKS];
    bf16x8 k_reg[DC_BLOCKS][DK32 > 0 ? DK32 : 1];
    shortx4 k_tail[DC_BLOCKS];
    uint2 v_reg[DC_BLOCKS][DB16];
#pragma unroll
    for (int b = 0; b < DC_BLOCKS; ++b) {
      const int key0 = chunk + 16 * b;
      live[b] = key0 <= key_end && key0 + 15 >= key_begin;      // a block outside the run may have no page
#pragma unroll
      for (int dk = 0; dk < DK32; ++dk) k_reg[b][dk] = bf16x8{};
      k_tail[b] = shortx4{};
#pragma unroll
      for (int db = 0; db < DB16; ++db) v_reg[b][db] = uint2{0u, 0u};
      if (!live[b]) continue;
      const int page = pages[b];
      const int64_t page_base = (static_cast<int64_t>(page) * kv_heads + kh) * block_size * D;
      const int offset = key0 % block_size;
      const bf16_t* k_row = k_cache + page_base + static_cast<int64_t>(offset + r) * D;
#pragma unroll
      for (int dk = 0; dk < DK32; ++dk) k_reg[b][dk] = *reinterpret_cast<const bf16x8*>(k_row + 32 * dk + 8 * g);
      if (DK_TAIL) k_tail[b] = *reinterpret_cast<const shortx4*>(k_row + (D - 16) + 4 * g);
      // Slots after the run's last key were never written by this request: what a former owner of the page
      // left there must not even be multiplied by a weight of zero (0 * NaN), so those values are cleared.
      const int written = key_end - (key0 + 4 * g) + 1;          // of this lane's four keys
      const uint32_t keep_lo = written >= 2 ? 0xffffffffu : (written == 1 ? 0x0000ffffu : 0u);
      const uint32_t keep_hi = written >= 4 ? 0xffffffffu : (written == 3 ? 0x0000ffffu : 0u);
      const bf16_t* v_col = v_cache + page_base + offset + 4 * g;
#pragma unroll
      for (int db = 0; db < DB16; ++db) {
        const uint2 raw = *reinterpret_cast<const uint2*>(v_col + static_cast<int64_t>(16 * db + r) * block_size);
        v_reg[b][db] = uint2{raw.x & keep_lo, raw.y & keep_hi};
      }
    }
    // the next chunk's pages, while this chunk's keys and values are on their way
    if (chunk + DC_KEYS <= key_end) {
#pragma unroll
      for (int b = 0; b < DC_BLOCKS; ++b)
        pages[b] = table[min((chunk + DC_KEYS + 16 * b) / block_size, table_width - 1)];
    }
    // ---- scores
    floatx4 s[MB][DC_BLOCKS];
#pragma unroll
    for (int b = 0; b < DC_BLOCKS; ++b) {
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) s[mb][b] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int dk = 0; dk < DK32; ++dk)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
          s[mb][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(k_reg[b][dk], q_reg[mb][dk], s[mb][b], 0, 0, 0);
      if (DK_TAIL) {
        // The last 16 dims go through the 16-deep instruction into an accumulator of their own, added on the
        // vector ALU: chained straight onto the 32-deep instruction's accumulator, the first two of its
        // four registers were read before they were written (results depended on timing).
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
          const floatx4 tail = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(k_tail[b], q_tail[mb], floatx4{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
#pragma unroll
          for (int i = 0; i < 4; ++i) s[mb][b][i] += tail[i];
        }
      }
    }
    // ---- softmax step per column
    bf16x8 p_reg[MB][DC_BLOCKS / 2];
    float alpha[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      float best = -INFINITY;
#pragma unroll
      for (int b = 0; b < DC_BLOCKS; ++b)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int key = chunk + 16 * b + 4 * g + i;
          const float v = (key >= key_begin && key <= key_end) ? s[mb][b][i] * scale_log2 : -INFINITY;
          s[mb][b][i] = v;
          best = fmaxf(best, v);
        }
      best = fmaxf(best, __shfl_xor(best, 16, DISTIE_WAVE));
      best = fmaxf(best, __shfl_xor(best, 32, DISTIE_WAVE));
      const float m_new = fmaxf(m_run[mb], best);      // finite: every chunk of the run holds a key
      alpha[mb] = fast_exp2(m_run[mb] - m_new);        // 0 while m_run is -inf
      float sum = 0.f;
#pragma unroll
      for (int b = 0; b < DC_BLOCKS; ++b)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float p = fast_exp2(s[mb][b][i] - m_new);
          sum += p;
          p_reg[mb][b / 2][4 * (b % 2) + i] = static_cast<bf16_t>(p);
        }
      l_run[mb] = l_run[mb] * alpha[mb] + sum;      // the lanes of a column each keep a part of the sum
      m_run[mb] = m_new;
    }
    // ---- rescale what is there; the lane holds columns 4g..4g+3 of each output block
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      float a4[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a4[i] = __shfl(alpha[mb], 4 * g + i, DISTIE_WAVE);
#pragma unroll
      for (int db = 0; db < DB16; ++db)
#pragma unroll
        for (int i = 0; i < 4; ++i) o_acc[mb][db][i] *= a4[i];
    }
    // ---- O += P . V, 32 keys (two blocks) a step; the vector is put together as whole 32-bit words
#pragma unroll
    for (int ks = 0; ks < DC_BLOCKS / 2; ++ks)
#pragma unroll
      for (int db = 0; db < DB16; ++db) {
        const uintx4 words = {v_reg[2 * ks][db].x, v_reg[2 * ks][db].y, v_reg[2 * ks + 1][db].x, v_reg[2 * ks + 1][db].y};
        const bf16x8 v = __builtin_bit_cast(bf16x8, words);
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
          o_acc[mb][db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(p_reg[mb][ks], v, o_acc[mb][db], 0, 0, 0);
      }
  }

  // ---- sums over the lanes of a column, then the partial result of this run
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    l_run[mb] += __shfl_xor(l_run[mb], 16, DISTIE_WAVE);
    l_run[mb] += __shfl_xor(l_run[mb], 32, DISTIE_WAVE);
  }
#pragma unroll
  for (int mb = 0; mb < MB; ++mb)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int col = 16 * mb + 4 * g + i;
      const float l_col = __shfl(l_run[mb], 4 * g + i, DISTIE_WAVE);
      const float m_col = __shfl(m_run[mb], 4 * g + i, DISTIE_WAVE);
      if (col >= group) continue;
      const int64_t slot = (static_cast<int64_t>(request) * heads + kh * group + col) * max_splits + run;
      float* po = part_o + slot * D;
#pragma unroll
      for (int db = 0; db < DB16; ++db) po[16 * db + r] = o_acc[mb][db][i];
      if (r == 0) {
        part_ml[2 * slot] = m_col;
        part_ml[2 * slot + 1] = l_col;
      }
    }
}

// Combines the partial results of the runs of keys of one (request, head): grid (heads, requests), four waves.
// All threads first find the maximum and the weight of every run; then each wave adds a quarter of the runs
// (in order) for the output dims its lanes own, and the four sums are added in order through LDS.
// FAST (at most RD_FAST_RUNS runs fit the buffers): every partial result the block may need is asked for at
// once, before the request's length says which runs exist (their places are inside the buffers either way,
// and what a run that does not exist left there is dropped by a select, never multiplied): one trip to
// memory instead of three.
constexpr int RD_WAVES = 4;
constexpr int RD_THREADS = RD_WAVES * DISTIE_WAVE;
constexpr int RD_MAX_RUNS = 1024;
constexpr int RD_FAST_PER_WAVE = 16;
constexpr int RD_FAST_RUNS = RD_FAST_PER_WAVE * RD_WAVES;

template <bool FAST>
__global__ __launch_bounds__(RD_THREADS) void attn_reduce_kernel(
    const float* __restrict__ part_o, const float* __restrict__ part_ml, const int32_t* __restrict__ kv_len,
    const int32_t* __restrict__ cu_q, bf16_t* __restrict__ out, int heads, int window, int max_splits,
    int dense_rows, const int32_t* __restrict__ shared_run_len) {
  __shared__ float weight_s[FAST ? RD_FAST_RUNS : RD_MAX_RUNS];
  __shared__ float sum_s[RD_WAVES][D];
  __shared__ float scratch[32];
  const int tid = threadIdx.x;
  const int wave = tid / DISTIE_WAVE;
  const int lane = tid % DISTIE_WAVE;
  const int request = blockIdx.y;
  const int head = blockIdx.x;
  const int64_t base0 = (static_cast<int64_t>(request) * heads + head) * max_splits;

  float early[FAST ? RD_FAST_PER_WAVE : 1][DIMS_PER_LANE];
  float2 early_ml = {0.f, 0.f};
  if constexpr (FAST) {
#pragma unroll
    for (int u = 0; u < RD_FAST_PER_WAVE; ++u) {
      const int j = min(wave + RD_WAVES * u, max_splits - 1);
#pragma unroll
      for (int i = 0; i < DIMS_PER_LANE; ++i) {
        const int d = lane + i * DISTIE_WAVE;
        early[u][i] = d < D ? part_o[(base0 + j) * D + d] : 0.f;
      }
    }
    early_ml = *reinterpret_cast<const float2*>(part_ml + 2 * (base0 + min(tid, max_splits - 1)));
  }

  const int token = dense_rows ? request : cu_q[request];
  if (!dense_rows && cu_q[request + 1] - token != 1) return;
  const int q_pos = kv_len[request] - 1;
  const int runs = key_runs(q_pos, window, max_splits, shared_run_len != nullptr ? *shared_run_len : 0).count;     // the first `runs` places hold results
  const int64_t base = base0;
  bf16_t* o = out + (static_cast<int64_t>(token) * heads + head) * D;

  if constexpr (FAST) {
    const bool mine = tid < runs;
    float m = mine ? early_ml.x : -INFINITY;
    m = wave_max(m);
    if (lane == 0) scratch[wave] = m;
    __syncthreads();
    m = fmaxf(fmaxf(scratch[0], scratch[1]), fmaxf(scratch[2], scratch[3]));
    const float w = mine ? fast_exp2(early_ml.x - m) : 0.f;
    if (tid < RD_FAST_RUNS) weight_s[tid] = w;
    const float l = block_sum(mine ? w * early_ml.y : 0.f, scratch + 16);     // has the barrier that publishes the weights
#pragma unroll
    for (int i = 0; i < DIMS_PER_LANE; ++i) {
      const int d = lane + i * DISTIE_WAVE;
      if (d >= D) continue;
      float a = 0.f;
#pragma unroll
      for (int u = 0; u < RD_FAST_PER_WAVE; ++u) {
        const int j = wave + RD_WAVES * u;
        const bool exists = j < runs;
        a = exists ? fmaf(weight_s[j], early[u][i], a) : a;
      }
      sum_s[wave][d] = a;
    }
    __syncthreads();
    if (wave != 0) return;
    const float inv = 1.f / l;
#pragma unroll
    for (int i = 0; i < DIMS_PER_LANE; ++i) {
      const int d = lane + i * DISTIE_WAVE;
      if (d < D) o[d] = static_cast<bf16_t>((((sum_s[0][d] + sum_s[1][d]) + sum_s[2][d]) + sum_s[3][d]) * inv);
    }
    return;
  }

  // the maximum over all runs (in units of log 2), then every run's weight
  float m = -INFINITY;
  for (int j = tid; j < runs; j += RD_THREADS) m = fmaxf(m, part_ml[2 * (base + j)]);
  m = wave_max(m);
  if (lane == 0) scratch[wave] = m;
  __syncthreads();
  m = fmaxf(fmaxf(scratch[0], scratch[1]), fmaxf(scratch[2], scratch[3]));
  float l = 0.f;
  for (int j = tid; j < runs; j += RD_THREADS) {
    const float w = fast_exp2(part_ml[2 * (base + j)] - m);
    weight_s[j] = w;
    l += w * part_ml[2 * (base + j) + 1];
  }
  l = block_sum(l, scratch + 16);           // has the barrier that publishes the weights
  const float* po = part_o + base * D;
#pragma unroll
  for (int i = 0; i < DIMS_PER_LANE; ++i) {
    const int d = lane + i * DISTIE_WAVE;
    if (d >= D) continue;
    float a = 0.f;
    int j = wave;
    for (; j + 3 * RD_WAVES < runs; j += 4 * RD_WAVES) {
      const float v0 = po[static_cast<int64_t>(j) * D + d], v1 = po[static_cast<int64_t>(j + RD_WAVES) * D + d];
      const float v2 = po[static_cast<int64_t>(j + 2 * RD_WAVES) * D + d], v3 = po[static_cast<int64_t>(j + 3 * RD_WAVES) * D + d];
      a = fmaf(weight_s[j], v0, a);
      a = fmaf(weight_s[j + RD_WAVES], v1, a);
      a = fmaf(weight_s[j + 2 * RD_WAVES], v2, a);
      a = fmaf(weight_s[j + 3 * RD_WAVES], v3, a);
    }
    for (; j < runs; j += RD_WAVES) a = fmaf(weight_s[j], po[static_cast<int64_t>(j) * D + d], a);
    sum_s[wave][d] = a;
  }
  __syncthreads();
  if (wave != 0) return;
  const float inv = 1.f / l;
#pragma unroll
  for (int i = 0; i < DIMS_PER_LANE; ++i) {
    const int d = lane + i * DISTIE_WAVE;
    if (d < D) o[d] = static_cast<bf16_t>((((sum_s[0][d] + sum_s[1][d]) + sum_s[2][d]) + sum_s[3][d]) * inv);
  }
}

constexpr int DECODE_MAX_MB = (D <= 128) ? 4 : 2;   // registers: the output tile is 16 * MB x D floats a wave

// most query heads per kv head the decode kernel takes
extern "C" int distie_attention_decode_columns() { return 16 * DECODE_MAX_MB; }

// The requests of a step that bring one token (others are skipped). kv_len: tokens cached after the step, per
// request. part_o: float32 [requests, heads, max_splits, D], part_ml: float32 [requests, heads, max_splits, 2]:
// every request's keys are cut into at most max_splits runs by its own length. split_hint, a multiple of 64, is
// the run length the caller expects of the longest request; it only saves time where it is right.
// shared_run_len (no window, every request of the step brings one token; else null): int32 [1], one run length for
// all requests, with which no request has more than max_splits runs (distie_attention_decode_run_len).
extern "C" int distie_attention_decode_bf16(const void* qkv, int64_t q_stride, const void* k_cache, const void* v_cache,
                                            const int32_t* kv_len, const int32_t* cu_q, const int32_t* block_table,
                                            int table_width, const int32_t* table_rows, void* out, float* part_o, float* part_ml,
                                            int num_requests, int heads, int kv_heads, int block_size, float scale,
                                            int window, int split_hint, int max_splits, int dense_rows,
                                            const int32_t* shared_run_len, hipStream_t stream) {
  if (num_requests <= 0) return 0;
  const int group = kv_heads > 0 ? heads / kv_heads : 0;
  if (heads < 1 || kv_heads < 1 || heads % kv_heads != 0 || block_size % 16 != 0 || table_width < 1 || window < 0 ||
      split_hint < RUN_STEP || split_hint % RUN_STEP != 0 || max_splits < 1 || max_splits > RD_MAX_RUNS ||
      group > 16 * DECODE_MAX_MB || kv_heads > 65535 || num_requests > 65535 || heads > 65535 ||
      (shared_run_len != nullptr && (window > 0 || !dense_rows)))
    return DISTIE_BAD_ARGUMENT;
  const dim3 grid = shared_run_len != nullptr ? dim3(kv_heads, num_requests, max_splits) : dim3(max_splits, kv_heads, num_requests);
  const bf16_t* q = static_cast<const bf16_t*>(qkv);
  const bf16_t* kc = static_cast<const bf16_t*>(k_cache);
  const bf16_t* vc = static_cast<const bf16_t*>(v_cache);
#define DECODE_LAUNCH(MB)                                                                                             \
  attn_decode_kernel<MB><<<grid, DISTIE_WAVE, 0, stream>>>(q, q_stride, kc, vc, kv_len, cu_q, block_table, table_width, table_rows, \
                                                           part_o, part_ml, heads, kv_heads, block_size, scale, window, \
                                                           split_hint, max_splits, dense_rows, shared_run_len)
  if (group <= 16) {
    DECODE_LAUNCH(1);
  } else if (group <= 32) {
    DECODE_LAUNCH(2);
  } else {
    DECODE_LAUNCH(DECODE_MAX_MB);
  }
#undef DECODE_LAUNCH
  int status = launch_status();
  if (status != 0) return status;
  if (max_splits <= RD_FAST_RUNS) {
    attn_reduce_kernel<true><<<dim3(heads, num_requests), RD_THREADS, 0, stream>>>(
        part_o, part_ml, kv_len, cu_q, static_cast<bf16_t*>(out), heads, window, max_splits, dense_rows, shared_run_len);
  } else {
    attn_reduce_kernel<false><<<dim3(heads, num_requests), RD_THREADS, 0, stream>>>(
        part_o, part_ml, kv_len, cu_q, static_cast<bf16_t*>(out), heads, window, max_splits, dense_rows, shared_run_len);
  }
  return launch_status();
}

// ===================================================================================================
//  * attn_prefill: the tiled kernel for portions of prompts. A workgroup of four waves owns PF_BM
//    consecutive new tokens of one request and one head; it walks over the keys 64 at a time. The K tile
//    [64, D] and the V^T tile [D, 64] are put into LDS once per workgroup (global loads of the next tile
//    are in flight while the current one is used) and every wave multiplies its own 32 query columns
//    against them with the 32 x 32 x 16 products (per flop they read half the operands of the 16-wide ones,
//    which is what bounds those here):
//        S^T[key, col] = K[key, :] . q[col, :]     K rows from LDS as the A operand, q in registers
//        O^T[d, col]  += V^T[d, key] . P^T[key, col]
//    A lane holds, of a 32 x 32 score tile, keys 8i + 4h + j (i, j < 4) of column c (c = lane % 32,
//    h = lane / 32): so a lane's 32 scores of a key tile, its running maximum and sum and its 32 D / 64
//    output sums all belong to one query token, and nothing but the column's maximum moves between lanes.
//    The B operand of the second product wants 8 of 16 summed keys per lane: those are the lane's own
//    scores if the 16 keys of a step are taken in the order (4h..4h+3, 8+4h..8+4h+3), and V^T is read
//    from LDS in the same order.
//    Head sizes that are no multiple of 32 compute a last block of 32 output rows of which 16 are zeros.
//    Requests that bring fewer than `min_q_len` tokens are left to the decode kernel.
// ===================================================================================================
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float floatx16;
constexpr int PF_BN = 64;                               // keys per tile
constexpr int PF_WAVES = 4;
constexpr int PF_THREADS = PF_WAVES * DISTIE_WAVE;
constexpr int PF_WAVE_COLS = 32;
constexpr int PF_BM = PF_WAVES * PF_WAVE_COLS;          // query tokens per workgroup
constexpr float PF_GROW = 8.f;                          // in units of log 2: how far a score may pass a column's reference
constexpr int PF_DK = D / 16;                           // steps of the q.k product
constexpr int PF_DB = (D + 31) / 32;                    // blocks of 32 output rows
#ifndef DISTIE_PF_AHEAD
#define DISTIE_PF_AHEAD 6
#endif
constexpr int PF_AHEAD = DISTIE_PF_AHEAD;               // reads from LDS in flight ahead of the products
// Rows in LDS, in elements. A lane reads 16 bytes of row (lane % 32) of K, and two times 8 bytes of row
// (lane % 32) of V^T: free of bank conflicts when a row is an odd number of such pieces long (measured: K rows
// of 272 and 304 bytes read at 198 B/clk a compute unit, of 288 at 112; V^T rows of 136 bytes 207, of 144 116).
constexpr int PF_K_STRIDE = D + 8;
constexpr int PF_V_STRIDE = PF_BN + 4;
constexpr int PF_BLOCK_CHUNKS = 2 * D;                  // 16-byte pieces of 16 keys of K, and of V^T: [16, D] or [D, 16]
constexpr int PF_PASSES = (PF_BLOCK_CHUNKS + DISTIE_WAVE - 1) / DISTIE_WAVE;   // pieces a lane carries per block
static_assert(PF_WAVES * 16 == PF_BN, "each wave brings one block of 16 keys of a tile");

__global__ __launch_bounds__(PF_THREADS, (D <= 128) ? 2 : 1) void attn_prefill_kernel(
    const bf16_t* __restrict__ qkv, int64_t q_stride, const bf16_t* __restrict__ k_cache,
    const bf16_t* __restrict__ v_cache, const int32_t* __restrict__ positions, const int32_t* __restrict__ cu_q,
    const int32_t* __restrict__ block_table, int table_width, const int32_t* __restrict__ table_rows, bf16_t* __restrict__ out, float* __restrict__ part_o,
    float* __restrict__ part_ml, int tokens, int num_requests, int heads, int kv_heads, int block_size, float scale,
    int window, int min_q_len) {
  __shared__ __attribute__((aligned(16))) bf16_t k_lds[PF_BN * PF_K_STRIDE];
  __shared__ __attribute__((aligned(16))) bf16_t v_lds[32 * PF_DB * PF_V_STRIDE];
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid / DISTIE_WAVE);   // uniform: what depends on it alone stays scalar
  const int lane = tid % DISTIE_WAVE;
  const int c = lane % 32;
  const int h = lane / 32;
  const int group = heads / kv_heads;
  const float scale_log2 = scale * 1.4426950408889634f;      // scores in units of log 2: weights are exp2

  // ---- which tokens: tiles of PF_BM tokens over the requests that are served here, the last first: the late
  // tokens of a portion see the most keys, and the longest work should start first
  int tile = gridDim.y - 1 - blockIdx.y;
  int request = 0, begin = 0, end = 0;
  for (; request < num_requests; ++request) {
    begin = cu_q[request];
    end = cu_q[request + 1];
    if (end - begin < min_q_len) continue;
    const int tiles = (end - begin + PF_BM - 1) / PF_BM;
    if (tile < tiles) break;
    tile -= tiles;
  }
  if (request >= num_requests) return;
  const int head = blockIdx.x;                            // heads vary fastest: the heavy tiles of all heads start first
  const int kh = head / group;
  const int token0 = begin + tile * PF_BM;
  const int columns = min(PF_BM, end - token0);           // of the workgroup
  const int pos0 = positions[token0];                     // the tokens of a portion have consecutive positions
  const int key_begin = window > 0 ? max(0, pos0 - window + 1) : 0;
  const int key_end = pos0 + columns - 1;
  const int32_t* table = block_table + static_cast<int64_t>(table_rows != nullptr ? table_rows[request] : request) * table_width;

  // the rows of V^T past the head size, read by the last block of output rows, stay zero
  if (D % 32 != 0)
    for (int i = tid; i < (32 * PF_DB - D) * PF_V_STRIDE; i += PF_THREADS) v_lds[D * PF_V_STRIDE + i] = static_cast<bf16_t>(0.f);

  // ---- this wave's columns; the lane's column
  const int wave_col0 = wave * PF_WAVE_COLS;
  const int wave_cols = max(0, min(PF_WAVE_COLS, columns - wave_col0));
  const int wave_last = pos0 + wave_col0 + wave_cols - 1;
  const int wave_first = window > 0 ? max(0, pos0 + wave_col0 - window + 1) : 0;
  const int col = min(wave_col0 + c, columns - 1);        // columns past the end repeat the last; dropped later
  const int col_last = pos0 + col;                        // the last key the column sees, and the first
  const int col_first = window > 0 ? max(0, col_last - window + 1) : 0;
  bf16x8 q_reg[PF_DK];
  {
    const bf16_t* q = qkv + (token0 + col) * q_stride + static_cast<int64_t>(head) * D;
#pragma unroll
    for (int dk = 0; dk < PF_DK; ++dk) q_reg[dk] = *reinterpret_cast<const bf16x8*>(q + 16 * dk + 8 * h);
  }
  floatx16 o_acc[PF_DB];
#pragma unroll
  for (int db = 0; db < PF_DB; ++db)
#pragma unroll
    for (int e = 0; e < 16; ++e) o_acc[db][e] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;

  // ---- staging of one tile in registers. Wave w brings block w of the tile (keys k0 + 16 w .. + 15): one page
  // lookup a wave, the 16 rows of K are one run of 16 D elements in their page, V^T is D runs of 16.
  uint4 k_stage[PF_PASSES], v_stage[PF_PASSES];
  const int block_shift = (block_size & (block_size - 1)) == 0 ? __builtin_ctz(block_size) : -1;
  // Every lane issues the same loads for every tile, with no branch around them: a block that belongs to no
  // page reads the start of the cache instead and is cleared when it is stored.
  auto block_live = [&](int key) { return key <= key_end && key + 15 >= key_begin; };
  // The page of a block is looked up two tiles before its keys are asked for (a scalar load, the block being
  // the same for the whole wave): asked for together, every tile would cost the wave two trips to memory
  // one after the other.
  auto lookup = [&](int k0) {
    const int key = k0 + 16 * wave;
    const int slot = block_shift >= 0 ? key >> block_shift : key / block_size;
    return table[min(slot, table_width - 1)];
  };
  auto fetch = [&](int k0, int page_of_block) {
    const int key = k0 + 16 * wave;
    const bool live = block_live(key);
    const int offset = live ? (block_shift >= 0 ? key & (block_size - 1) : key % block_size) : 0;
    const int page = live ? page_of_block : 0;
    const int64_t base = live ? (static_cast<int64_t>(page) * kv_heads + kh) * block_size * D : 0;
    const bf16_t* k_block = k_cache + base + static_cast<int64_t>(offset) * D;
    const bf16_t* v_block = v_cache + base + offset;
#pragma unroll
    for (int p = 0; p < PF_PASSES; ++p) {
      const int j = min(lane + p * DISTIE_WAVE, PF_BLOCK_CHUNKS - 1);
      k_stage[p] = *reinterpret_cast<const uint4*>(k_block + 8 * j);
      v_stage[p] = *reinterpret_cast<const uint4*>(v_block + static_cast<int64_t>(j / 2) * block_size + 8 * (j % 2));
    }
  };
  // where a lane's pieces go in LDS: the same for every tile (a row of V^T is a multiple of 8 bytes long,
  // not of 16: its pieces are stored as two halves)
  int k_slot[PF_PASSES], v_slot[PF_PASSES];
#pragma unroll
  for (int p = 0; p < PF_PASSES; ++p) {
    const int j = min(lane + p * DISTIE_WAVE, PF_BLOCK_CHUNKS - 1);
    k_slot[p] = (16 * wave + j / (D / 8)) * PF_K_STRIDE + 8 * (j % (D / 8));
    v_slot[p] = (j / 2) * PF_V_STRIDE + 16 * wave + 8 * (j % 2);
  }
  auto stash = [&](int k0) {
    const int key = k0 + 16 * wave;                       // the same for the whole wave: the branches are uniform
    const bool live = block_live(key);
    // Slots after the last key of this workgroup were not written by this request, and blocks outside the keys
    // of this workgroup were not read: cleared (a weight of zero times NaN would still be NaN).
    const bool whole = live && key + 15 <= key_end;
    if (whole) {
#pragma unroll
      for (int p = 0; p < PF_PASSES; ++p) {
        if (lane + p * DISTIE_WAVE >= PF_BLOCK_CHUNKS) continue;
        *reinterpret_cast<uint4*>(k_lds + k_slot[p]) = k_stage[p];
        *reinterpret_cast<uint2*>(v_lds + v_slot[p]) = uint2{v_stage[p].x, v_stage[p].y};
        *reinterpret_cast<uint2*>(v_lds + v_slot[p] + 4) = uint2{v_stage[p].z, v_stage[p].w};
      }
      return;
    }
#pragma unroll
    for (int p = 0; p < PF_PASSES; ++p) {
      const int j = lane + p * DISTIE_WAVE;
      if (j >= PF_BLOCK_CHUNKS) continue;
      *reinterpret_cast<uint4*>(k_lds + k_slot[p]) = live ? k_stage[p] : uint4{0u, 0u, 0u, 0u};
      const int written = live ? key_end - (key + 8 * (j % 2)) + 1 : 0;        // of this piece's eight keys
      const uint32_t w[4] = {v_stage[p].x, v_stage[p].y, v_stage[p].z, v_stage[p].w};
      uint32_t m[4];
#pragma unroll
      for (int e = 0; e < 4; ++e)
        m[e] = written >= 2 * e + 2 ? w[e] : (written == 2 * e + 1 ? (w[e] & 0x0000ffffu) : 0u);
      *reinterpret_cast<uint2*>(v_lds + v_slot[p]) = uint2{m[0], m[1]};
      *reinterpret_cast<uint2*>(v_lds + v_slot[p] + 4) = uint2{m[2], m[3]};
    }
  };

  auto compute = [&](int k0) {
    if (wave_cols <= 0 || k0 > wave_last || k0 + PF_BN - 1 < wave_first) return;

    // ---- scores: 64 keys x the wave's 32 columns, as two blocks of 32 keys
    floatx16 s[2];
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int e = 0; e < 16; ++e) s[kb][e] = 0.f;
    // PF_AHEAD reads from LDS are under way when the first product is issued, and every product is followed
    // by one more read: left to itself the compiler keeps two reads in flight, which is less than the trip takes
    {
      bf16x8 a[2 * PF_DK];
#pragma unroll
      for (int i = 0; i < 2 * PF_DK; ++i)
        a[i] = *reinterpret_cast<const bf16x8*>(k_lds + (32 * (i % 2) + c) * PF_K_STRIDE + 16 * (i / 2) + 8 * h);
#pragma unroll
      for (int i = 0; i < 2 * PF_DK; ++i)
        s[i % 2] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], q_reg[i / 2], s[i % 2], 0, 0, 0);
      constexpr int ahead = 2 * PF_DK < PF_AHEAD ? 2 * PF_DK : PF_AHEAD;
      __builtin_amdgcn_sched_group_barrier(0x100, ahead, 0);
#pragma unroll
      for (int i = 0; i < 2 * PF_DK - ahead; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
      __builtin_amdgcn_sched_group_barrier(0x008, ahead, 0);
    }
    // ---- softmax step of the lane's column. A tile whose keys every column of the wave sees needs no mask:
    // that is every tile but those on the diagonal and at a window's edge.
    const bool tile_open = k0 + PF_BN - 1 <= pos0 + wave_col0 &&
                           (window <= 0 || k0 >= pos0 + wave_col0 + wave_cols - window);
    if (!tile_open) {
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int key = k0 + 32 * kb + 8 * (e / 4) + 4 * h + e % 4;
          if (key < col_first || key > col_last) s[kb][e] = -INFINITY;
        }
    }
    // The running reference m of a column (scores count from it: weights are 2^(score - m)) follows the
    // largest score only when that has grown by more than PF_GROW since m was set: then the sums so far are
    // scaled down, for all columns of the wave at once. In between a weight may reach 2^PF_GROW, which
    // float32 sums and bfloat16 weights hold as well as they hold 1, and the scaling of the sums becomes rare.
    float top = -INFINITY;
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int e = 0; e < 16; ++e) top = fmaxf(top, s[kb][e]);
    top = fmaxf(top, __shfl_xor(top, 32, DISTIE_WAVE));
    const float best = top * scale_log2;                  // the scale is positive: the largest stays the largest
    if (__any(best > m_run + PF_GROW)) {                  // also the first score of a column (m = -inf)
      const float m_new = fmaxf(m_run, best);
      const float alpha = m_new == -INFINITY ? 1.f : fast_exp2(m_run - m_new);   // 0 while m was -inf
      l_run *= alpha;
      m_run = m_new;
#pragma unroll
      for (int db = 0; db < PF_DB; ++db)
#pragma unroll
        for (int e = 0; e < 16; ++e) o_acc[db][e] *= alpha;
    }
    const float from = m_run == -INFINITY ? 0.f : -m_run;
    bf16x8 p_reg[4];                                      // step t: keys 16 t + (4h..4h+3, 8+4h..8+4h+3) of the tile
    float sum = 0.f;
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const float p = fast_exp2(fmaf(s[kb][e], scale_log2, from));
        sum += p;
        p_reg[2 * kb + e / 8][e % 8] = static_cast<bf16_t>(p);
      }
    l_run += sum;
    // ---- O^T += V^T . P^T: four steps of 16 keys
    {
      bf16x8 vt[4 * PF_DB];
#pragma unroll
      for (int i = 0; i < 4 * PF_DB; ++i) {
        const bf16_t* v_row = v_lds + (32 * (i % PF_DB) + c) * PF_V_STRIDE + 16 * (i / PF_DB) + 4 * h;
        const uint2 lo = *reinterpret_cast<const uint2*>(v_row);
        const uint2 hi = *reinterpret_cast<const uint2*>(v_row + 8);
        const uintx4 words = {lo.x, lo.y, hi.x, hi.y};
        vt[i] = __builtin_bit_cast(bf16x8, words);
      }
#pragma unroll
      for (int i = 0; i < 4 * PF_DB; ++i)
        o_acc[i % PF_DB] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vt[i], p_reg[i / PF_DB], o_acc[i % PF_DB], 0, 0, 0);
      constexpr int ahead = 4 * PF_DB < PF_AHEAD ? 4 * PF_DB : PF_AHEAD;
      __builtin_amdgcn_sched_group_barrier(0x100, ahead, 1);
#pragma unroll
      for (int i = 0; i < 4 * PF_DB - ahead; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 1);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 1);
      }
      __builtin_amdgcn_sched_group_barrier(0x008, ahead, 1);
    }
  };

  // With gridDim.z > 1 the key tiles of these tokens are cut in that many parts, one workgroup each, which write
  // unnormalised partial results that attn_prefill_merge_kernel combines: the last tokens of a long
  // portion walk over many key tiles one after the other, and this shortens the longest walk.
  // One tile of loads is in flight (tiles past the last key load the start of the cache and are not used).
  const int all_tile0 = key_begin / PF_BN * PF_BN;
  const int all_tiles = (key_end - all_tile0) / PF_BN + 1;
  const int per_split = (all_tiles + gridDim.z - 1) / gridDim.z;
  const int tile0 = all_tile0 + static_cast<int>(blockIdx.z) * per_split * PF_BN;
  const int loop_end = min(key_end, tile0 + per_split * PF_BN - 1);            // last key of this workgroup's walk
  fetch(tile0, lookup(tile0));
  int page_ahead = lookup(tile0 + PF_BN);
  for (int k0 = tile0; k0 <= loop_end; k0 += PF_BN) {
    __syncthreads();                       // every wave is done with the tile in LDS
    stash(k0);
    __syncthreads();
    fetch(k0 + PF_BN, page_ahead);
    page_ahead = lookup(k0 + 2 * PF_BN);
    compute(k0);
  }
  // ---- write: the lane holds, of its column, output rows 32 db + 8 i + 4 h + (0..3)
  l_run += __shfl_xor(l_run, 32, DISTIE_WAVE);
  if (wave_col0 + c >= columns) return;
  const int64_t row = static_cast<int64_t>(token0 + wave_col0 + c) * heads + head;
  if (gridDim.z == 1) {
    bf16_t* o = out + row * D;
    const float inv = 1.f / l_run;
#pragma unroll
    for (int db = 0; db < PF_DB; ++db)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int d = 32 * db + 8 * i + 4 * h;
        if (d >= D) continue;
        uint32_t half[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) half[j] = __builtin_bit_cast(uint16_t, static_cast<bf16_t>(o_acc[db][4 * i + j] * inv));
        *reinterpret_cast<uint2*>(o + d) = uint2{half[0] | (half[1] << 16), half[2] | (half[3] << 16)};
      }
  } else {
    // a part without a key for this column leaves l = 0, and the merge does not read its sums
    const int64_t at = static_cast<int64_t>(blockIdx.z) * tokens * heads + row;
    float* po = part_o + at * D;
#pragma unroll
    for (int db = 0; db < PF_DB; ++db)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int d = 32 * db + 8 * i + 4 * h;
        if (d >= D) continue;
        *reinterpret_cast<float4*>(po + d) = float4{o_acc[db][4 * i], o_acc[db][4 * i + 1], o_acc[db][4 * i + 2], o_acc[db][4 * i + 3]};
      }
    if (h == 0) {
      part_ml[2 * at] = m_run;
      part_ml[2 * at + 1] = l_run;
    }
  }
}

// Combines the `splits` parts of attn_prefill_kernel with gridDim.z > 1, in order: one block per token; tokens
// of requests that the kernel skipped (fewer than min_q_len tokens) are skipped here as well.
constexpr int PF_MAX_SPLITS = 16;

template <typename OUT, int MOST>
__global__ void attn_prefill_merge_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                                          const int32_t* __restrict__ token_request, const int32_t* __restrict__ cu_q,
                                          OUT* __restrict__ out, int tokens, int heads, int min_q_len, int splits) {
  const int64_t token = blockIdx.x;
  const int request = token_request[token];
  if (cu_q[request + 1] - cu_q[request] < min_q_len) return;
  const int64_t part = static_cast<int64_t>(tokens) * heads;
  for (int i = threadIdx.x; i < heads * (D / 4); i += blockDim.x) {
    const int head = i / (D / 4);
    const int d = 4 * (i % (D / 4));
    const int64_t row = token * heads + head;
    float2 ml[MOST];
    float4 o[MOST];
    float m = -INFINITY;
#pragma unroll
    for (int s = 0; s < MOST; ++s) {
      ml[s] = float2{-INFINITY, 0.f};
      o[s] = float4{0.f, 0.f, 0.f, 0.f};
      if (s < splits) ml[s] = *reinterpret_cast<const float2*>(part_ml + 2 * (s * part + row));
      // a part without a key for this token has l = 0; what it left in part_o is not read (for a prompt
      // without a past that is a third of all reads: asking for them anyway, to save the second trip to
      // memory, made this kernel slower where it runs, 12.2 -> 14.7 us, and 10.0 -> 10.5 once the registers of
      // the parts that are not there no longer held waves back)
      if (s < splits && ml[s].y > 0.f) {
        o[s] = *reinterpret_cast<const float4*>(part_o + (s * part + row) * D + d);
        m = fmaxf(m, ml[s].x);
      }
    }
    float l = 0.f;
    float4 sum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < MOST; ++s) {
      const float w = ml[s].y > 0.f ? fast_exp2(ml[s].x - m) : 0.f;
      l += w * ml[s].y;
      sum.x += w * o[s].x;
      sum.y += w * o[s].y;
      sum.z += w * o[s].z;
      sum.w += w * o[s].w;
    }
    const float inv = 1.f / l;
    const float v[4] = {sum.x * inv, sum.y * inv, sum.z * inv, sum.w * inv};
    if constexpr (sizeof(OUT) == 4) {
      *reinterpret_cast<float4*>(out + row * D + d) = float4{v[0], v[1], v[2], v[3]};
    } else {
      uint32_t h[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) h[e] = __builtin_bit_cast(uint16_t, static_cast<bf16_t>(v[e]));
      *reinterpret_cast<uint2*>(out + row * D + d) = uint2{h[0] | (h[1] << 16), h[2] | (h[3] << 16)};
    }
  }
}

// The merge holds every part's maximum, sum and four outputs in registers: compiled for at most 4, 8 and 16 parts,
// so that few parts leave room for more waves on a compute unit.
template <typename OUT>
static void launch_merge(const float* part_o, const float* part_ml, const int32_t* token_request, const int32_t* cu_q,
                         OUT* out, int tokens, int heads, int min_q_len, int splits, hipStream_t stream) {
  const int work = heads * (D / 4);
  const int threads = work >= 512 ? 512 : (work >= 256 ? 256 : 64);
  if (splits <= 4)
    attn_prefill_merge_kernel<OUT, 4><<<tokens, threads, 0, stream>>>(part_o, part_ml, token_request, cu_q, out, tokens,
                                                                       heads, min_q_len, splits);
  else if (splits <= 8)
    attn_prefill_merge_kernel<OUT, 8><<<tokens, threads, 0, stream>>>(part_o, part_ml, token_request, cu_q, out, tokens,
                                                                       heads, min_q_len, splits);
  else
    attn_prefill_merge_kernel<OUT, PF_MAX_SPLITS><<<tokens, threads, 0, stream>>>(part_o, part_ml, token_request, cu_q, out,
                                                                                   tokens, heads, min_q_len, splits);
}

// Portions of prompts (and whole mixed steps). bfloat16 only; block_size must be a multiple of 16. Requests that
// bring fewer than min_q_len tokens are skipped (the decode kernel serves them).
extern "C" int distie_attention_prefill_bf16(const void* qkv, int64_t q_stride, const void* k_cache, const void* v_cache,
                                             const int32_t* positions, const int32_t* cu_q, const int32_t* block_table,
                                             int table_width, const int32_t* table_rows, void* out, int tokens, int num_requests, int heads,
                                             int kv_heads, int block_size, float scale, int window, int min_q_len,
                                             const int32_t* token_request, float* part_o, float* part_ml,
                                             int splits, hipStream_t stream) {
  // splits > 1: the keys are walked in that many parts side by side (worth it for long portions), with
  // part_o (float32 [splits, tokens, heads, D]) and part_ml (float32 [splits, tokens, heads, 2]) in between.
  if (tokens <= 0) return 0;
  if (heads < 1 || kv_heads < 1 || heads % kv_heads != 0 || block_size % 16 != 0 || table_width < 1 || window < 0 ||
      num_requests < 1 || heads > 65535 || min_q_len < 1 || splits < 1 || splits > PF_MAX_SPLITS || !(scale > 0.f) ||
      (splits > 1 && (part_o == nullptr || part_ml == nullptr || token_request == nullptr)))
    return DISTIE_BAD_ARGUMENT;
  const int tiles = (tokens + PF_BM - 1) / PF_BM + num_requests;     // an upper bound; spare blocks leave at once
  if (tiles > 65535) return DISTIE_BAD_ARGUMENT;
  attn_prefill_kernel<<<dim3(heads, tiles, splits), PF_THREADS, 0, stream>>>(
      static_cast<const bf16_t*>(qkv), q_stride, static_cast<const bf16_t*>(k_cache), static_cast<const bf16_t*>(v_cache),
      positions, cu_q, block_table, table_width, table_rows, static_cast<bf16_t*>(out), part_o, part_ml, tokens, num_requests, heads,
      kv_heads, block_size, scale, window, min_q_len);
  int status = launch_status();
  if (status != 0 || splits == 1) return status;
  launch_merge(part_o, part_ml, token_request, cu_q, static_cast<bf16_t*>(out), tokens, heads, min_q_len, splits, stream);
  return launch_status();
}

// ===================================================================================================
//  * attn_prefill_f32: the tiled kernel in float32, for head sizes that are multiples of 32 up to 128. The same
//    walk as attn_prefill (a workgroup of four waves owns 128 new tokens of one head, 32 query columns a wave,
//    K and V^T tiles of 64 keys through LDS, the keys cut into parts that are merged) on the float32 products
//    v_mfma_f32_32x32x2_f32: float32 operands, products and sums, no reduced precision anywhere. Such a product
//    sums over two values, one from each half of the wave; four of them in a row take a lane's 16 bytes of a K or
//    V^T row, so the head dimension (first product) and the keys (second product) are summed in the order in
//    which the lanes hold them: d = 8 g + 4 h + e and key = 8 i + 4 h + j for step e or j of group g or i.
//    The weights stay where the scores were (the accumulators' layout is the B operand's), in float32.
// ===================================================================================================
#if (DISTIE_HEAD_DIM % 32 == 0) && (DISTIE_HEAD_DIM <= 128)
constexpr int PF32_K_STRIDE = D + 4;                    // floats: rows of an odd number of 16-byte pieces
constexpr int PF32_V_STRIDE = PF_BN + 4;
constexpr int PF32_CHUNKS = 4 * D;                      // 16-byte pieces of 16 keys of K ([16, D]), and of V^T ([D, 16])
constexpr int PF32_PASSES = PF32_CHUNKS / DISTIE_WAVE;  // pieces a lane carries per block
constexpr int PF32_AHEAD = 2;                           // reads from LDS ahead of the products (four products a read)

__global__ __launch_bounds__(PF_THREADS, 1) void attn_prefill_f32_kernel(
    const float* __restrict__ qkv, int64_t q_stride, const float* __restrict__ k_cache,
    const float* __restrict__ v_cache, const int32_t* __restrict__ positions, const int32_t* __restrict__ cu_q,
    const int32_t* __restrict__ block_table, int table_width, const int32_t* __restrict__ table_rows, float* __restrict__ out,
    float* __restrict__ part_o, float* __restrict__ part_ml, int tokens, int num_requests, int heads, int kv_heads,
    int block_size, float scale, int window, int min_q_len) {
  __shared__ __attribute__((aligned(16))) float k_lds[PF_BN * PF32_K_STRIDE];
  __shared__ __attribute__((aligned(16))) float v_lds[D * PF32_V_STRIDE];
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid / DISTIE_WAVE);
  const int lane = tid % DISTIE_WAVE;
  const int c = lane % 32;
  const int h = lane / 32;
  const int group = heads / kv_heads;
  const float scale_log2 = scale * 1.4426950408889634f;

  // ---- which tokens (as in attn_prefill)
  int tile = gridDim.y - 1 - blockIdx.y;
  int request = 0, begin = 0, end = 0;
  for (; request < num_requests; ++request) {
    begin = cu_q[request];
    end = cu_q[request + 1];
    if (end - begin < min_q_len) continue;
    const int tiles = (end - begin + PF_BM - 1) / PF_BM;
    if (tile < tiles) break;
    tile -= tiles;
  }
  if (request >= num_requests) return;
  const int head = blockIdx.x;
  const int kh = head / group;
  const int token0 = begin + tile * PF_BM;
  const int columns = min(PF_BM, end - token0);
  const int pos0 = positions[token0];
  const int key_begin = window > 0 ? max(0, pos0 - window + 1) : 0;
  const int key_end = pos0 + columns - 1;
  const int32_t* table = block_table + static_cast<int64_t>(table_rows != nullptr ? table_rows[request] : request) * table_width;

  const int wave_col0 = wave * PF_WAVE_COLS;
  const int wave_cols = max(0, min(PF_WAVE_COLS, columns - wave_col0));
  const int wave_last = pos0 + wave_col0 + wave_cols - 1;
  const int wave_first = window > 0 ? max(0, pos0 + wave_col0 - window + 1) : 0;
  const int col = min(wave_col0 + c, columns - 1);
  const int col_last = pos0 + col;
  const int col_first = window > 0 ? max(0, col_last - window + 1) : 0;
  float4 q_reg[D / 8];                                    // of the lane's column: d = 8 g + 4 h + (0..3)
  {
    const float* q = qkv + (token0 + col) * q_stride + static_cast<int64_t>(head) * D;
#pragma unroll
    for (int g = 0; g < D / 8; ++g) q_reg[g] = *reinterpret_cast<const float4*>(q + 8 * g + 4 * h);
  }
  floatx16 o_acc[D / 32];
#pragma unroll
  for (int db = 0; db < D / 32; ++db)
#pragma unroll
    for (int e = 0; e < 16; ++e) o_acc[db][e] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;

  // ---- staging: wave w brings block w of the tile (keys k0 + 16 w .. + 15)
  uint4 k_stage[PF32_PASSES], v_stage[PF32_PASSES];
  const int block_shift = (block_size & (block_size - 1)) == 0 ? __builtin_ctz(block_size) : -1;
  auto block_live = [&](int key) { return key <= key_end && key + 15 >= key_begin; };
  auto lookup = [&](int k0) {
    const int key = k0 + 16 * wave;
    const int slot = block_shift >= 0 ? key >> block_shift : key / block_size;
    return table[min(slot, table_width - 1)];
  };
  auto fetch = [&](int k0, int page_of_block) {
    const int key = k0 + 16 * wave;
    const bool live = block_live(key);
    const int offset = live ? (block_shift >= 0 ? key & (block_size - 1) : key % block_size) : 0;
    const int64_t base = live ? (static_cast<int64_t>(page_of_block) * kv_heads + kh) * block_size * D : 0;
    const float* k_block = k_cache + base + static_cast<int64_t>(offset) * D;
    const float* v_block = v_cache + base + offset;
#pragma unroll
    for (int p = 0; p < PF32_PASSES; ++p) {
      const int j = lane + p * DISTIE_WAVE;
      k_stage[p] = *reinterpret_cast<const uint4*>(k_block + 4 * j);
      v_stage[p] = *reinterpret_cast<const uint4*>(v_block + static_cast<int64_t>(j / 4) * block_size + 4 * (j % 4));
    }
  };
  int k_slot[PF32_PASSES], v_slot[PF32_PASSES];
#pragma unroll
  for (int p = 0; p < PF32_PASSES; ++p) {
    const int j = lane + p * DISTIE_WAVE;
    k_slot[p] = (16 * wave + j / (D / 4)) * PF32_K_STRIDE + 4 * (j % (D / 4));
    v_slot[p] = (j / 4) * PF32_V_STRIDE + 16 * wave + 4 * (j % 4);
  }
  // Slots after the last key of this workgroup were not written by this request, and blocks outside the keys
  // of this workgroup were not read: cleared (a weight of zero times NaN would still be NaN).
  auto stash = [&](int k0) {
    const int key = k0 + 16 * wave;
    const bool live = block_live(key);
    if (live && key + 15 <= key_end) {
#pragma unroll
      for (int p = 0; p < PF32_PASSES; ++p) {
        *reinterpret_cast<uint4*>(k_lds + k_slot[p]) = k_stage[p];
        *reinterpret_cast<uint4*>(v_lds + v_slot[p]) = v_stage[p];
      }
      return;
    }
#pragma unroll
    for (int p = 0; p < PF32_PASSES; ++p) {
      const int j = lane + p * DISTIE_WAVE;
      *reinterpret_cast<uint4*>(k_lds + k_slot[p]) = live ? k_stage[p] : uint4{0u, 0u, 0u, 0u};
      const int written = live ? key_end - (key + 4 * (j % 4)) + 1 : 0;        // of this piece's four keys
      *reinterpret_cast<uint4*>(v_lds + v_slot[p]) =
          uint4{written >= 1 ? v_stage[p].x : 0u, written >= 2 ? v_stage[p].y : 0u, written >= 3 ? v_stage[p].z : 0u,
                written >= 4 ? v_stage[p].w : 0u};
    }
  };

  auto compute = [&](int k0) {
    if (wave_cols <= 0 || k0 > wave_last || k0 + PF_BN - 1 < wave_first) return;
    // ---- scores: 64 keys x the wave's 32 columns, as two blocks of 32 keys
    floatx16 s[2];
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int e = 0; e < 16; ++e) s[kb][e] = 0.f;
    {
      float4 a[D / 4];
#pragma unroll
      for (int i = 0; i < D / 4; ++i)
        a[i] = *reinterpret_cast<const float4*>(k_lds + (32 * (i % 2) + c) * PF32_K_STRIDE + 8 * (i / 2) + 4 * h);
#pragma unroll
      for (int i = 0; i < D / 4; ++i) {
        s[i % 2] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i].x, q_reg[i / 2].x, s[i % 2], 0, 0, 0);
        s[i % 2] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i].y, q_reg[i / 2].y, s[i % 2], 0, 0, 0);
        s[i % 2] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i].z, q_reg[i / 2].z, s[i % 2], 0, 0, 0);
        s[i % 2] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i].w, q_reg[i / 2].w, s[i % 2], 0, 0, 0);
      }
      __builtin_amdgcn_sched_group_barrier(0x100, PF32_AHEAD, 0);
#pragma unroll
      for (int i = 0; i < D / 4 - PF32_AHEAD; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
      __builtin_amdgcn_sched_group_barrier(0x008, 4 * PF32_AHEAD, 0);
    }
    const bool tile_open = k0 + PF_BN - 1 <= pos0 + wave_col0 &&
                           (window <= 0 || k0 >= pos0 + wave_col0 + wave_cols - window);
    if (!tile_open) {
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int key = k0 + 32 * kb + 8 * (e / 4) + 4 * h + e % 4;
          if (key < col_first || key > col_last) s[kb][e] = -INFINITY;
        }
    }
    // the column's reference follows its largest score when that has outgrown it (see attn_prefill)
    float top = -INFINITY;
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int e = 0; e < 16; ++e) top = fmaxf(top, s[kb][e]);
    top = fmaxf(top, __shfl_xor(top, 32, DISTIE_WAVE));
    const float best = top * scale_log2;
    if (__any(best > m_run + PF_GROW)) {
      const float m_new = fmaxf(m_run, best);
      const float alpha = m_new == -INFINITY ? 1.f : fast_exp2(m_run - m_new);
      l_run *= alpha;
      m_run = m_new;
#pragma unroll
      for (int db = 0; db < D / 32; ++db)
#pragma unroll
        for (int e = 0; e < 16; ++e) o_acc[db][e] *= alpha;
    }
    const float from = m_run == -INFINITY ? 0.f : -m_run;
    float sum = 0.f;
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        s[kb][e] = fast_exp2(fmaf(s[kb][e], scale_log2, from));
        sum += s[kb][e];
      }
    l_run += sum;
    // ---- O^T += V^T . P^T: eight groups of four keys for each block of 32 output rows
    {
      constexpr int reads = 8 * (D / 32);
      float4 vt[reads];
#pragma unroll
      for (int i = 0; i < reads; ++i) {
        const int db = i % (D / 32), group_of_keys = i / (D / 32);        // group: kb = / 4, i = % 4
        vt[i] = *reinterpret_cast<const float4*>(v_lds + (32 * db + c) * PF32_V_STRIDE + 8 * group_of_keys + 4 * h);
      }
#pragma unroll
      for (int i = 0; i < reads; ++i) {
        const int db = i % (D / 32), kb = (i / (D / 32)) / 4, e = 4 * ((i / (D / 32)) % 4);
        o_acc[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(vt[i].x, s[kb][e], o_acc[db], 0, 0, 0);
        o_acc[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(vt[i].y, s[kb][e + 1], o_acc[db], 0, 0, 0);
        o_acc[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(vt[i].z, s[kb][e + 2], o_acc[db], 0, 0, 0);
        o_acc[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(vt[i].w, s[kb][e + 3], o_acc[db], 0, 0, 0);
      }
      __builtin_amdgcn_sched_group_barrier(0x100, PF32_AHEAD, 1);
#pragma unroll
      for (int i = 0; i < reads - PF32_AHEAD; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 4, 1);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 1);
      }
      __builtin_amdgcn_sched_group_barrier(0x008, 4 * PF32_AHEAD, 1);
    }
  };

  const int all_tile0 = key_begin / PF_BN * PF_BN;
  const int all_tiles = (key_end - all_tile0) / PF_BN + 1;
  const int per_split = (all_tiles + gridDim.z - 1) / gridDim.z;
  const int tile0 = all_tile0 + static_cast<int>(blockIdx.z) * per_split * PF_BN;
  const int loop_end = min(key_end, tile0 + per_split * PF_BN - 1);
  fetch(tile0, lookup(tile0));
  int page_ahead = lookup(tile0 + PF_BN);
  for (int k0 = tile0; k0 <= loop_end; k0 += PF_BN) {
    __syncthreads();                       // every wave is done with the tile in LDS
    stash(k0);
    __syncthreads();
    fetch(k0 + PF_BN, page_ahead);
    page_ahead = lookup(k0 + 2 * PF_BN);
    compute(k0);
  }
  // ---- write: the lane holds, of its column, output rows 32 db + 8 i + 4 h + (0..3)
  l_run += __shfl_xor(l_run, 32, DISTIE_WAVE);
  if (wave_col0 + c >= columns) return;
  const int64_t row = static_cast<int64_t>(token0 + wave_col0 + c) * heads + head;
  const bool whole = gridDim.z == 1;
  const int64_t at = whole ? row : static_cast<int64_t>(blockIdx.z) * tokens * heads + row;
  float* o = (whole ? out : part_o) + at * D;
  const float factor = whole ? 1.f / l_run : 1.f;         // a part without a key for this column leaves l = 0: not read
#pragma unroll
  for (int db = 0; db < D / 32; ++db)
#pragma unroll
    for (int i = 0; i < 4; ++i)
      *reinterpret_cast<float4*>(o + 32 * db + 8 * i + 4 * h) =
          float4{o_acc[db][4 * i] * factor, o_acc[db][4 * i + 1] * factor, o_acc[db][4 * i + 2] * factor, o_acc[db][4 * i + 3] * factor};
  if (!whole && h == 0) {
    part_ml[2 * at] = m_run;
    part_ml[2 * at + 1] = l_run;
  }
}
#endif

extern "C" int distie_attention_prefill_f32_fits() { return (D % 32 == 0 && D <= 128) ? 1 : 0; }

// As distie_attention_prefill_bf16, for float32 queries and a float32 cache; head sizes for which
// distie_attention_prefill_f32_fits() says 1.
extern "C" int distie_attention_prefill_f32(const void* qkv, int64_t q_stride, const void* k_cache, const void* v_cache,
                                            const int32_t* positions, const int32_t* cu_q, const int32_t* block_table,
                                            int table_width, const int32_t* table_rows, void* out, int tokens, int num_requests, int heads,
                                            int kv_heads, int block_size, float scale, int window, int min_q_len,
                                            const int32_t* token_request, float* part_o, float* part_ml,
                                            int splits, hipStream_t stream) {
#if (DISTIE_HEAD_DIM % 32 == 0) && (DISTIE_HEAD_DIM <= 128)
  if (tokens <= 0) return 0;
  if (heads < 1 || kv_heads < 1 || heads % kv_heads != 0 || block_size % 16 != 0 || table_width < 1 || window < 0 ||
      num_requests < 1 || heads > 65535 || min_q_len < 1 || splits < 1 || splits > PF_MAX_SPLITS || !(scale > 0.f) ||
      q_stride % 4 != 0 ||
      (splits > 1 && (part_o == nullptr || part_ml == nullptr || token_request == nullptr)))
    return DISTIE_BAD_ARGUMENT;
  const int tiles = (tokens + PF_BM - 1) / PF_BM + num_requests;
  if (tiles > 65535) return DISTIE_BAD_ARGUMENT;
  attn_prefill_f32_kernel<<<dim3(heads, tiles, splits), PF_THREADS, 0, stream>>>(
      static_cast<const float*>(qkv), q_stride, static_cast<const float*>(k_cache), static_cast<const float*>(v_cache),
      positions, cu_q, block_table, table_width, table_rows, static_cast<float*>(out), part_o, part_ml, tokens, num_requests,
      heads, kv_heads, block_size, scale, window, min_q_len);
  int status = launch_status();
  if (status != 0 || splits == 1) return status;
  launch_merge(part_o, part_ml, token_request, cu_q, static_cast<float*>(out), tokens, heads, min_q_len, splits, stream);
  return launch_status();
#else
  return DISTIE_BAD_ARGUMENT;
#endif
}

#else   // a head size that is no multiple of 16: the wave-per-token kernel is all there is

extern "C" int distie_attention_decode_columns() { return 0; }

extern "C" int distie_attention_decode_bf16(const void*, int64_t, const void*, const void*, const int32_t*, const int32_t*,
                                            const int32_t*, int, const int32_t*, void*, void*, void*, int, int, int, int, float, int, int,
                                            int, int, const int32_t*, hipStream_t) {
  return DISTIE_BAD_ARGUMENT;
}

extern "C" int distie_attention_decode_run_len(const int32_t*, int, int, int, int32_t*, hipStream_t) { return DISTIE_BAD_ARGUMENT; }

extern "C" int distie_attention_prefill_bf16(const void*, int64_t, const void*, const void*, const int32_t*, const int32_t*,
                                             const int32_t*, int, const int32_t*, void*, int, int, int, int, int, float, int, int,
                                             const int32_t*, void*, void*, int, hipStream_t) {
  return DISTIE_BAD_ARGUMENT;
}

extern "C" int distie_attention_prefill_f32_fits() { return 0; }

extern "C" int distie_attention_prefill_f32(const void*, int64_t, const void*, const void*, const int32_t*, const int32_t*,
                                            const int32_t*, int, const int32_t*, void*, int, int, int, int, int, float, int, int,
                                            const int32_t*, void*, void*, int, hipStream_t) {
  return DISTIE_BAD_ARGUMENT;
}

#endif
