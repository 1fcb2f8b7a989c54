// The matrix products of a decode step (up to 16 rows of x) with what stands around them in a layer folded
// in, so that a layer is a chain of six kernels instead of eight and no product hands partial sums to the
// kernel after it:
//
//   * a norm in front (NORM): x = rmsnorm(residual) * weight is computed by every workgroup for itself, from
//     the float32 residual stream, into LDS; the loads of the first weights are issued before that, so the
//     norm runs while they are on their way (worker/src/inference/qwen2/model.py:85-90 for the formula);
//   * the residual sum behind (RESIDUAL): y is the float32 residual stream itself and the product is added
//     to it in place, each element by the one lane that owns it (model.py:288-290);
//   * the epilogues of the packed products: gated activation (model.py:236), bias + rotation + cache write
//     of q/k/v (model.py:108-117, 216-219; worker/src/inference/qwen2/paged_attn.py:360-371).
//
// All of them read the packed copy of the weight (tiles of 16 rows x 32 k in the matrix cores' lane order,
// see gemm.hip) with v_mfma_f32_16x16x32_bf16. A workgroup is WR x WK waves: WR row blocks side by side, the
// k tiles of a row block dealt to WK waves whose sums meet in LDS (in wave order, so the result does not
// depend on timing). Nothing is cut across workgroups. A wave keeps up to two rounds of ROUND tiles of
// weights in flight, asked for before the first product of the round before; with the few waves a decode
// product has, what bounds it is how many bytes are on their way, not how many waves there are.

#include "packed.h"

namespace {

// A barrier for what the waves of a workgroup hand each other through LDS. `__syncthreads()` also waits for
// every load from memory that the wave has in flight, which here would be the weights asked for ahead: the
// products could not start before all of them had arrived. This one waits for the wave's LDS traffic only;
// registers that loads are still filling are guarded by the compiler's own waits where they are used.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

constexpr int XPAD = 8;            // elements between the rows of x in LDS: keeps the reads (lane (r, g): row r, 16 bytes
                                   // at 8 g) spread over the banks

// ------------------------------------------------------------------------------------------------ x into LDS
// xs[XR][kp]: rows of x in bfloat16, k padded with zeros to whole tiles, rows beyond M all zeros. KV:
// float4s of a row that a lane keeps (rows of up to 256 KV elements). Rows are dealt to the waves RA at a
// time (two short rows, one long one, so that the registers suffice beside the weights on their way).
// `load` asks for a wave's first rows, `finish` norms them into LDS (and loads and norms further rows, if the
// wave has any). Loads return in the order in which they were issued: what is asked for before the weights
// arrives before them, and the norm does not wait for the weights.
template <int XR, int WAVES, int KV>
struct NormRows {
  static constexpr int RA = (KV > 8 || XR <= WAVES) ? 1 : 2;
  static constexpr bool EARLY = KV <= 8;       // the norm's weights travel together with the rows
  float4 v[RA][KV];
  float4 w[EARLY ? KV : 1];

  __device__ __forceinline__ static float4 weights_at(const float* __restrict__ norm_weight, int q) {
    return *reinterpret_cast<const float4*>(norm_weight + 4 * q);
  }

  __device__ __forceinline__ void load(const float* __restrict__ residual, const float* __restrict__ norm_weight,
                                       int M, int K, int m0) {
    const int lane = threadIdx.x % 64;
    const int quads = K / 4;
#pragma unroll
    for (int u = 0; u < RA; ++u) {
      const float* row = residual + static_cast<int64_t>(min(m0 + u, M - 1)) * K;
#pragma unroll
      for (int e = 0; e < KV; ++e) v[u][e] = *reinterpret_cast<const float4*>(row + 4 * min(lane + 64 * e, quads - 1));
    }
    if constexpr (EARLY) {
#pragma unroll
      for (int e = 0; e < KV; ++e) w[e] = weights_at(norm_weight, min(lane + 64 * e, quads - 1));
    }
  }

  __device__ __forceinline__ void write(bf16_t* xs, int kp, const float* __restrict__ norm_weight, float eps, int M, int K,
                                        int m0) {
    const int lane = threadIdx.x % 64;
    const int quads = K / 4;
#pragma unroll
    for (int u = 0; u < RA; ++u) {
      const int m = m0 + u;
      if (m >= XR) break;
      bf16_t* dst = xs + static_cast<int64_t>(m) * kp;
      float ss = 0.f;
#pragma unroll
      for (int e = 0; e < KV; ++e)
        if (lane + 64 * e < quads)
          ss += v[u][e].x * v[u][e].x + v[u][e].y * v[u][e].y + v[u][e].z * v[u][e].z + v[u][e].w * v[u][e].w;
      // a row beyond M is written as zeros: its products are dropped, and they must not be NaN on the way
      const float scale = m < M ? rsqrtf(wave_sum(ss) / static_cast<float>(K) + eps) : 0.f;
#pragma unroll
      for (int e = 0; e < KV; ++e) {
        const int q = lane + 64 * e;
        if (q >= quads) continue;
        float4 nw;
        if constexpr (EARLY) nw = w[e]; else nw = weights_at(norm_weight, q);
        const float out[4] = {v[u][e].x * scale * nw.x, v[u][e].y * scale * nw.y, v[u][e].z * scale * nw.z,
                              v[u][e].w * scale * nw.w};
        *reinterpret_cast<uint2*>(dst + 4 * q) = m < M ? pack_bf16x4(out) : uint2{0u, 0u};
      }
      for (int q = quads + lane; q < kp / 4; q += 64) *reinterpret_cast<uint2*>(dst + 4 * q) = uint2{0u, 0u};
    }
  }

  __device__ __forceinline__ void finish(bf16_t* xs, int kp, const float* __restrict__ residual,
                                         const float* __restrict__ norm_weight, float eps, int M, int K, int m0) {
    write(xs, kp, norm_weight, eps, M, K, m0);
#pragma unroll 1
    for (int m = m0 + RA * WAVES; m < XR; m += RA * WAVES) {
      load(residual, norm_weight, M, K, m);
      write(xs, kp, norm_weight, eps, M, K, m);
    }
  }
};

// Rows of x as they are (bfloat16 [M, K] in memory), into the same layout: a wave asks for up to CH 16-byte
// pieces a lane before the weights (`load`) and puts them into LDS afterwards (`finish`, which also fetches
// what did not fit the first time).
template <int XR, int WAVES, int CH>
struct CopyRows {
  uint4 v[CH];

  // piece i of this wave: row and 16-byte chunk, walking the wave's rows one after the other
  __device__ __forceinline__ static void place(int i, int padded, int& m, int& c) {
    const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
    const int per_row = (padded + 63) / 64;
    m = wave + WAVES * (i / per_row);
    c = lane + 64 * (i % per_row);
  }

  __device__ __forceinline__ void load(const bf16_t* __restrict__ x, int kp, int M, int K) {
    const int chunks = K / 8, padded = kp / 8;
#pragma unroll
    for (int i = 0; i < CH; ++i) {
      int m, c;
      place(i, padded, m, c);
      v[i] = *reinterpret_cast<const uint4*>(x + static_cast<int64_t>(min(m, M - 1)) * K + 8 * min(c, chunks - 1));
    }
  }

  __device__ __forceinline__ void finish(bf16_t* xs, const bf16_t* __restrict__ x, int kp, int M, int K) {
    const int chunks = K / 8, padded = kp / 8;
    const int per_row = (padded + 63) / 64;
    const int pieces = per_row * ((XR - static_cast<int>(threadIdx.x / 64) + WAVES - 1) / WAVES);
#pragma unroll
    for (int i = 0; i < CH; ++i) {
      int m, c;
      place(i, padded, m, c);
      if (i < pieces && m < XR && c < padded)
        *reinterpret_cast<uint4*>(xs + static_cast<int64_t>(m) * kp + 8 * c) = (m < M && c < chunks) ? v[i] : uint4{0u, 0u, 0u, 0u};
    }
    for (int i = CH; i < pieces; ++i) {
      int m, c;
      place(i, padded, m, c);
      if (m >= XR || c >= padded) continue;
      uint4 value = uint4{0u, 0u, 0u, 0u};
      if (m < M && c < chunks) value = *reinterpret_cast<const uint4*>(x + static_cast<int64_t>(m) * K + 8 * c);
      *reinterpret_cast<uint4*>(xs + static_cast<int64_t>(m) * kp + 8 * c) = value;
    }
  }
};

// ------------------------------------------------------------------------------------------------ the stream
// Sums of one row block over the k tiles [t_begin, t_end): acc[i] = row 4 g + i of the block, x row r.
// wp: the block's first tile + 8 * lane; `loads`: false for a lane whose rows are not this workgroup's (its
// weights count as zeros). XLDS: x comes from LDS (xrow: this lane's row + 8 g); else from memory (xrow: x
// row min(r, M - 1) + 8 g; k beyond K is not read: the copy holds zeros there).
// `early` runs first (it asks for what x is made from), then two rounds of ROUND tiles are asked for at once,
// then `between` runs (the norm or copy that fills LDS, and its barrier: every wave calls both, with or
// without tiles of its own), then the products begin; a round's registers are asked for again as soon as its
// products are done.
template <bool XLDS, int ROUND, typename Early, typename Between>
__device__ __forceinline__ floatx4 stream_row_block(const bf16_t* __restrict__ wp, bool loads, const bf16_t* xrow,
                                                    int t_begin, int t_end, int K, int g, Early&& early,
                                                    Between&& between) {
  floatx4 acc = {0.f, 0.f, 0.f, 0.f};
  bf16x8 a0[ROUND], a1[ROUND];
  bf16x8 x0[XLDS ? 1 : ROUND], x1[XLDS ? 1 : ROUND];
  const int last = max(t_end - 1, 0);
  // Loads are unconditional (addresses clamped into the block) and nothing looks at a round's registers
  // before its products: a branch or a select between would make the wave wait for all that is in flight.
  auto fetch = [&](bf16x8 (&a)[ROUND], bf16x8 (&xb)[XLDS ? 1 : ROUND], int base) {
#pragma unroll
    for (int j = 0; j < ROUND; ++j) {
      const int t = min(base + j, last);
      a[j] = bf16x8{};
      if (loads) a[j] = *reinterpret_cast<const bf16x8*>(wp + static_cast<int64_t>(t) * PK_TILE);
      if constexpr (!XLDS) xb[j] = *reinterpret_cast<const bf16x8*>(xrow + min(32 * t, K - 8 - 8 * g));
    }
  };
  auto products = [&](bf16x8 (&a)[ROUND], bf16x8 (&xb)[XLDS ? 1 : ROUND], int base) {
#pragma unroll
    for (int j = 0; j < ROUND; ++j) {
      const int t = base + j;
      if (t >= t_end) break;                                       // the same for the whole wave
      bf16x8 b;
      if constexpr (XLDS) {
        b = *reinterpret_cast<const bf16x8*>(xrow + 32 * t);
      } else {
        b = xb[j];
        if (32 * t + 8 * g >= K) b = bf16x8{};                       // the last tile may reach beyond K
      }
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[j], b, acc, 0, 0, 0);
    }
  };
  int base = t_begin;
  // the fences keep the compiler from issuing the loads in another order: it would ask for x last, and the
  // norm would wait for every weight
  early();
  __builtin_amdgcn_sched_barrier(0);
  fetch(a0, x0, base);
  if (base + ROUND < t_end) fetch(a1, x1, base + ROUND);
  __builtin_amdgcn_sched_barrier(0);
  between();
  while (base < t_end) {
    products(a0, x0, base);
    if (base + 2 * ROUND < t_end) fetch(a0, x0, base + 2 * ROUND);
    base += ROUND;
    if (base >= t_end) break;
    products(a1, x1, base);
    if (base + 2 * ROUND < t_end) fetch(a1, x1, base + 2 * ROUND);
    base += ROUND;
  }
  return acc;
}

struct ProductArgs {
  const bf16_t* x;             // [M, K] (X_COPY, X_DIRECT)
  const float* residual;       // [M, K] float32 (X_NORM)
  const float* norm_weight;    // [K]
  float eps;
  const bf16_t* w;             // the packed copy
  const float* bias;           // [N] or null
  void* y;
  int M, N, K;
  int row_blocks;              // of 16 rows of the weight
  RotaryOut rotary;
};

#define OUT_BF16 0       // y: bfloat16 [M, N] ([M, N / 2] when gated)
#define OUT_F32 1        // y: float32 [M, N]
#define OUT_RESIDUAL 2   // y: float32 [M, N], the product is added to what it holds

#define X_NORM 0         // x = rmsnorm(residual) * weight, computed into LDS by the workgroup
#define X_COPY 1         // x copied into LDS by the workgroup
#define X_DIRECT 2       // x read from memory by every lane for itself (rows too long for LDS)

// blockIdx.x: a group of WR row blocks; with HALF, one half (8 rows) of one row block: twice the workgroups
// for weights with few rows, which need every compute unit pulling.
template <int MODE, int XSRC, int OUT, int XR, int WR, int WK, int KV, int ROUND, bool HALF>
__global__ __launch_bounds__(64 * WR * WK) void decode_product_kernel(ProductArgs p) {
  constexpr int WAVES = WR * WK;
  static_assert(!HALF || (WR == 1 && MODE == PK_PLAIN), "halves of row blocks: plain products, one block a workgroup");
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  const int lane = threadIdx.x % 64;
  const int wave = threadIdx.x / 64;
  const int r = lane % 16;
  const int g = lane / 16;
  const int M = p.M, N = p.N, K = p.K;
  const int k_tiles = (K + 31) / 32;
  const int kp = 32 * k_tiles + XPAD;
  const int wr = wave / WK;                    // which of the workgroup's row blocks
  const int wk = wave % WK;                    // which share of its k tiles
  const int block = HALF ? blockIdx.x / 2 : blockIdx.x * WR + wr;
  const int half_of_block = HALF ? blockIdx.x % 2 : 0;
  const bool active = block < p.row_blocks;
  const int per_wave = (k_tiles + WK - 1) / WK;
  const int t_begin = min(k_tiles, wk * per_wave);
  const int t_end = active ? min(k_tiles, t_begin + per_wave) : t_begin;
  const bf16_t* wp = p.w + static_cast<int64_t>(min(block, p.row_blocks - 1)) * k_tiles * PK_TILE + lane * 8;
  const bool loads = !HALF || r / 8 == half_of_block;              // this lane's weight row is the workgroup's
  const bool writes = !HALF || g / 2 == half_of_block;             // this lane's sums are

  // what the epilogue reads is asked for now, so that it has arrived when the sums are there
  float before[4] = {0.f, 0.f, 0.f, 0.f};
  if constexpr (MODE == PK_PLAIN) {
    if (wk == 0 && active && writes && r < M) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int64_t n = static_cast<int64_t>(block) * 16 + 4 * g + i;
        if (n >= N) continue;
        if (p.bias != nullptr) before[i] = p.bias[n];
        if constexpr (OUT == OUT_RESIDUAL) before[i] += static_cast<const float*>(p.y)[static_cast<int64_t>(r) * N + n];
      }
    }
  }
  float2 angle[4] = {};
  int64_t slot = 0;
  if constexpr (MODE == PK_ROTARY) {
    const int half = p.rotary.dim / 2;
    const int per_head = p.rotary.dim / 16;
    const int head = block / per_head, sub = block % per_head;
    const bool turns = block < (p.rotary.heads + p.rotary.kv_heads) * per_head;
    if (wk == 0 && active && r < M) {
      const int d0 = turns ? (g / 2) * half + 8 * sub + 4 * (g % 2) : 16 * sub + 4 * g;
#pragma unroll
      for (int i = 0; i < 4; ++i) before[i] = p.bias != nullptr ? p.bias[static_cast<int64_t>(head) * p.rotary.dim + d0 + i] : 0.f;
      if (turns) {
        const float2* angles = p.rotary.table + static_cast<int64_t>(r) * half + 8 * sub + 4 * (g % 2);
#pragma unroll
        for (int i = 0; i < 4; ++i) angle[i] = angles[i];
      }
      if (p.rotary.write && head >= p.rotary.heads) slot = p.rotary.slots[r];
    }
  }

  floatx4 acc;
  float* part = reinterpret_cast<float*>(lds);                     // [WAVES][4][64] sums that meet in LDS (WK > 1)
  if constexpr (XSRC == X_DIRECT) {
    acc = stream_row_block<false, ROUND>(wp, loads, p.x + static_cast<int64_t>(min(r, M - 1)) * K + 8 * g, t_begin, t_end,
                                         K, g, []() {}, []() {});
  } else if constexpr (XSRC == X_NORM) {
    bf16_t* xs = reinterpret_cast<bf16_t*>(lds + (WK > 1 ? WAVES * 4 * 64 * sizeof(float) : 0));
    NormRows<XR, WAVES, KV> rows;
    const int m0 = NormRows<XR, WAVES, KV>::RA * wave;
    // x is made while the weights are on their way
    acc = stream_row_block<true, ROUND>(
        wp, loads, xs + static_cast<int64_t>(r % XR) * kp + 8 * g, t_begin, t_end, K, g,
        [&]() {
          rows.load(p.residual, p.norm_weight, M, K, m0);
        },
        [&]() {
          rows.finish(xs, kp, p.residual, p.norm_weight, p.eps, M, K, m0);
          lds_barrier();
        });
  } else {
    bf16_t* xs = reinterpret_cast<bf16_t*>(lds + (WK > 1 ? WAVES * 4 * 64 * sizeof(float) : 0));
    CopyRows<XR, WAVES, 8> rows;
    acc = stream_row_block<true, ROUND>(
        wp, loads, xs + static_cast<int64_t>(r % XR) * kp + 8 * g, t_begin, t_end, K, g,
        [&]() { rows.load(p.x, kp, M, K); },
        [&]() {
          rows.finish(xs, p.x, kp, M, K);
          lds_barrier();
        });
  }

  if constexpr (WK > 1) {
    if (wk > 0) {
#pragma unroll
      for (int i = 0; i < 4; ++i) part[(wave * 4 + i) * 64 + lane] = acc[i];
    }
    __syncthreads();
    if (wk > 0) return;
#pragma unroll
    for (int v = 1; v < WK; ++v)
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[i] += part[((wave + v) * 4 + i) * 64 + lane];
  }
  if (!active) return;

  // acc[i]: row 4 g + i of the block, x row r
  if constexpr (MODE == PK_GATED) {
    bf16_t* y = static_cast<bf16_t*>(p.y);
    const int half = N / 2;
    float up[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) up[i] = __shfl_xor(acc[i], 32, 64);          // rows 8..15 of the block: up
    if (g < 2 && r < M) {
      float v[4];
      const int64_t n0 = static_cast<int64_t>(block) * 8 + 4 * g;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float gate = acc[i], u = up[i];
        if (p.bias != nullptr && n0 + i < half) { gate += p.bias[n0 + i]; u += p.bias[half + n0 + i]; }
        v[i] = gate / (1.f + expf(-gate)) * u;
      }
      if (n0 + 3 < half && half % 4 == 0) {
        *reinterpret_cast<uint2*>(y + static_cast<int64_t>(r) * half + n0) = pack_bf16x4(v);
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (n0 + i < half) y[static_cast<int64_t>(r) * half + n0 + i] = from_float<bf16_t>(v[i]);
      }
    }
  } else if constexpr (MODE == PK_ROTARY) {
    bf16_t* y = static_cast<bf16_t*>(p.y);
    const RotaryOut& rotary = p.rotary;
    const int dim = rotary.dim;
    const int half = dim / 2;
    const int per_head = dim / 16;                                  // blocks of a head
    const int rotated_blocks = (rotary.heads + rotary.kv_heads) * per_head;
    const bool turns = block < rotated_blocks;
    const int head = block / per_head;                              // among q, k, v heads in this order
    const int sub = block % per_head;
    // the first of this lane's four columns within its head
    const int d0 = turns ? (g / 2) * half + 8 * sub + 4 * (g % 2) : 16 * sub + 4 * g;
    float own[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) own[i] = acc[i] + before[i];
    float other[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) other[i] = __shfl_xor(own[i], 32, 64);
    if (r >= M) return;
    float v[4];
    if (turns) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        // first half: x1 cos - x2 sin; second half: x2 cos + x1 sin
        v[i] = g < 2 ? own[i] * angle[i].x - other[i] * angle[i].y : own[i] * angle[i].x + other[i] * angle[i].y;
      }
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] = own[i];
    }
    const uint2 packed = pack_bf16x4(v);
    *reinterpret_cast<uint2*>(y + static_cast<int64_t>(r) * N + static_cast<int64_t>(head) * dim + d0) = packed;
    if (rotary.write && head >= rotary.heads) {
      const int64_t page = slot / rotary.block_size;
      const int offset = static_cast<int>(slot % rotary.block_size);
      if (turns) {
        const int kv_head = head - rotary.heads;
        *reinterpret_cast<uint2*>(rotary.k_cache + ((page * rotary.kv_heads + kv_head) * rotary.block_size + offset) * dim + d0) =
            packed;
      } else {
        const int kv_head = head - rotary.heads - rotary.kv_heads;
        bf16_t* at = rotary.v_cache + ((page * rotary.kv_heads + kv_head) * dim + d0) * rotary.block_size + offset;
#pragma unroll
        for (int i = 0; i < 4; ++i) at[static_cast<int64_t>(i) * rotary.block_size] = static_cast<bf16_t>(v[i]);
      }
    }
  } else {
    if (r >= M || !writes) return;
    const int64_t n0 = static_cast<int64_t>(block) * 16 + 4 * g;
    const int64_t at = static_cast<int64_t>(r) * N + n0;
    float sum[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) sum[i] = acc[i] + before[i];        // bias, and for the residual what it held
    if (n0 + 3 < N && N % 4 == 0) {
      if constexpr (OUT == OUT_BF16) {
        *reinterpret_cast<uint2*>(static_cast<bf16_t*>(p.y) + at) = pack_bf16x4(sum);
      } else {
        *reinterpret_cast<float4*>(static_cast<float*>(p.y) + at) = float4{sum[0], sum[1], sum[2], sum[3]};
      }
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if (n0 + i >= N) continue;
        if constexpr (OUT == OUT_BF16) {
          static_cast<bf16_t*>(p.y)[at + i] = from_float<bf16_t>(sum[i]);
        } else {
          static_cast<float*>(p.y)[at + i] = sum[i];
        }
      }
    }
  }
}

template <int MODE, int XSRC, int OUT, int XR, int WR, int WK, int KV, int ROUND, bool HALF>
int launch_one(const ProductArgs& p, hipStream_t stream) {
  constexpr int WAVES = WR * WK;
  const int k_tiles = (p.K + 31) / 32;
  size_t lds = WK > 1 ? WAVES * 4 * 64 * sizeof(float) : 0;
  if (XSRC != X_DIRECT) lds += static_cast<size_t>(XR) * (32 * k_tiles + XPAD) * sizeof(bf16_t);
  if (lds > 160 * 1024) return DISTIE_BAD_ARGUMENT;
  if (lds > 48 * 1024) {
    // more LDS than a launch gets without asking (the compute unit has 160 KB)
    const hipError_t status = hipFuncSetAttribute(
        reinterpret_cast<const void*>(&decode_product_kernel<MODE, XSRC, OUT, XR, WR, WK, KV, ROUND, HALF>),
        hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds));
    if (status != hipSuccess) return static_cast<int>(status);
  }
  const int groups = HALF ? 2 * p.row_blocks : (p.row_blocks + WR - 1) / WR;
  decode_product_kernel<MODE, XSRC, OUT, XR, WR, WK, KV, ROUND, HALF><<<groups, 64 * WAVES, lds, stream>>>(p);
  return launch_status();
}

size_t x_lds_bytes(int rows, int K) { return static_cast<size_t>(rows) * (32 * ((K + 31) / 32) + XPAD) * sizeof(bf16_t); }

// Waves that share a row block's k tiles: each should own what it can have in flight at once (two rounds of 16
// tiles), eight at most.
int waves_along_k(int K) {
  const int tiles = (K + 31) / 32;
  int waves = 1;
  while (waves < 8 && tiles > waves * 16) waves *= 2;
  return waves;
}

bool norm_fits(int K) { return K % 4 == 0 && K <= 4096; }

// x = rmsnorm(residual): MODE, OUT as given; rows of x in LDS: 8 or 16 by M; long rows keep fewer at a time
template <int MODE, int OUT, int WR, int WK, int ROUND>
int launch_norm(const ProductArgs& p, hipStream_t stream) {
  if (p.M <= 8) {
    return p.K > 2048 ? launch_one<MODE, X_NORM, OUT, 8, WR, WK, 16, ROUND, false>(p, stream)
                      : launch_one<MODE, X_NORM, OUT, 8, WR, WK, 8, ROUND, false>(p, stream);
  }
  return p.K > 2048 ? launch_one<MODE, X_NORM, OUT, 16, WR, WK, 16, ROUND, false>(p, stream)
                    : launch_one<MODE, X_NORM, OUT, 16, WR, WK, 8, ROUND, false>(p, stream);
}

template <int WK, bool HALF>
int launch_residual(const ProductArgs& p, hipStream_t stream) {
  const int rows = p.M <= 8 ? 8 : 16;
  if (x_lds_bytes(rows, p.K) + WK * 1024 > 150 * 1024)
    return launch_one<PK_PLAIN, X_DIRECT, OUT_RESIDUAL, 16, 1, WK, 8, 8, HALF>(p, stream);
  if (rows == 8) return launch_one<PK_PLAIN, X_COPY, OUT_RESIDUAL, 8, 1, WK, 8, 16, HALF>(p, stream);
  return launch_one<PK_PLAIN, X_COPY, OUT_RESIDUAL, 16, 1, WK, 8, 16, HALF>(p, stream);
}

}  // namespace

// 1 if the products with a norm in front take rows of K elements (they keep a row in registers).
extern "C" int distie_decode_norm_fits(int K) { return norm_fits(K) ? 1 : 0; }

// residual[M, N] (float32) += x[M, K] * W^T (+ bias): the output projection of a mixer or feed-forward, added
// to the residual stream in place. w_packed: the PLAIN copy. M <= 16.
extern "C" int distie_decode_product_residual(const void* x, const void* w_packed, const float* bias, float* residual,
                                              int M, int N, int K, hipStream_t stream) {
  if (M <= 0) return 0;
  if (M > 16 || N <= 0 || K <= 0 || K % 8 != 0) return DISTIE_BAD_ARGUMENT;
  ProductArgs p = {};
  p.x = static_cast<const bf16_t*>(x);
  p.w = static_cast<const bf16_t*>(w_packed);
  p.bias = bias;
  p.y = residual;
  p.M = M; p.N = N; p.K = K;
  p.row_blocks = (N + 15) / 16;
  // few row blocks (the width of the model): halves of blocks, so that more compute units pull
  const bool halves = p.row_blocks < 192;
#define RESIDUAL(WK) (halves ? launch_residual<WK, true>(p, stream) : launch_residual<WK, false>(p, stream))
  switch (waves_along_k(K)) {
    case 8: return RESIDUAL(8);
    case 4: return RESIDUAL(4);
    case 2: return RESIDUAL(2);
    default: return RESIDUAL(1);
  }
#undef RESIDUAL
}

// y = rmsnorm(residual) * norm_weight times W^T, with the epilogue that `mode` names:
//   0 (plain)  y float32 [M, N] (+ bias): the head;
//   1 (gated)  y bfloat16 [M, N / 2] = silu(gate) * up, w_packed the GATED copy;
//   2 (rotary) y bfloat16 [M, N], bias, rotation by `table`, k and v into the cache, w_packed the ROTARY copy.
// residual: float32 [M, K], K <= 4,096 (distie_decode_norm_fits); norm_weight: float32 [K]; M <= 16.
extern "C" int distie_decode_norm_product(const float* residual, const float* norm_weight, float eps,
                                          const void* w_packed, const float* bias, void* y, int mode,
                                          int M, int N, int K, const void* table, const int32_t* slots, void* k_cache,
                                          void* v_cache, int heads, int kv_heads, int dim, int block_size, int write,
                                          hipStream_t stream) {
  if (M <= 0) return 0;
  if (M > 16 || N <= 0 || K <= 0 || K % 8 != 0 || !norm_fits(K) || mode < 0 || mode > 2 ||
      residual == nullptr || norm_weight == nullptr)
    return DISTIE_BAD_ARGUMENT;
  ProductArgs p = {};
  p.residual = residual;
  p.norm_weight = norm_weight;
  p.eps = eps;
  p.w = static_cast<const bf16_t*>(w_packed);
  p.bias = bias;
  p.y = y;
  p.M = M; p.N = N; p.K = K;
  if (mode == PK_GATED) {
    if (N % 2 != 0) return DISTIE_BAD_ARGUMENT;
    p.row_blocks = (N / 2 + 7) / 8;
    // four row blocks share a workgroup's x, one wave each
    return launch_norm<PK_GATED, OUT_BF16, 4, 1, 16>(p, stream);
  }
  if (mode == PK_ROTARY) {
    if (heads < 1 || kv_heads < 1 || dim < 16 || dim % 16 != 0 || block_size < 1 || table == nullptr ||
        N != (heads + 2 * kv_heads) * dim || (write && (slots == nullptr || k_cache == nullptr || v_cache == nullptr)))
      return DISTIE_BAD_ARGUMENT;
    p.row_blocks = N / 16;
    p.rotary = RotaryOut{static_cast<const float2*>(table), slots, static_cast<bf16_t*>(k_cache),
                         static_cast<bf16_t*>(v_cache), heads, kv_heads, dim, block_size, write};
    switch (waves_along_k(K)) {
      case 8: return launch_norm<PK_ROTARY, OUT_BF16, 1, 8, 16>(p, stream);
      case 4: return launch_norm<PK_ROTARY, OUT_BF16, 1, 4, 16>(p, stream);
      case 2: return launch_norm<PK_ROTARY, OUT_BF16, 1, 2, 16>(p, stream);
      default: return launch_norm<PK_ROTARY, OUT_BF16, 1, 1, 16>(p, stream);
    }
  }
  p.row_blocks = (N + 15) / 16;
  // many row blocks (the vocabulary): eight of them share a workgroup's copy of x
  return launch_norm<PK_PLAIN, OUT_F32, 8, 1, 16>(p, stream);
}
