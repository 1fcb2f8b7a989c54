// Matrix products y[M,N] = x[M,K] * W[N,K]^T (+ bias[N]); W has the layout of the checkpoint.
//
//  * gemm_generic: every combination of float32 / bfloat16 for x, W and y, any M, N, K. Products
//    and sums are float32 FMAs on the vector ALU: this is the true 32-bit path (no matrix-core
//    mode of reduced precision), and the path for weights that a file keeps in 32-bit.
//  * gemm_skinny_bf16: bfloat16 x and W, M <= 64 (decode). Weight-streaming on the matrix cores
//    (v_mfma_f32_16x16x32_bf16): a wave owns 16 rows of W and a slice of K, reads W straight from
//    memory into the A operand (every weight byte is read once), and the small x is the B operand.
//    Slices of K are written side by side and added, in order, by the kernel that reads them.
//  * pack_rows + gemm_packed (up to 16 rows of x a group) and gemm_packed_wide (up to 96 rows a pass): the same streaming on a
//    second copy of W laid out tile by tile in the matrix cores' lane order, with epilogues that finish
//    what follows the product (gated activation; bias, rotation and cache write of q/k/v). Described at
//    their definitions.
//
// The reference leaves these products to a library (worker/src/inference/qwen2/model.py:149-152,
// 231-233, 301); bfloat16 products of many rows (prefill) are left to the library here as well.

#include "common.h"
#include "packed.h"
#include <algorithm>

// ---------------------------------------------------------------- generic
#define GT 64   // tile of M and of N
#define GK 16   // tile of K

template <typename X, typename W, typename Y>
__global__ __launch_bounds__(256) void gemm_generic_kernel(const X* __restrict__ x, const W* __restrict__ w,
                                                           const float* __restrict__ bias, Y* __restrict__ y,
                                                           int M, int N, int K) {
  __shared__ float xs[GK][GT + 4];
  __shared__ float ws[GK][GT + 4];
  const int tx = threadIdx.x % 16;   // columns (N)
  const int ty = threadIdx.x / 16;   // rows (M)
  const int64_t m0 = static_cast<int64_t>(blockIdx.y) * GT;
  const int64_t n0 = static_cast<int64_t>(blockIdx.x) * GT;
  float acc[4][4] = {};
  for (int k0 = 0; k0 < K; k0 += GK) {
    // 64 rows x 16 k of each operand: 1024 elements, 4 per thread; k runs fastest (contiguous reads)
    for (int e = threadIdx.x; e < GT * GK; e += 256) {
      const int r = e / GK;
      const int k = e % GK;
      const bool in_k = k0 + k < K;
      xs[k][r] = (in_k && m0 + r < M) ? to_float(x[(m0 + r) * K + k0 + k]) : 0.f;
      ws[k][r] = (in_k && n0 + r < N) ? to_float(w[(n0 + r) * K + k0 + k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < GK; ++k) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = xs[k][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = ws[k][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int64_t m = m0 + ty * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int64_t n = n0 + tx * 4 + j;
      if (n >= N) continue;
      const float v = acc[i][j] + (bias != nullptr ? bias[n] : 0.f);
      y[m * N + n] = from_float<Y>(v);
    }
  }
}

template <typename X, typename W>
static int gemm_generic_out(const X* x, const W* w, const float* bias, void* y, int y_dtype, int M, int N, int K,
                            hipStream_t stream) {
  dim3 grid((N + GT - 1) / GT, (M + GT - 1) / GT);
  DISTIE_DISPATCH(y_dtype, Y, gemm_generic_kernel<X, W, Y><<<grid, 256, 0, stream>>>(x, w, bias, static_cast<Y*>(y), M, N, K));
  return launch_status();
}

extern "C" int distie_gemm_generic(const void* x, int x_dtype, const void* w, int w_dtype, const float* bias,
                                   void* y, int y_dtype, int M, int N, int K, hipStream_t stream) {
  if (M <= 0) return 0;
  if (N <= 0 || K <= 0) return DISTIE_BAD_ARGUMENT;
  DISTIE_DISPATCH(x_dtype, X, DISTIE_DISPATCH(w_dtype, W, return gemm_generic_out<X, W>(
      static_cast<const X*>(x), static_cast<const W*>(w), bias, y, y_dtype, M, N, K, stream)));
  return DISTIE_BAD_ARGUMENT;
}

// ---------------------------------------------------------------- skinny, bfloat16, matrix cores

#define SK_ROWS 16          // rows of W per wave
#define SK_KSTEP 128        // k per wave iteration: four MFMAs of 32 k each

// One wave per block. blockIdx.x: block of 16 rows of W; blockIdx.y: slice of K.
// MB = ceil(M / 16) column blocks of x (1..4).
// In a k-step, MFMA j works on k0 + 32 j .. + 31; the lane (r = lane % 16, g = lane / 16) holds
// W[n0 + r][k0 + 32 j + 8 g .. + 7] and the same places of x's rows: the four lanes of a row read 64
// contiguous bytes with one instruction. Blocks start at different k-steps of their slice and wrap
// around, so that the waves of a launch do not all pull on the same memory channels at once.
//
// With more than one slice, slice s writes its float32 sums to y + s * M * N (slice 0 adds the bias):
// the consumer adds the slices in order (the kernels that read activations here all can). A sum
// across workgroups inside this kernel would need a device-wide release per wave, which on this
// multi-die part costs more than the product itself.
template <int MB, typename Y>
__global__ __launch_bounds__(64) void gemm_skinny_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
                                                         const float* __restrict__ bias, Y* __restrict__ y,
                                                         int M, int N, int K, int k_per_slice) {
  const int lane = threadIdx.x;
  const int r = lane % 16;
  const int g = lane / 16;
  const int64_t n0 = static_cast<int64_t>(blockIdx.x) * SK_ROWS;
  const int k_begin = blockIdx.y * k_per_slice;
  const int k_end = min(K, k_begin + k_per_slice);

  // rows outside W or x are read from the last valid row and their results dropped
  const int64_t w_row = (n0 + r < N) ? (n0 + r) : static_cast<int64_t>(N - 1);
  const bf16_t* wp = w + w_row * K + 8 * g;
  const bf16_t* xp[MB];
#pragma unroll
  for (int b = 0; b < MB; ++b) xp[b] = x + static_cast<int64_t>(min(b * 16 + r, M - 1)) * K + 8 * g;

  floatx4 acc[MB];
#pragma unroll
  for (int b = 0; b < MB; ++b) acc[b] = floatx4{0.f, 0.f, 0.f, 0.f};

  const int steps = (k_end - k_begin) / SK_KSTEP;
  int step = steps > 0 ? static_cast<int>(blockIdx.x % steps) : 0;
  // Three k-steps at a time with every load issued before the first product: a wave that owns only a few
  // steps (small layers, many slices) then pays one trip to memory instead of one per step.
  constexpr int UN = MB == 1 ? 3 : 1;
  int it = 0;
  for (; it + UN <= steps; it += UN) {
    bf16x8 a[UN][4], xb[UN][MB][4];
#pragma unroll
    for (int u = 0; u < UN; ++u) {
      const int k = k_begin + step * SK_KSTEP;
      step = step + 1 == steps ? 0 : step + 1;
#pragma unroll
      for (int j = 0; j < 4; ++j) a[u][j] = *reinterpret_cast<const bf16x8*>(wp + k + 32 * j);
#pragma unroll
      for (int b = 0; b < MB; ++b)
#pragma unroll
        for (int j = 0; j < 4; ++j) xb[u][b][j] = *reinterpret_cast<const bf16x8*>(xp[b] + k + 32 * j);
    }
#pragma unroll
    for (int u = 0; u < UN; ++u)
#pragma unroll
      for (int b = 0; b < MB; ++b)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u][j], xb[u][b][j], acc[b], 0, 0, 0);
  }
  for (; it < steps; ++it) {
    const int k = k_begin + step * SK_KSTEP;
    step = step + 1 == steps ? 0 : step + 1;
    bf16x8 a[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) a[j] = *reinterpret_cast<const bf16x8*>(wp + k + 32 * j);
#pragma unroll
    for (int b = 0; b < MB; ++b) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const bf16x8 xb = *reinterpret_cast<const bf16x8*>(xp[b] + k + 32 * j);
        acc[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[j], xb, acc[b], 0, 0, 0);
      }
    }
  }
  // the rest of the slice (K is a multiple of 8; the slice's end need not be a multiple of 128)
  for (int k = k_begin + steps * SK_KSTEP; k < k_end; k += 32) {
    bf16x8 a = {};
    const bool in = k + 8 * g < k_end;
    if (in) a = *reinterpret_cast<const bf16x8*>(wp + k);
#pragma unroll
    for (int b = 0; b < MB; ++b) {
      bf16x8 xb = {};
      if (in) xb = *reinterpret_cast<const bf16x8*>(xp[b] + k);
      acc[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, xb, acc[b], 0, 0, 0);
    }
  }

  // acc[b][i] = sum for W row n0 + 4 g + i and x row 16 b + r
  Y* out = y + static_cast<int64_t>(blockIdx.y) * M * N;
  const bool with_bias = bias != nullptr && blockIdx.y == 0;
#pragma unroll
  for (int b = 0; b < MB; ++b) {
    const int m = b * 16 + r;
    if (m >= M) continue;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int64_t n = n0 + 4 * g + i;
      if (n < N) out[static_cast<int64_t>(m) * N + n] = from_float<Y>(acc[b][i] + (with_bias ? bias[n] : 0.f));
    }
  }
}

// How a product is cut along K: enough waves to fill the chip (one to two thousand), slices that are a multiple
// of the k-step and at least 384 long. More waves than that make the product slower and give the kernel that adds
// the slices more to read: the 7B shape's down product (224 row blocks, K = 18,944) took 31.4 us in 30 slices,
// 30.2 in 15, 28.3 in 8, 33.7 in 4, the norm behind it 6.2, 5.2, 4.8 us; its o product 7.5 us in 7 slices, 8.2 in 4,
// 10.5 in 2; the 1.5B shape's down 8.4 us in 14 slices, 8.9 in 8, 12.1 in 4.
static void skinny_plan(int N, int K, int* slices, int* k_per_slice) {
  const int row_blocks = (N + SK_ROWS - 1) / SK_ROWS;
  int want = 1;
  while (want < 64 && row_blocks * want <= 1024 && K / (want * 2) >= 384) want *= 2;
  int per = (K + want - 1) / want;
  per = (per + SK_KSTEP - 1) / SK_KSTEP * SK_KSTEP;
  *k_per_slice = per;
  *slices = (K + per - 1) / per;
}

// The number of K slices the launcher will use for this shape.
extern "C" int distie_gemm_skinny_slices(int M, int N, int K) {
  (void)M;
  int slices, per;
  skinny_plan(N, K, &slices, &per);
  return slices;
}

// y: [M, N] of y_dtype if the shape gets one slice, else float32 [slices, M, N] (y_dtype must be float32).
extern "C" int distie_gemm_skinny_bf16(const void* x, const void* w, const float* bias, void* y, int y_dtype,
                                       int M, int N, int K, hipStream_t stream) {
  if (M <= 0) return 0;
  if (M > 64 || N <= 0 || K <= 0 || K % 8 != 0) return DISTIE_BAD_ARGUMENT;
  int slices, k_per_slice;
  skinny_plan(N, K, &slices, &k_per_slice);
  if (slices > 1 && y_dtype != DISTIE_F32) return DISTIE_BAD_ARGUMENT;
  dim3 grid((N + SK_ROWS - 1) / SK_ROWS, slices);
  const bf16_t* xb = static_cast<const bf16_t*>(x);
  const bf16_t* wb = static_cast<const bf16_t*>(w);
  const int mb = (M + 15) / 16;
#define SKINNY(MB)                                                                                          \
  DISTIE_DISPATCH(y_dtype, Y, gemm_skinny_kernel<MB, Y><<<grid, 64, 0, stream>>>(                           \
                                  xb, wb, bias, static_cast<Y*>(y), M, N, K, k_per_slice))
  switch (mb) {
    case 1: SKINNY(1); break;
    case 2: SKINNY(2); break;
    case 3: SKINNY(3); break;
    default: SKINNY(4); break;
  }
#undef SKINNY
  return launch_status();
}

// ---------------------------------------------------------------- skinny on packed weights
// A second copy of a weight in the order in which the matrix cores take it: tiles of 16 rows x 32 k,
// the 1 KB of a tile in lane order (lane = 16 g + r holds row r of the block, k 32 kt + 8 g .. + 7), tiles
// ordered [row block][k tile], k padded with zeros to whole tiles. One load instruction of a wave then
// reads 1 KB of consecutive bytes (eight whole cache lines) instead of 64 bytes from each of 16 rows,
// which brought 15-25 % on every shape measured.
//
// Which row of W sits at which place of a block is given by a row map (-1: a row of zeros), so that a
// wave can own the rows its epilogue needs together:
//  * PLAIN: rows in order.
//  * GATED: the weight stacks a gate and an up projection ([2 I, K]); block b holds gate rows 8 b .. + 7 and
//    then up rows 8 b .. + 7, and the kernel writes silu(gate) * up ([M, I]) itself.
//  * ROTARY: the weight stacks q, k and v heads of size D, all of D rotated (pairs j, j + D / 2). Block
//    (head, s) of a q or k head holds its rows 8 s .. + 7 and D / 2 + 8 s .. + 7, blocks of v heads hold 16 rows
//    in order. The kernel adds the bias, turns the pairs by the token's angle, writes q, k, v to the
//    [M, N] result and k and v into the paged cache.
// In all of them lanes 0-31 of the accumulator hold rows 0-7 of the block and lanes 32-63 rows 8-15 for
// the same tokens, so partners meet through one exchange between lane l and lane l ^ 32.

__global__ __launch_bounds__(256) void pack_rows_kernel(const bf16_t* __restrict__ w, bf16_t* __restrict__ out,
                                                        const int32_t* __restrict__ row_map, int K, int64_t row_blocks,
                                                        int k_tiles) {
  const int64_t chunk = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;     // 8 elements
  if (chunk >= row_blocks * k_tiles * 64) return;
  const int lane = static_cast<int>(chunk % 64);
  const int64_t tile = chunk / 64;
  const int kt = static_cast<int>(tile % k_tiles);
  const int64_t nb = tile / k_tiles;
  const int64_t n = row_map[nb * 16 + lane % 16];
  const int k = 32 * kt + 8 * (lane / 16);
  uint4 v = {0u, 0u, 0u, 0u};
  if (n >= 0 && k < K) v = *reinterpret_cast<const uint4*>(w + n * K + k);       // K is a multiple of 8
  *reinterpret_cast<uint4*>(out + chunk * 8) = v;
}

// out: row_blocks * ceil(K / 32) * 512 elements; row_map: int32 [16 * row_blocks] on the device, entries in
// [-1, N) (the caller's duty).
extern "C" int distie_pack_rows(const void* w, void* out, const int32_t* row_map, int row_blocks, int K,
                                hipStream_t stream) {
  if (row_blocks <= 0 || K <= 0 || K % 8 != 0) return DISTIE_BAD_ARGUMENT;
  const int k_tiles = (K + 31) / 32;
  const int64_t chunks = static_cast<int64_t>(row_blocks) * k_tiles * 64;
  pack_rows_kernel<<<static_cast<unsigned>((chunks + 255) / 256), 256, 0, stream>>>(
      static_cast<const bf16_t*>(w), static_cast<bf16_t*>(out), row_map, K, row_blocks, k_tiles);
  return launch_status();
}

// The four tiles of one k-step for COUNT k-steps: every load issued before the first product.
template <int COUNT>
__device__ __forceinline__ void packed_steps(const bf16_t* wp, const bf16_t* xp, int t_begin, int steps, int& step,
                                             floatx4& acc) {
  bf16x8 a[COUNT][4], xb[COUNT][4];
#pragma unroll
  for (int u = 0; u < COUNT; ++u) {
    const int t = t_begin + 4 * step;
    step = step + 1 == steps ? 0 : step + 1;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      a[u][j] = *reinterpret_cast<const bf16x8*>(wp + static_cast<int64_t>(t + j) * PK_TILE);
      xb[u][j] = *reinterpret_cast<const bf16x8*>(xp + 32 * (t + j));
    }
  }
#pragma unroll
  for (int u = 0; u < COUNT; ++u)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u][j], xb[u][j], acc, 0, 0, 0);
}

// The sums of one row block over the k tiles [t_begin, t_end): acc[i] = row 4 g + i of the block, x row r.
// wp: the block's first tile + 8 * lane; xp: x row min(r, M - 1) + 8 g.
__device__ __forceinline__ floatx4 packed_accumulate(const bf16_t* wp, const bf16_t* xp, int t_begin, int t_end, int K,
                                                     int g, unsigned stagger) {
  constexpr int UN = 4;
  floatx4 acc = {0.f, 0.f, 0.f, 0.f};
  const int t_whole = min(K / 32, t_end);                 // tiles before this one lie inside K for every lane
  const int steps = max(0, t_whole - t_begin) / 4;
  int step = steps > 0 ? static_cast<int>(stagger % steps) : 0;      // staggered start, wraps around
  int it = 0;
  for (; it + UN <= steps; it += UN) packed_steps<UN>(wp, xp, t_begin, steps, step, acc);
  switch (steps - it) {
    case 3: packed_steps<3>(wp, xp, t_begin, steps, step, acc); break;
    case 2: packed_steps<2>(wp, xp, t_begin, steps, step, acc); break;
    case 1: packed_steps<1>(wp, xp, t_begin, steps, step, acc); break;
    default: break;
  }
  // the last tiles, at most three whole ones and one that reaches beyond K (the copy holds zeros there, x
  // is not read): loaded together
  const int t_rest = t_begin + 4 * steps;
  if (t_rest < t_end) {
    bf16x8 a[4], xb[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int t = t_rest + j;
      a[j] = bf16x8{};
      xb[j] = bf16x8{};
      if (t < t_end) a[j] = *reinterpret_cast<const bf16x8*>(wp + static_cast<int64_t>(t) * PK_TILE);
      if (t < t_end && 32 * t + 8 * g < K) xb[j] = *reinterpret_cast<const bf16x8*>(xp + 32 * t);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[j], xb[j], acc, 0, 0, 0);
  }
  return acc;
}


// blockIdx.x: row block; blockIdx.y: slice of K (PLAIN only; slices side by side in y, bias on slice 0, as
// gemm_skinny_kernel); blockIdx.z: a group of 16 rows of x (with more than 16 rows the weights are read once
// per group, from the L2 after the first: the choice for weights too small to occupy the chip through the
// wide kernel below). The WAVES waves of a workgroup share the slice's tiles and add their sums through
// LDS; wave 0 writes.
template <typename Y, int MODE, int WAVES>
__global__ __launch_bounds__(64 * WAVES) void gemm_packed_kernel(const bf16_t* __restrict__ x,
                                                                 const bf16_t* __restrict__ w,
                                                                 const float* __restrict__ bias, Y* __restrict__ y,
                                                                 int M, int N, int K, int tiles_per_slice,
                                                                 RotaryOut rotary) {
  const int lane = threadIdx.x % 64;
  const int wave = threadIdx.x / 64;
  const int r = lane % 16;
  const int g = lane / 16;
  const int m_all = M;
  const int m0 = 16 * blockIdx.z;
  x += static_cast<int64_t>(m0) * K;
  M = min(16, M - m0);
  if constexpr (MODE == PK_ROTARY) {
    y += static_cast<int64_t>(m0) * N;
    rotary.table += static_cast<int64_t>(m0) * (rotary.dim / 2);
    if (rotary.slots != nullptr) rotary.slots += m0;
  } else if constexpr (MODE == PK_GATED) {
    y += static_cast<int64_t>(m0) * (N / 2);
  } else {
    y += static_cast<int64_t>(m0) * N;
  }
  const int k_tiles = (K + 31) / 32;
  const int s_begin = blockIdx.y * tiles_per_slice;
  const int s_end = min(k_tiles, s_begin + tiles_per_slice);
  int t_begin = s_begin, t_end = s_end;
  if constexpr (WAVES > 1) {
    const int per_wave = ((s_end - s_begin + WAVES - 1) / WAVES + 3) / 4 * 4;
    t_begin = min(s_end, s_begin + wave * per_wave);
    t_end = min(s_end, t_begin + per_wave);
  }
  const bf16_t* wp = w + static_cast<int64_t>(blockIdx.x) * k_tiles * PK_TILE + lane * 8;
  const bf16_t* xp = x + static_cast<int64_t>(min(r, M - 1)) * K + 8 * g;      // rows beyond M: results dropped
  floatx4 acc = packed_accumulate(wp, xp, t_begin, t_end, K, g, blockIdx.x + wave);

  if constexpr (WAVES > 1) {
    __shared__ float part[WAVES - 1][4][64];
    if (wave > 0) {
#pragma unroll
      for (int i = 0; i < 4; ++i) part[wave - 1][i][lane] = acc[i];
    }
    __syncthreads();
    if (wave > 0) return;
#pragma unroll
    for (int v = 0; v < WAVES - 1; ++v)
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[i] += part[v][i][lane];
  }

  if constexpr (MODE == PK_GATED) {
    const int half = N / 2;
    float up[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) up[i] = __shfl_xor(acc[i], 32, 64);          // rows 8..15 of the block: up
    if (g < 2 && r < M) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int64_t n = static_cast<int64_t>(blockIdx.x) * 8 + 4 * g + i;
        if (n >= half) continue;
        float gate = acc[i], u = up[i];
        if (bias != nullptr) { gate += bias[n]; u += bias[half + n]; }
        y[static_cast<int64_t>(r) * half + n] = from_float<Y>(gate / (1.f + expf(-gate)) * u);
      }
    }
  } else if constexpr (MODE == PK_ROTARY) {
    const int dim = rotary.dim;
    const int half = dim / 2;
    const int per_head = dim / 16;                                  // blocks of a head
    const int rotated_blocks = (rotary.heads + rotary.kv_heads) * per_head;
    const int b = blockIdx.x;
    const bool turns = b < rotated_blocks;
    const int head = b / per_head;                                  // among q, k, v heads in this order
    const int sub = b % per_head;
    // the first of this lane's four columns within its head
    const int d0 = turns ? (g / 2) * half + 8 * sub + 4 * (g % 2) : 16 * sub + 4 * g;
    float own[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) own[i] = acc[i] + (bias != nullptr ? bias[static_cast<int64_t>(head) * dim + d0 + i] : 0.f);
    float other[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) other[i] = __shfl_xor(own[i], 32, 64);
    if (r >= M) return;
    float v[4];
    if (turns) {
      const float2* angles = rotary.table + static_cast<int64_t>(r) * half + 8 * sub + 4 * (g % 2);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float2 cs = angles[i];
        // first half: x1 cos - x2 sin; second half: x2 cos + x1 sin
        v[i] = g < 2 ? own[i] * cs.x - other[i] * cs.y : own[i] * cs.x + other[i] * cs.y;
      }
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] = own[i];
    }
    const uint2 packed = pack_bf16x4(v);
    *reinterpret_cast<uint2*>(y + static_cast<int64_t>(r) * N + static_cast<int64_t>(head) * dim + d0) = packed;
    if (rotary.write && head >= rotary.heads) {
      const int64_t slot = rotary.slots[r];
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
    Y* out = y + static_cast<int64_t>(blockIdx.y) * m_all * N;
    const bool with_bias = bias != nullptr && blockIdx.y == 0;
    if (r < M) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int64_t n = static_cast<int64_t>(blockIdx.x) * 16 + 4 * g + i;
        if (n < N) out[static_cast<int64_t>(r) * N + n] = from_float<Y>(acc[i] + (with_bias ? bias[n] : 0.f));
      }
    }
  }
}

// Waves of a workgroup: each should own about four k-steps (one trip to memory).
static int packed_waves(int K) {
  const int steps = K / SK_KSTEP;
  return steps >= 48 ? 16 : steps >= 24 ? 8 : steps >= 8 ? 4 : steps >= 4 ? 2 : 1;
}

// y: as distie_gemm_skinny_bf16 (the same cut along K: slices go to other workgroups, hence to other
// compute units, which a product with few rows of W needs to pull its bytes fast enough);
// gated: [M, N / 2] of y_dtype, never cut. Up to 256 rows of x, in groups of 16.
extern "C" int distie_gemm_packed_bf16(const void* x, const void* w_packed, const float* bias, void* y, int y_dtype,
                                       int M, int N, int K, int gated, hipStream_t stream) {
  if (M <= 0) return 0;
  if (M > 256 || N <= 0 || K <= 0 || K % 8 != 0 || (gated && N % 2 != 0)) return DISTIE_BAD_ARGUMENT;
  int slices = 1, k_per_slice = (K + SK_KSTEP - 1) / SK_KSTEP * SK_KSTEP;
  if (!gated) skinny_plan(N, K, &slices, &k_per_slice);
  if (slices > 1 && y_dtype != DISTIE_F32) return DISTIE_BAD_ARGUMENT;
  const int row_blocks = gated ? (N / 2 + 7) / 8 : (N + 15) / 16;
  dim3 grid(row_blocks, slices, (M + 15) / 16);
  const bf16_t* xb = static_cast<const bf16_t*>(x);
  const bf16_t* wb = static_cast<const bf16_t*>(w_packed);
  const RotaryOut none = {};
  if (gated && M <= 8) {
    // The gated product is not cut along K (the activation needs the whole sum), so a row block's K goes to the four
    // waves of a workgroup, which add their sums through LDS: up to 8 rows of x that is faster than one wave a row
    // block (gate+up of the 1.5B shape 13.2 -> 12.3 us at 8 rows, 12.8 -> 11.4 at one row; the 7B shape's 54.9 -> 50.8;
    // the decode step at batch 1 and 4 2.7 % faster, at batch 8 the same), at 16 rows slower (15.7 -> 16.3 us); with
    // eight waves slower everywhere but at the 7B shape.
    DISTIE_DISPATCH(y_dtype, Y, (gemm_packed_kernel<Y, PK_GATED, 4><<<grid, 256, 0, stream>>>(
                                    xb, wb, bias, static_cast<Y*>(y), M, N, K, k_per_slice / 32, none)));
  } else if (gated) {
    DISTIE_DISPATCH(y_dtype, Y, (gemm_packed_kernel<Y, PK_GATED, 1><<<grid, 64, 0, stream>>>(
                                    xb, wb, bias, static_cast<Y*>(y), M, N, K, k_per_slice / 32, none)));
  } else {
    DISTIE_DISPATCH(y_dtype, Y, (gemm_packed_kernel<Y, PK_PLAIN, 1><<<grid, 64, 0, stream>>>(
                                    xb, wb, bias, static_cast<Y*>(y), M, N, K, k_per_slice / 32, none)));
  }
  return launch_status();
}

// ---------------------------------------------------------------- packed weights, up to 96 rows of x a pass
// A workgroup of WAVES waves owns as many row blocks (one a wave) and one slice of K. Per k-step of 128 the
// weights go straight into registers, some k-steps ahead; the x tile ([16 MB rows, 128 k], the same for
// all waves) is fetched as far ahead, into registers, and put into LDS (two stages) right before it is used,
// so that x is read from the L2 once per workgroup and not once per wave.
// Epilogues as in gemm_packed_kernel, for every block of 16 rows of x.
//
//
// WAVES is two for the gated product of up to 32 rows of x in all, else four. What streams the weights fastest here is many small
// workgroups, spread evenly over the compute units (the same loop with x left out, gate+up of the 1.5B shape,
// 55 MB: 13.0 us with one wave a workgroup, 13.7 with two, 15.8 with four, of which there are 280 for 256 compute
// units); but a smaller workgroup reads x more often. At 32 rows two waves are best (15.8 us against 18.3 with
// four and 17.2 with one; the decode step at batch 24 and 32 is 6 and 5 % faster); from 48 rows on, and with the
// rows taken in two passes, four are (batch 64: 3 % slower with two, a portion of 200 tokens 8 %). The products whose
// K is cut into slices (more workgroups already) are faster with four at every number of rows.
// How far ahead the loads run matters little beside that (four, six or eight k-steps: the same time), as long as
// the wave never waits for all of them at once.
template <int MB, int WAVES>
constexpr int wd_stages() { return WAVES == 2 && MB == 1 ? 8 : 4; }    // (k-steps under way; eight with four waves filled the registers so far that fewer workgroups fit a compute unit)
// elements of an x row in LDS: a stride of 32 bytes more than a multiple of 64 keeps the reads (lane (r, g):
// row r, byte 16 g) free of bank conflicts; with 16 bytes more every read costs twice (measured)
constexpr int WD_XROW = SK_KSTEP + 16;
// blocks of 16 rows of x a pass at most: with seven and eight the registers (x is fetched as far ahead as the weights)
// leave one wave a SIMD, and eight waves a workgroup spill or gain nothing (7B shape, decode step at batch 128: one
// pass of 8 blocks 11.4 ms with four waves, 9.7 with eight, as two passes of 4; at batch 80 and 96 one pass of 5 and
// 6 blocks takes 6.8 and 8.1 ms against 7.7 and 8.3 in two passes, the weights coming from memory once)
constexpr int WD_MAX_BLOCKS = 6;

// MODE PK_ROTARY here: the weight is the ROTARY copy of a stacked q/k/v weight (rotation partners in one block), the
// result is the plain product, every sum written to the column its row of W has: the rotation needs the whole
// sum over K, which this kernel cuts into slices, so it is left to the kernel that adds the slices.
struct HeadRows {
  int heads, kv_heads, dim;
};

template <typename Y, int MODE, int MB, int WD_WAVES>
__global__ __launch_bounds__(64 * WD_WAVES) void gemm_packed_wide_kernel(const bf16_t* __restrict__ x,
                                                               const bf16_t* __restrict__ w,
                                                               const float* __restrict__ bias, Y* __restrict__ y,
                                                               int M, int N, int K, int row_blocks, int tiles_per_slice,
                                                               int m_group, HeadRows head_rows) {
  __shared__ __attribute__((aligned(16))) bf16_t xs[2][MB * 16][WD_XROW];
  // blockIdx.z: a group of m_group rows of x. The groups run one after the other over the whole weight, so
  // the second reads it from the memory-side cache (if it fits there; the launcher decides).
  const int m_all = M;
  const int m0 = blockIdx.z * m_group;
  x += static_cast<int64_t>(m0) * K;
  y += static_cast<int64_t>(m0) * (MODE == PK_GATED ? N / 2 : N);
  M = min(m_group, M - m0);
  constexpr int WD_STAGES = wd_stages<MB, WD_WAVES>();
  const int tid = threadIdx.x;
  const int lane = tid % 64;
  const int wave = tid / 64;
  const int r = lane % 16;
  const int g = lane / 16;
  const int k_tiles = (K + 31) / 32;
  const int s_begin = blockIdx.y * tiles_per_slice;
  const int s_end = min(k_tiles, s_begin + tiles_per_slice);
  const int steps = (s_end - s_begin + 3) / 4;
  const int block = blockIdx.x * WD_WAVES + wave;
  const bool active = block < row_blocks;                       // a wave without a row block still carries x
  const bf16_t* wp = w + static_cast<int64_t>(min(block, row_blocks - 1)) * k_tiles * PK_TILE + lane * 8;
  // this thread's part of an x tile: rows XROWS p + tid / 16 (p < XP), k 8 (tid % 16) .. + 7 of the step
  const int x_row = tid / 16;
  const int x_chunk = tid % 16;
  constexpr int XP = (MB * 4 + WD_WAVES - 1) / WD_WAVES;         // pieces of an x tile a thread carries
  constexpr int XROWS = 4 * WD_WAVES;                           // rows of the tile the threads cover at once
  const bf16_t* xsrc[XP];
#pragma unroll
  for (int p = 0; p < XP; ++p) xsrc[p] = x + static_cast<int64_t>(min(XROWS * p + x_row, M - 1)) * K;

  bf16x8 a[WD_STAGES][4];
  uint4 xr[WD_STAGES][XP];
  floatx4 acc[MB];
#pragma unroll
  for (int b = 0; b < MB; ++b) acc[b] = floatx4{0.f, 0.f, 0.f, 0.f};

  // Loads are unconditional, and nothing but arithmetic stands between a load and its use, in the same order in
  // every path into the loop: only then does the compiler count how many younger loads may stay in flight at each
  // use (a load under a branch, a select that it turns into one, or paths that issue different loads, and it
  // waits for all of them instead: measured, one trip to memory per WD_STAGES k-steps with nothing else under
  // way). Addresses are clamped into the buffers instead. A weight tile past the slice's end is read from the
  // slice's last tile (the same rows, so whatever it holds reaches no output it would not reach anyway) and
  // meets zeros in x: x past the slice or past K is masked to zeros when it is put into LDS. A wave without a
  // row block computes on the last block's weights and writes nothing.
  auto x_inside = [&](int step) {
    const int t0 = s_begin + 4 * step;
    return 32 * t0 + 8 * x_chunk < K && t0 + x_chunk / 4 < s_end;
  };
  auto fetch = [&](int step, int slot) {
    const int t0 = s_begin + 4 * step;
#pragma unroll
    for (int j = 0; j < 4; ++j)
      a[slot][j] = *reinterpret_cast<const bf16x8*>(wp + static_cast<int64_t>(min(t0 + j, s_end - 1)) * PK_TILE);
    const int k = x_inside(step) ? 32 * t0 + 8 * x_chunk : 0;
#pragma unroll
    for (int p = 0; p < XP; ++p) xr[slot][p] = *reinterpret_cast<const uint4*>(xsrc[p] + k);
  };

#pragma unroll
  for (int slot = 0; slot < WD_STAGES; ++slot) fetch(slot, slot);         // (beyond the last step: clamped, unused)

  // One k-step: x of this step into LDS, barrier, products. Stage `slot % 2` was last read two k-steps ago;
  // every wave has passed the barrier of the k-step in between, so all of them are done with it.
  auto k_step = [&](int step, int slot) {
    const int stage = slot % 2;
    const uint32_t keep = x_inside(step) ? 0xffffffffu : 0u;
#pragma unroll
    for (int p = 0; p < XP; ++p) {
      const uint4 v = xr[slot][p];
      if (XROWS * (p + 1) <= MB * 16 || XROWS * p + x_row < MB * 16)       // (the last piece may reach past the tile)
        *reinterpret_cast<uint4*>(&xs[stage][XROWS * p + x_row][8 * x_chunk]) = uint4{v.x & keep, v.y & keep, v.z & keep, v.w & keep};
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int b = 0; b < MB; ++b) {
        const bf16x8 xb = *reinterpret_cast<const bf16x8*>(&xs[stage][16 * b + r][32 * j + 8 * g]);
        acc[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[slot][j], xb, acc[b], 0, 0, 0);
      }
  };
  int s = 0;
  for (; s + 2 * WD_STAGES <= steps; s += WD_STAGES) {
#pragma unroll
    for (int slot = 0; slot < WD_STAGES; ++slot) {
      k_step(s + slot, slot);
      fetch(s + slot + WD_STAGES, slot);
    }
  }
  // the last k-steps: what they need is under way already
#pragma unroll
  for (int round = 0; round < 2; ++round) {
#pragma unroll
    for (int slot = 0; slot < WD_STAGES; ++slot) {
      if (s + slot >= steps) break;
      k_step(s + slot, slot);
      if (round == 0 && s + slot + WD_STAGES < steps) fetch(s + slot + WD_STAGES, slot);
    }
    s += WD_STAGES;
    if (s >= steps) break;
  }
  if (!active) return;

  // acc[b][i] = sum for row 4 g + i of the block and x row 16 b + r
#pragma unroll
  for (int b = 0; b < MB; ++b) {
    const int m = 16 * b + r;
    if constexpr (MODE == PK_GATED) {
      const int half = N / 2;
      float up[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) up[i] = __shfl_xor(acc[b][i], 32, 64);
      if (g < 2 && m < M) {
        float v[4];
        const int64_t n0 = static_cast<int64_t>(block) * 8 + 4 * g;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          float gate = acc[b][i], u = up[i];
          if (bias != nullptr && n0 + i < half) { gate += bias[n0 + i]; u += bias[half + n0 + i]; }
          v[i] = gate / (1.f + expf(-gate)) * u;
        }
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (n0 + i < half) y[static_cast<int64_t>(m) * half + n0 + i] = from_float<Y>(v[i]);
      }
    } else {
      Y* out = y + static_cast<int64_t>(blockIdx.y) * m_all * N;
      const bool with_bias = bias != nullptr && blockIdx.y == 0;
      int64_t n0 = static_cast<int64_t>(block) * 16 + 4 * g;        // the column of the lane's first sum
      if constexpr (MODE == PK_ROTARY) {
        // block (head, sub) of a q or k head holds the head's rows 8 sub .. + 7 and dim / 2 + 8 sub .. + 7
        const int per_head = head_rows.dim / 16;
        const int head = block / per_head;
        const int sub = block % per_head;
        if (head < head_rows.heads + head_rows.kv_heads)
          n0 = static_cast<int64_t>(head) * head_rows.dim + (g / 2) * (head_rows.dim / 2) + 8 * sub + 4 * (g % 2);
      }
      if (m < M) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int64_t n = n0 + i;
          if (n < N) out[static_cast<int64_t>(m) * N + n] = from_float<Y>(acc[b][i] + (with_bias ? bias[n] : 0.f));
        }
      }
    }
  }
}

// Slices of K for the wide kernel (the products that are cut run in workgroups of four waves): enough waves for the
// chip, five hundred and more (with a thousand the 7B shape's down, o and q/k/v products at 48 and 64 rows were 4-10 %
// slower, the 1.5B shape's the same), slices of whole k-steps, at least two k-steps long.
static void wide_plan(int row_blocks, int K, int* slices, int* tiles_per_slice) {
  constexpr int WD_WAVES = 4;
  const int groups = (row_blocks + WD_WAVES - 1) / WD_WAVES;
  const int steps = (K + SK_KSTEP - 1) / SK_KSTEP;
  int want = 1;
  while (want < 64 && groups * want * WD_WAVES < 512 && steps / (want * 2) >= 2) want *= 2;
  int per = (steps + want - 1) / want;
  *tiles_per_slice = 4 * per;
  *slices = (steps + per - 1) / per;
}

extern "C" int distie_gemm_packed_wide_slices(int N, int K) {
  int slices, per;
  wide_plan((N + 15) / 16, K, &slices, &per);
  return slices;
}

// Up to 256 rows of x, at most 96 a pass. mode 0: y [M, N] of y_dtype, or float32 [slices, M, N] when the plan cuts K
// (distie_gemm_packed_wide_slices); 1 (gated): [M, N / 2].
static int packed_wide_launch(const bf16_t* x, const bf16_t* w, const float* bias, void* y, int y_dtype, int M, int N,
                              int K, int mode, int pass_blocks, hipStream_t stream, HeadRows head_rows = HeadRows{0, 0, 0}) {
  const int row_blocks = mode == PK_GATED ? (N / 2 + 7) / 8 : (N + 15) / 16;
  int slices = 1, tiles_per_slice = 4 * ((K + SK_KSTEP - 1) / SK_KSTEP);
  if (mode != PK_GATED) wide_plan(row_blocks, K, &slices, &tiles_per_slice);
  if (slices > 1 && y_dtype != DISTIE_F32) return DISTIE_BAD_ARGUMENT;
  // pass_blocks: the rows of x are taken in passes of 16 * pass_blocks rows over the weight (0: 64 rows a pass),
  // with more workgroups and fewer registers and less LDS each; worth it if the weight fits the memory-side
  // cache, from which the later passes then read it (measured at 64 rows in two passes, cold: down 18.3 ->
  // 15.4 us, gate+up 22.4 -> 21.3 us; a weight of 270 MB gets slower, being fetched from memory twice).
  const int m_group = (pass_blocks >= 1 && pass_blocks <= WD_MAX_BLOCKS) ? 16 * pass_blocks : 64;
  const int groups = (M + m_group - 1) / m_group;
  const int mb = (std::min(M, m_group) + 15) / 16;
  // two waves a workgroup for the gated product of up to 32 rows; the products whose K is cut are faster with four
  // at every number of rows (at 32 rows: the 7B shape's o + down 42.5 -> 36.2 us, its head 239 -> 220, the 1.5B shape's
  // down 9.7 -> 9.1, its head 107 -> 96; gate+up 15.6 with two against 17.1 at the 1.5B shape, 57.3 and 57.4 at the 7B)
  const int waves = (mode == PK_GATED && M <= 32) ? 2 : 4;
  dim3 grid((row_blocks + waves - 1) / waves, slices, groups);
#define WIDE(MODE, MB, WAVES)                                                                                   \
  DISTIE_DISPATCH(y_dtype, Y, (gemm_packed_wide_kernel<Y, MODE, MB, WAVES><<<grid, 64 * WAVES, 0, stream>>>(    \
                                  x, w, bias, static_cast<Y*>(y), M, N, K, row_blocks, tiles_per_slice, m_group, head_rows)))
#define WIDE_MB(MODE)                                   \
  switch (mb) {                                         \
    case 1:                                             \
      if (waves == 2) WIDE(MODE, 1, 2);                 \
      else WIDE(MODE, 1, 4);                            \
      break;                                            \
    case 2:                                             \
      if (waves == 2) WIDE(MODE, 2, 2);                 \
      else WIDE(MODE, 2, 4);                            \
      break;                                            \
    case 3: WIDE(MODE, 3, 4); break;                    \
    case 4: WIDE(MODE, 4, 4); break;                    \
    case 5: WIDE(MODE, 5, 4); break;                    \
    default: WIDE(MODE, 6, 4); break;                   \
  }
  if (mode == PK_GATED) {
    WIDE_MB(PK_GATED);
  } else if (mode == PK_ROTARY) {
    WIDE_MB(PK_ROTARY);
  } else {
    WIDE_MB(PK_PLAIN);
  }
#undef WIDE_MB
#undef WIDE
  return launch_status();
}

extern "C" int distie_gemm_packed_wide_bf16(const void* x, const void* w_packed, const float* bias, void* y,
                                            int y_dtype, int M, int N, int K, int gated, int pass_blocks,
                                            hipStream_t stream) {
  if (M <= 0) return 0;
  if (M > 256 || N <= 0 || K <= 0 || K % 8 != 0 || (gated && N % 2 != 0)) return DISTIE_BAD_ARGUMENT;
  return packed_wide_launch(static_cast<const bf16_t*>(x), static_cast<const bf16_t*>(w_packed), bias, y, y_dtype, M, N,
                            K, gated ? PK_GATED : PK_PLAIN, pass_blocks, stream);
}

// The stacked q/k/v product alone, on the ROTARY copy of its weight, for 17 rows of x and more against a weight large
// enough for the wide kernel: y as distie_gemm_packed_wide_bf16 writes it (columns in the weight's own order; float32
// [slices, M, N] when K is cut, distie_gemm_packed_wide_slices(N, K) says), bias on the first slice. Rotation and
// cache write are the caller's next kernel.
extern "C" int distie_gemm_packed_wide_qkv_bf16(const void* x, const void* w_packed, const float* bias, void* y,
                                                int y_dtype, int M, int K, int heads, int kv_heads, int dim,
                                                int pass_blocks, hipStream_t stream) {
  if (M <= 0) return 0;
  if (M > 256 || K <= 0 || K % 8 != 0 || heads < 1 || kv_heads < 1 || dim < 16 || dim % 16 != 0) return DISTIE_BAD_ARGUMENT;
  const int N = (heads + 2 * kv_heads) * dim;
  return packed_wide_launch(static_cast<const bf16_t*>(x), static_cast<const bf16_t*>(w_packed), bias, y, y_dtype, M, N,
                            K, PK_ROTARY, pass_blocks, stream, HeadRows{heads, kv_heads, dim});
}

// The stacked q/k/v product with the rotation and the cache write in its epilogue. w_packed: the ROTARY
// copy of the [(heads + 2 kv_heads) * dim, K] weight. y: bfloat16 [M, N], rotated. dim a multiple of 16;
// table: [M, dim / 2] (cos, sin). Up to 256 rows of x, in groups of 16: a workgroup owns one row block of
// one group, so that even this small weight is pulled by hundreds of workgroups.
extern "C" int distie_gemm_packed_rotary_bf16(const void* x, const void* w_packed, const float* bias, void* y,
                                              const void* table, const int32_t* slots, void* k_cache, void* v_cache,
                                              int M, int K, int heads, int kv_heads, int dim, int block_size,
                                              int write, hipStream_t stream) {
  if (M <= 0) return 0;
  if (M > 256 || K <= 0 || K % 8 != 0 || heads < 1 || kv_heads < 1 || dim < 16 || dim % 16 != 0 || block_size < 1 ||
      table == nullptr || (write && (slots == nullptr || k_cache == nullptr || v_cache == nullptr)))
    return DISTIE_BAD_ARGUMENT;
  const int N = (heads + 2 * kv_heads) * dim;
  const RotaryOut rotary = {static_cast<const float2*>(table), slots, static_cast<bf16_t*>(k_cache),
                            static_cast<bf16_t*>(v_cache), heads, kv_heads, dim, block_size, write};
  const bf16_t* xb = static_cast<const bf16_t*>(x);
  const bf16_t* wb = static_cast<const bf16_t*>(w_packed);
  bf16_t* out = static_cast<bf16_t*>(y);
  const int tiles = (K + 31) / 32;
  dim3 grid(N / 16, 1, (M + 15) / 16);
#define ROTARY(WAVES) \
  gemm_packed_kernel<bf16_t, PK_ROTARY, WAVES><<<grid, 64 * WAVES, 0, stream>>>(xb, wb, bias, out, M, N, K, tiles, rotary)
  switch (packed_waves(K)) {
    case 16: ROTARY(16); break;
    case 8: ROTARY(8); break;
    case 4: ROTARY(4); break;
    case 2: ROTARY(2); break;
    default: ROTARY(1); break;
  }
#undef ROTARY
  return launch_status();
}
