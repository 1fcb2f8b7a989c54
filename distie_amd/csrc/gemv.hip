// Weight-streaming products on the vector ALU for few rows of x: y[M, N] = x[M, K] * W[N, K]^T (+ bias), any mix
// of float32 and bfloat16 for x, W and y, products and sums in float32 FMAs. This is the decode product of
// the true 32-bit path (no matrix-core mode) and of weights that a file keeps in 32-bit; gemm_generic's
// 64 x 64 tiles spend 7/8 of their work on padding at 8 rows and leave most of the chip idle.
//
// A workgroup of four waves owns four rows of W (several such groups, one after the other, when the rows are
// short enough for a thread's share of x to stay in registers); its waves take the pieces of a row in turn
// (wave w the pieces w, w + 4, ...), so every load of a wave reads 1 KB of a row in one run. A lane keeps the
// sums of its pieces for 4 rows of W x MB rows of x; they meet across the lanes by halving exchanges and
// across the waves in LDS, always in the same order: the result does not depend on timing or on what else
// is in the batch. More than eight rows of x are taken eight at a time (blockIdx.y), which reads W again;
// the later readings mostly come from the caches.
//
// The reference leaves these products to a library (worker/src/inference/qwen2/model.py:149-152, 231-233).

#include "common.h"

namespace {

constexpr int GV_ROWS = 4;       // rows of W a workgroup owns
constexpr int GV_WAVES = 4;
constexpr int GV_STRIDE = 68;    // floats between the rows of a wave's patch of LDS (64 lanes, 16-byte reads, banks spread)

// eight consecutive elements as floats
__device__ __forceinline__ void load8(const float* p, float v[8]) {
  const float4 a = *reinterpret_cast<const float4*>(p);
  const float4 b = *reinterpret_cast<const float4*>(p + 4);
  v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}
__device__ __forceinline__ void load8(const bf16_t* p, float v[8]) {
  const uint4 raw = *reinterpret_cast<const uint4*>(p);
  const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    v[2 * e] = __uint_as_float(w[e] << 16);
    v[2 * e + 1] = __uint_as_float(w[e] & 0xffff0000u);
  }
}

// Long rows: a workgroup owns ROWS rows of W and walks their pieces; x is read again for every piece (from the
// caches: it is small), so more rows a workgroup mean less of that traffic per byte of W.
template <typename WT, typename XT, typename YT, int MB, int ROWS>
__global__ __launch_bounds__(64 * GV_WAVES) void gemv_rows_kernel(const XT* __restrict__ x, const WT* __restrict__ w,
                                                                  const float* __restrict__ bias, YT* __restrict__ y,
                                                                  int M, int N, int K) {
  constexpr int COUNT = ROWS * MB;
  __shared__ __attribute__((aligned(16))) float rows_lds[GV_WAVES][COUNT * GV_STRIDE];
  __shared__ float part[GV_WAVES][COUNT];
  const int lane = threadIdx.x % 64;
  const int wave = threadIdx.x / 64;
  const int64_t n0 = static_cast<int64_t>(blockIdx.x) * ROWS;
  const int m0 = blockIdx.y * 8;
  const int rows_here = min(MB, M - m0);
  const WT* wrow[ROWS];
#pragma unroll
  for (int i = 0; i < ROWS; ++i) wrow[i] = w + min(n0 + i, static_cast<int64_t>(N) - 1) * K;
  const XT* xrow[MB];
#pragma unroll
  for (int m = 0; m < MB; ++m) xrow[m] = x + static_cast<int64_t>(min(m0 + m, M - 1)) * K;

  float acc[COUNT];
#pragma unroll
  for (int j = 0; j < COUNT; ++j) acc[j] = 0.f;

  // pieces of 8 elements; piece p belongs to wave (p / 64) % 4, lane p % 64
  const int pieces = K / 8;
  for (int p = wave * 64 + lane; p < pieces; p += 64 * GV_WAVES) {
    float wv[ROWS][8];
#pragma unroll
    for (int i = 0; i < ROWS; ++i) load8(wrow[i] + 8 * p, wv[i]);
#pragma unroll
    for (int m = 0; m < MB; ++m) {
      float xv[8];
      load8(xrow[m] + 8 * p, xv);
#pragma unroll
      for (int i = 0; i < ROWS; ++i)
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[i * MB + m] = fmaf(wv[i][e], xv[e], acc[i * MB + m]);
    }
  }

  // across the lanes through the wave's own patch of LDS (sum j of every lane into row j, lane j adds up row
  // j), then across the waves, always in the same order
  float* rows = rows_lds[wave];
#pragma unroll
  for (int j = 0; j < COUNT; ++j) rows[j * GV_STRIDE + lane] = acc[j];
  __builtin_amdgcn_wave_barrier();
  if (lane < COUNT) {
    float sum = 0.f;
#pragma unroll
    for (int q = 0; q < 64; q += 4) {
      const float4 four = *reinterpret_cast<const float4*>(rows + lane * GV_STRIDE + q);
      sum += (four.x + four.y) + (four.z + four.w);
    }
    part[wave][lane] = sum;
  }
  __syncthreads();
  if (threadIdx.x < COUNT) {
    const int i = threadIdx.x / MB, m = threadIdx.x % MB;
    float sum = 0.f;
#pragma unroll
    for (int wv = 0; wv < GV_WAVES; ++wv) sum += part[wv][threadIdx.x];
    const int64_t n = n0 + i;
    if (n < N && m < rows_here) {
      if (bias != nullptr) sum += bias[n];
      y[static_cast<int64_t>(m0 + m) * N + n] = from_float<YT>(sum);
    }
  }
}

// Rows of at most 2,048 PP elements: a thread owns the same PP pieces of every row, so its share of x stays in
// registers while the workgroup walks RG groups of four rows of W (the next group's weights are asked for
// before the current group is multiplied). The sums of all groups meet in LDS behind one barrier.
template <typename WT, typename XT, typename YT, int MB, int PP>
__global__ __launch_bounds__(64 * GV_WAVES) void gemv_rows_regx_kernel(const XT* __restrict__ x, const WT* __restrict__ w,
                                                                       const float* __restrict__ bias, YT* __restrict__ y,
                                                                       int M, int N, int K, int groups) {
  constexpr int COUNT = GV_ROWS * MB;
  extern __shared__ __attribute__((aligned(16))) float dynamic_lds[];
  float* reduce_all = dynamic_lds;                                     // [GV_WAVES][COUNT][GV_STRIDE]
  float* part_all = dynamic_lds + GV_WAVES * COUNT * GV_STRIDE;        // [groups][GV_WAVES][COUNT]
  const int lane = threadIdx.x % 64;
  const int wave = threadIdx.x / 64;
  const int m0 = blockIdx.y * 8;
  const int rows_here = min(MB, M - m0);
  const int pieces = K / 8;
  int piece[PP];
  bool has[PP];
#pragma unroll
  for (int u = 0; u < PP; ++u) {
    piece[u] = threadIdx.x + 64 * GV_WAVES * u;
    has[u] = piece[u] < pieces;
    piece[u] = min(piece[u], pieces - 1);
  }
  float xv[PP][MB][8];
#pragma unroll
  for (int u = 0; u < PP; ++u)
#pragma unroll
    for (int m = 0; m < MB; ++m) {
      load8(x + static_cast<int64_t>(min(m0 + m, M - 1)) * K + 8 * piece[u], xv[u][m]);
      if (!has[u]) {
#pragma unroll
        for (int e = 0; e < 8; ++e) xv[u][m][e] = 0.f;
      }
    }
  const int64_t first_row = static_cast<int64_t>(blockIdx.x) * groups * GV_ROWS;
  auto fetch = [&](float (&wv)[PP][GV_ROWS][8], int group) {
#pragma unroll
    for (int u = 0; u < PP; ++u)
#pragma unroll
      for (int i = 0; i < GV_ROWS; ++i) {
        const int64_t n = min(first_row + static_cast<int64_t>(group) * GV_ROWS + i, static_cast<int64_t>(N) - 1);
        load8(w + n * K + 8 * piece[u], wv[u][i]);
      }
  };
  auto work = [&](float (&wv)[PP][GV_ROWS][8], int group) {
    float v[COUNT];
#pragma unroll
    for (int j = 0; j < COUNT; ++j) v[j] = 0.f;
#pragma unroll
    for (int u = 0; u < PP; ++u)
#pragma unroll
      for (int i = 0; i < GV_ROWS; ++i)
#pragma unroll
        for (int m = 0; m < MB; ++m)
#pragma unroll
          for (int e = 0; e < 8; ++e) v[i * MB + m] = fmaf(wv[u][i][e], xv[u][m][e], v[i * MB + m]);
    // The COUNT sums of the 64 lanes meet through the wave's own patch of LDS: sum j of every lane goes into
    // row j, then lane j adds up row j (exchanges between lanes, sum by sum, cost four times the products).
    float* rows = reduce_all + wave * (COUNT * GV_STRIDE);
    __builtin_amdgcn_wave_barrier();            // the reads of the group before are done (the wave's LDS traffic is in order)
#pragma unroll
    for (int j = 0; j < COUNT; ++j) rows[j * GV_STRIDE + lane] = v[j];
    __builtin_amdgcn_wave_barrier();
    if (lane < COUNT) {
      float sum = 0.f;
#pragma unroll
      for (int q = 0; q < 64; q += 4) {
        const float4 four = *reinterpret_cast<const float4*>(rows + lane * GV_STRIDE + q);
        sum += (four.x + four.y) + (four.z + four.w);
      }
      part_all[(group * GV_WAVES + wave) * COUNT + lane] = sum;
    }
  };
  float w0[PP][GV_ROWS][8], w1[PP][GV_ROWS][8];
  fetch(w0, 0);
  for (int group = 0; group < groups; group += 2) {
    if (group + 1 < groups) fetch(w1, group + 1);
    work(w0, group);
    if (group + 1 >= groups) break;
    if (group + 2 < groups) fetch(w0, group + 2);
    work(w1, group + 1);
  }
  __syncthreads();
  for (int o = threadIdx.x; o < groups * COUNT; o += 64 * GV_WAVES) {
    const int group = o / COUNT, j = o % COUNT;
    const int i = j / MB, m = j % MB;
    float sum = 0.f;
#pragma unroll
    for (int wv = 0; wv < GV_WAVES; ++wv) sum += part_all[(group * GV_WAVES + wv) * COUNT + j];
    const int64_t n = first_row + static_cast<int64_t>(group) * GV_ROWS + i;
    if (n < N && m < rows_here) {
      if (bias != nullptr) sum += bias[n];
      y[static_cast<int64_t>(m0 + m) * N + n] = from_float<YT>(sum);
    }
  }
}

template <typename WT, typename XT, typename YT, int MB>
int launch_regx(const XT* x, const WT* w, const float* bias, YT* y, int M, int N, int K, hipStream_t stream) {
  // groups of four rows a workgroup: enough workgroups to fill the chip twice, at most 16 groups
  int groups = N / (GV_ROWS * 512);
  groups = groups < 1 ? 1 : (groups > 16 ? 16 : groups);
  const int per_block = groups * GV_ROWS;
  dim3 grid((N + per_block - 1) / per_block, (M + 7) / 8);
  const size_t lds = (static_cast<size_t>(groups) + GV_STRIDE) * GV_WAVES * GV_ROWS * MB * sizeof(float);
  if (K / 8 <= 64 * GV_WAVES) {
    gemv_rows_regx_kernel<WT, XT, YT, MB, 1><<<grid, 64 * GV_WAVES, lds, stream>>>(x, w, bias, y, M, N, K, groups);
  } else {
    gemv_rows_regx_kernel<WT, XT, YT, MB, 2><<<grid, 64 * GV_WAVES, lds, stream>>>(x, w, bias, y, M, N, K, groups);
  }
  return launch_status();
}

template <typename WT, typename XT, typename YT>
int launch_rows(const XT* x, const WT* w, const float* bias, YT* y, int M, int N, int K, hipStream_t stream) {
  const int mb = M >= 5 ? 8 : (M >= 3 ? 4 : M);
  if (K / 8 <= 2 * 64 * GV_WAVES) {            // short rows: x stays in registers
    switch (mb) {
      case 1: return launch_regx<WT, XT, YT, 1>(x, w, bias, y, M, N, K, stream);
      case 2: return launch_regx<WT, XT, YT, 2>(x, w, bias, y, M, N, K, stream);
      case 4: return launch_regx<WT, XT, YT, 4>(x, w, bias, y, M, N, K, stream);
      default: return launch_regx<WT, XT, YT, 8>(x, w, bias, y, M, N, K, stream);
    }
  }
  // eight rows a workgroup where that still leaves a workgroup for every compute unit
  const int rows = N >= 8 * 256 / 2 ? 8 : 4;
  dim3 grid((N + rows - 1) / rows, (M + 7) / 8);
#define ROWS_KERNEL(MB)                                                                                            \
  if (rows == 8) gemv_rows_kernel<WT, XT, YT, MB, 8><<<grid, 64 * GV_WAVES, 0, stream>>>(x, w, bias, y, M, N, K);   \
  else gemv_rows_kernel<WT, XT, YT, MB, 4><<<grid, 64 * GV_WAVES, 0, stream>>>(x, w, bias, y, M, N, K)
  switch (mb) {
    case 1: ROWS_KERNEL(1); break;
    case 2: ROWS_KERNEL(2); break;
    case 4: ROWS_KERNEL(4); break;
    default: ROWS_KERNEL(8); break;
  }
#undef ROWS_KERNEL
  return launch_status();
}

}  // namespace

// y[M, N] = x[M, K] * W[N, K]^T (+ bias[N]) for M <= 64 and K a multiple of 8; dtypes as in distie_gemm_generic.
extern "C" int distie_gemv_rows(const void* x, int x_dtype, const void* w, int w_dtype, const float* bias, void* y,
                                int y_dtype, int M, int N, int K, hipStream_t stream) {
  if (M <= 0) return 0;
  if (M > 64 || N <= 0 || K <= 0 || K % 8 != 0) return DISTIE_BAD_ARGUMENT;
  DISTIE_DISPATCH(x_dtype, X, DISTIE_DISPATCH(w_dtype, W, DISTIE_DISPATCH(y_dtype, Y, return launch_rows<W, X, Y>(
      static_cast<const X*>(x), static_cast<const W*>(w), bias, static_cast<Y*>(y), M, N, K, stream))));
  return DISTIE_BAD_ARGUMENT;
}
