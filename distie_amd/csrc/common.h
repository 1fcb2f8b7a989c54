// Shared helpers of the HIP kernels (gfx950, 64-wide wavefronts).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

typedef __bf16 bf16_t;

// dtype codes of the C interface
#define DISTIE_F32 0
#define DISTIE_BF16 1

// status codes of the C interface: 0 = launched; >0 = hipError_t; <0 = refused (bad argument)
#define DISTIE_BAD_ARGUMENT (-1)

#define DISTIE_WAVE 64

__device__ __forceinline__ float to_float(float x) { return x; }
__device__ __forceinline__ float to_float(bf16_t x) { return static_cast<float>(x); }

template <typename T>
__device__ __forceinline__ T from_float(float x);
template <>
__device__ __forceinline__ float from_float<float>(float x) { return x; }
template <>
__device__ __forceinline__ bf16_t from_float<bf16_t>(float x) { return static_cast<bf16_t>(x); }  // round to nearest even

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = DISTIE_WAVE / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, DISTIE_WAVE);
  return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = DISTIE_WAVE / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, DISTIE_WAVE));
  return v;
}

// Sum over a block of up to 1024 threads; `scratch` holds one float per wave (16).
// The order of the additions depends only on the block size, never on the data's place in a batch.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  v = wave_sum(v);
  const int wave = threadIdx.x / DISTIE_WAVE;
  const int lane = threadIdx.x % DISTIE_WAVE;
  const int waves = (blockDim.x + DISTIE_WAVE - 1) / DISTIE_WAVE;
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = 0.f;
  for (int w = 0; w < waves; ++w) total += scratch[w];
  return total;
}

// Sum of `slices` values that lie `stride` elements apart, added in order. The loads of four slices are
// issued together (the last group re-reads the last slice where it has fewer than four and does not add
// it), so the sum costs a few memory round trips instead of one per slice.
template <typename T>
__device__ __forceinline__ float sum_strided(const T* p, int slices, int64_t stride) {
  float sum = 0.f;
  for (int s = 0; s < slices; s += 4) {
    const int last = slices - 1;
    const float a = to_float(p[s * stride]);
    const float b = to_float(p[min(s + 1, last) * stride]);
    const float c = to_float(p[min(s + 2, last) * stride]);
    const float d = to_float(p[min(s + 3, last) * stride]);
    sum += a;
    if (s + 1 <= last) sum += b;
    if (s + 2 <= last) sum += c;
    if (s + 3 <= last) sum += d;
  }
  return sum;
}

static inline int launch_status() { return static_cast<int>(hipGetLastError()); }

// Calls `body` with a value of the element type that `code` names.
#define DISTIE_DISPATCH(code, T, ...)                 \
  do {                                                \
    if ((code) == DISTIE_F32) {                       \
      using T = float;                                \
      __VA_ARGS__;                                    \
    } else if ((code) == DISTIE_BF16) {               \
      using T = bf16_t;                               \
      __VA_ARGS__;                                    \
    } else {                                          \
      return DISTIE_BAD_ARGUMENT;                     \
    }                                                 \
  } while (0)
