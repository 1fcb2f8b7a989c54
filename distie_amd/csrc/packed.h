// What the kernels on packed weight copies share: vector types of the matrix cores' operands, the tile of
// a packed copy, and the description of the q/k/v epilogue.
#pragma once

#include "common.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

#define PK_TILE 512         // elements of a tile: 16 rows x 32 k, in lane order
#define PK_PLAIN 0
#define PK_GATED 1
#define PK_ROTARY 2

struct RotaryOut {
  const float2* table;        // [M, D / 2] cosine and sine of each token's angles
  const int32_t* slots;       // [M] place of each token in the cache
  bf16_t* k_cache;            // [pages, kv_heads, block_size, D]
  bf16_t* v_cache;            // [pages, kv_heads, D, block_size]
  int heads, kv_heads, dim, block_size, write;
};

static __device__ __forceinline__ uint2 pack_bf16x4(const float v[4]) {
  uint32_t h[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) h[i] = __builtin_bit_cast(uint16_t, static_cast<bf16_t>(v[i]));
  return uint2{h[0] | (h[1] << 16), h[2] | (h[3] << 16)};
}
