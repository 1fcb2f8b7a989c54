// Choosing a token from a row of float32 logits.
//
//   argmax: the greedy pick of the reference (worker/src/inference/model_runner.py:124-126), lowest
//           index among equals.
//   sample: rows with temperature <= 0 are greedy; others draw once from softmax(logits / t)
//           (worker/src/inference/model_runner.py:127-129). The reference draws from a global
//           generator; here the uniform number is a hash of (seed, counter) of the request, so a run
//           can be repeated. The draw inverts the cumulative sum: the token is the first index whose
//           cumulative weight exceeds u * total.

#include "common.h"
#include "no_alloc.h"

#include <mutex>

#define SAMPLE_THREADS 256

struct Best {
  float value;
  int index;
};

__device__ __forceinline__ Best better(Best a, Best b) {
  if (b.value > a.value || (b.value == a.value && b.index < a.index)) return b;
  return a;
}

__device__ __forceinline__ Best block_best(Best mine, Best* scratch) {
#pragma unroll
  for (int o = DISTIE_WAVE / 2; o > 0; o >>= 1) {
    Best other{__shfl_xor(mine.value, o, DISTIE_WAVE), __shfl_xor(mine.index, o, DISTIE_WAVE)};
    mine = better(mine, other);
  }
  const int wave = threadIdx.x / DISTIE_WAVE;
  const int waves = blockDim.x / DISTIE_WAVE;
  __syncthreads();
  if (threadIdx.x % DISTIE_WAVE == 0) scratch[wave] = mine;
  __syncthreads();
  Best out = scratch[0];
  for (int w = 1; w < waves; ++w) out = better(out, scratch[w]);
  return out;
}

__device__ __forceinline__ Best row_best(const float* row, int vocab, Best* scratch) {
  Best mine{-INFINITY, 0x7fffffff};
  for (int i = threadIdx.x; i < vocab; i += blockDim.x) mine = better(mine, Best{row[i], i});
  Best out = block_best(mine, scratch);
  if (out.index >= vocab) out.index = 0;   // a row of NaN or -inf
  return out;
}

__global__ __launch_bounds__(SAMPLE_THREADS) void argmax_kernel(const float* __restrict__ logits,
                                                                int32_t* __restrict__ out, int vocab) {
  __shared__ Best scratch[SAMPLE_THREADS / DISTIE_WAVE];
  const Best best = row_best(logits + static_cast<int64_t>(blockIdx.x) * vocab, vocab, scratch);
  if (threadIdx.x == 0) out[blockIdx.x] = best.index;
}

// Large vocabularies: a row is cut into `parts` pieces (grid: parts x rows), each block writes the best of its
// piece, and a second launch takes the best of the pieces (lowest index among equals, as everywhere).
__global__ __launch_bounds__(SAMPLE_THREADS) void argmax_pieces_kernel(const float* __restrict__ logits,
                                                                       float* __restrict__ piece_value,
                                                                       int32_t* __restrict__ piece_index, int vocab,
                                                                       int piece_len, int by_four) {
  __shared__ Best scratch[SAMPLE_THREADS / DISTIE_WAVE];
  const float* row = logits + static_cast<int64_t>(blockIdx.y) * vocab;
  const int begin = blockIdx.x * piece_len;
  const int end = min(vocab, begin + piece_len);
  Best mine{-INFINITY, 0x7fffffff};
  if (by_four) {
    // pieces begin and end at multiples of four and the rows are 16-byte aligned: four logits a load
    // (64 rows of 151,936: 22.4 -> 10.2 us, 8 rows: 10.0 -> 5.0)
    for (int i = begin + 4 * static_cast<int>(threadIdx.x); i < end; i += 4 * static_cast<int>(blockDim.x)) {
      const float4 v = *reinterpret_cast<const float4*>(row + i);
      mine = better(mine, Best{v.x, i});
      mine = better(mine, Best{v.y, i + 1});
      mine = better(mine, Best{v.z, i + 2});
      mine = better(mine, Best{v.w, i + 3});
    }
  } else {
    for (int i = begin + threadIdx.x; i < end; i += blockDim.x) mine = better(mine, Best{row[i], i});
  }
  const Best best = block_best(mine, scratch);
  if (threadIdx.x == 0) {
    piece_value[blockIdx.y * gridDim.x + blockIdx.x] = best.value;
    piece_index[blockIdx.y * gridDim.x + blockIdx.x] = best.index;
  }
}

__global__ __launch_bounds__(DISTIE_WAVE) void argmax_combine_kernel(const float* __restrict__ piece_value,
                                                                     const int32_t* __restrict__ piece_index,
                                                                     int32_t* __restrict__ out, int parts, int vocab) {
  Best mine{-INFINITY, 0x7fffffff};
  for (int i = threadIdx.x; i < parts; i += DISTIE_WAVE)
    mine = better(mine, Best{piece_value[blockIdx.x * parts + i], piece_index[blockIdx.x * parts + i]});
#pragma unroll
  for (int o = DISTIE_WAVE / 2; o > 0; o >>= 1) {
    Best other{__shfl_xor(mine.value, o, DISTIE_WAVE), __shfl_xor(mine.index, o, DISTIE_WAVE)};
    mine = better(mine, other);
  }
  if (threadIdx.x == 0) out[blockIdx.x] = mine.index < vocab ? mine.index : 0;
}

// pieces a row is cut into (1 = the single-launch kernel); the caller sizes the scratch from it
extern "C" int distie_argmax_parts(int rows, int vocab) {
  if (vocab < 16384) return 1;
  int parts = 1024 / (rows < 1 ? 1 : rows);
  if (parts > vocab / 4096) parts = vocab / 4096;
  return parts < 2 ? 1 : (parts > 64 ? 64 : parts);
}

// scratch: float [rows * parts] and int32 [rows * parts]; may be null when distie_argmax_parts is 1
extern "C" int distie_argmax(const float* logits, int32_t* out, int rows, int vocab, float* piece_value,
                             int32_t* piece_index, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (vocab <= 0) return DISTIE_BAD_ARGUMENT;
  const int parts = distie_argmax_parts(rows, vocab);
  if (parts == 1) {
    argmax_kernel<<<rows, SAMPLE_THREADS, 0, stream>>>(logits, out, vocab);
    return launch_status();
  }
  if (piece_value == nullptr || piece_index == nullptr) return DISTIE_BAD_ARGUMENT;
  const int by_four = vocab % 4 == 0 && reinterpret_cast<uintptr_t>(logits) % 16 == 0;
  const int piece_len = by_four ? ((vocab / 4 + parts - 1) / parts) * 4 : (vocab + parts - 1) / parts;
  argmax_pieces_kernel<<<dim3(parts, rows), SAMPLE_THREADS, 0, stream>>>(logits, piece_value, piece_index, vocab, piece_len,
                                                                         by_four);
  argmax_combine_kernel<<<rows, DISTIE_WAVE, 0, stream>>>(piece_value, piece_index, out, parts, vocab);
  return launch_status();
}

// ---- the same pick with the scratch in a device array of this file (see no_alloc.h)
//
// In host code `scratch` is only a stand-in for the device array: its address on a device comes from
// hipGetSymbolAddress, once per device with that device current, and only that address is handed to kernels.
static __device__ __align__(256) unsigned char scratch[DISTIE_ARGMAX_STATIC_ENTRIES * (sizeof(float) + sizeof(int32_t))];

constexpr int STATIC_MAX_DEVICES = 64;
static void* scratch_of_device[STATIC_MAX_DEVICES];
static std::mutex scratch_lookup;

// -> 0 and the array's address on the current device, or a hipError_t. The address is looked up once per device;
// that lookup is no operation a capturing stream may see, so with `may_look_up` false (the caller's stream
// captures) a device whose address is not known yet is an error instead.
static int static_scratch(void** address, bool may_look_up) {
  int device = -1;
  hipError_t status = hipGetDevice(&device);
  if (status != hipSuccess) return static_cast<int>(status);
  if (device < 0 || device >= STATIC_MAX_DEVICES) return static_cast<int>(hipErrorInvalidDevice);
  std::lock_guard<std::mutex> hold(scratch_lookup);
  if (scratch_of_device[device] == nullptr) {
    if (!may_look_up) return static_cast<int>(hipErrorStreamCaptureUnsupported);
    void* found = nullptr;
    status = hipGetSymbolAddress(&found, HIP_SYMBOL(scratch));
    if (status != hipSuccess) return static_cast<int>(status);
    if (found == nullptr) return static_cast<int>(hipErrorInvalidSymbol);
    scratch_of_device[device] = found;
  }
  *address = scratch_of_device[device];
  return 0;
}

extern "C" int distie_argmax_static_prepare(void) {
  void* base = nullptr;
  return static_scratch(&base, true);
}

extern "C" void distie_argmax_static_limits(int* max_rows, int* max_entries) {
  if (max_rows != nullptr) *max_rows = DISTIE_ARGMAX_STATIC_MAX_ROWS;
  if (max_entries != nullptr) *max_entries = DISTIE_ARGMAX_STATIC_ENTRIES;
}

extern "C" int distie_argmax_static(const float* logits, int32_t* out, int rows, int vocab, hipStream_t stream) {
  if (rows < 0 || vocab <= 0 || (rows > 0 && (logits == nullptr || out == nullptr))) return DISTIE_BAD_ARGUMENT;
  if (rows == 0) return 0;
  if (rows > DISTIE_ARGMAX_STATIC_MAX_ROWS) return DISTIE_TOO_LARGE;
  const int parts = distie_argmax_parts(rows, vocab);
  if (parts == 1) {
    argmax_kernel<<<rows, SAMPLE_THREADS, 0, stream>>>(logits, out, vocab);
    return launch_status();
  }
  if (static_cast<int64_t>(rows) * parts > DISTIE_ARGMAX_STATIC_ENTRIES) return DISTIE_TOO_LARGE;
  hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &capturing) != hipSuccess) capturing = hipStreamCaptureStatusNone;
  void* base = nullptr;
  const int status = static_scratch(&base, capturing == hipStreamCaptureStatusNone);
  if (status != 0) return status;
  // every entry that the second launch reads is written by the first: nothing has to be cleared
  float* piece_value = static_cast<float*>(base);
  int32_t* piece_index = reinterpret_cast<int32_t*>(piece_value + DISTIE_ARGMAX_STATIC_ENTRIES);
  const int by_four = vocab % 4 == 0 && reinterpret_cast<uintptr_t>(logits) % 16 == 0;
  const int piece_len = by_four ? ((vocab / 4 + parts - 1) / parts) * 4 : (vocab + parts - 1) / parts;
  argmax_pieces_kernel<<<dim3(parts, rows), SAMPLE_THREADS, 0, stream>>>(logits, piece_value, piece_index, vocab, piece_len,
                                                                         by_four);
  argmax_combine_kernel<<<rows, DISTIE_WAVE, 0, stream>>>(piece_value, piece_index, out, parts, vocab);
  return launch_status();
}

// splitmix64 of (seed, counter) -> a float in [0, 1) with 24 random bits
__device__ __forceinline__ float uniform_of(uint64_t seed, uint64_t counter) {
  uint64_t z = seed * 0x9E3779B97F4A7C15ull + counter * 0xD1B54A32D192ED03ull + 0x94D049BB133111EBull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  z = z ^ (z >> 31);
  return static_cast<float>(z >> 40) * (1.0f / 16777216.0f);
}

__global__ __launch_bounds__(SAMPLE_THREADS) void sample_kernel(const float* __restrict__ logits,
                                                                const float* __restrict__ temperature,
                                                                const int64_t* __restrict__ seeds,
                                                                const int64_t* __restrict__ counters,
                                                                int32_t* __restrict__ out, int vocab) {
  __shared__ Best best_scratch[SAMPLE_THREADS / DISTIE_WAVE];
  __shared__ float sums[SAMPLE_THREADS];
  __shared__ float reduce_scratch[16];
  const float* row = logits + static_cast<int64_t>(blockIdx.x) * vocab;
  const Best best = row_best(row, vocab, best_scratch);
  const float t = temperature[blockIdx.x];
  if (!(t > 0.f)) {
    if (threadIdx.x == 0) out[blockIdx.x] = best.index;
    return;
  }
  // every thread owns a contiguous run of the vocabulary
  const int per = (vocab + SAMPLE_THREADS - 1) / SAMPLE_THREADS;
  const int begin = min(vocab, static_cast<int>(threadIdx.x) * per);
  const int end = min(vocab, begin + per);
  const float inv_t = 1.f / t;
  float mine = 0.f;
  for (int i = begin; i < end; ++i) mine += expf((row[i] - best.value) * inv_t);
  sums[threadIdx.x] = mine;
  const float total = block_sum(mine, reduce_scratch);
  __syncthreads();
  const float target = uniform_of(static_cast<uint64_t>(seeds[blockIdx.x]), static_cast<uint64_t>(counters[blockIdx.x])) * total;
  if (threadIdx.x == 0) {
    // find the run that holds the target, then the token inside it
    float before = 0.f;
    int owner = 0;
    for (; owner < SAMPLE_THREADS - 1; ++owner) {
      if (before + sums[owner] > target) break;
      before += sums[owner];
    }
    int b = min(vocab, owner * per), e = min(vocab, b + per);
    int pick = -1;
    float running = before;
    for (int i = b; i < e; ++i) {
      running += expf((row[i] - best.value) * inv_t);
      if (running > target) {
        pick = i;
        break;
      }
    }
    if (pick < 0) {
      // rounding left the target beyond the last run: take the last token with weight
      pick = best.index;
      for (int i = vocab - 1; i >= 0; --i)
        if (expf((row[i] - best.value) * inv_t) > 0.f) {
          pick = i;
          break;
        }
    }
    out[blockIdx.x] = pick;
  }
}

// Large vocabularies: one block per row walks 150,000 logits three times, alone (0.4 ms). As for argmax the row
// is cut into pieces (grid: parts x rows): a block writes its piece's best and, for rows that draw, the piece's
// sum of weights relative to that best. A second launch, one block per row, puts the pieces together (the
// row's best, every piece's sum rescaled to it, added in order), finds the piece in which the cumulative
// weight passes the target and walks that piece alone.
__global__ __launch_bounds__(SAMPLE_THREADS) void sample_pieces_kernel(const float* __restrict__ logits,
                                                                       const float* __restrict__ temperature,
                                                                       float* __restrict__ piece_value,
                                                                       int32_t* __restrict__ piece_index,
                                                                       float* __restrict__ piece_sum, int vocab,
                                                                       int piece_len) {
  __shared__ Best scratch[SAMPLE_THREADS / DISTIE_WAVE];
  __shared__ float reduce_scratch[16];
  const float* row = logits + static_cast<int64_t>(blockIdx.y) * vocab;
  const int begin = blockIdx.x * piece_len;
  const int end = min(vocab, begin + piece_len);
  Best mine{-INFINITY, 0x7fffffff};
  for (int i = begin + threadIdx.x; i < end; i += blockDim.x) mine = better(mine, Best{row[i], i});
  const Best best = block_best(mine, scratch);
  const float t = temperature[blockIdx.y];
  float sum = 0.f;
  if (t > 0.f && best.value > -INFINITY) {
    const float inv_t = 1.f / t;
    for (int i = begin + threadIdx.x; i < end; i += blockDim.x) sum += expf((row[i] - best.value) * inv_t);
    sum = block_sum(sum, reduce_scratch);
  }
  if (threadIdx.x == 0) {
    const int slot = blockIdx.y * gridDim.x + blockIdx.x;
    piece_value[slot] = best.value;
    piece_index[slot] = best.index;
    piece_sum[slot] = sum;
  }
}

constexpr int SAMPLE_MAX_PARTS = 64;

__global__ __launch_bounds__(SAMPLE_THREADS) void sample_pick_kernel(
    const float* __restrict__ logits, const float* __restrict__ temperature, const int64_t* __restrict__ seeds,
    const int64_t* __restrict__ counters, const float* __restrict__ piece_value,
    const int32_t* __restrict__ piece_index, const float* __restrict__ piece_sum, int32_t* __restrict__ out, int parts,
    int vocab, int piece_len) {
  __shared__ float scaled[SAMPLE_MAX_PARTS];
  __shared__ float sums[SAMPLE_THREADS];
  __shared__ float before_s, target_s;
  __shared__ int piece_s;
  const int tid = threadIdx.x;
  const int r = blockIdx.x;
  // every wave finds the row's best among the pieces for itself
  const int lane = tid % DISTIE_WAVE;
  Best best{-INFINITY, 0x7fffffff};
  if (lane < parts) best = Best{piece_value[r * parts + lane], piece_index[r * parts + lane]};
  const float own_value = best.value;
#pragma unroll
  for (int o = DISTIE_WAVE / 2; o > 0; o >>= 1) {
    Best other{__shfl_xor(best.value, o, DISTIE_WAVE), __shfl_xor(best.index, o, DISTIE_WAVE)};
    best = better(best, other);
  }
  if (best.index >= vocab) best.index = 0;           // a row of NaN or -inf
  const float t = temperature[r];
  if (!(t > 0.f) || !(best.value > -INFINITY)) {
    if (tid == 0) out[r] = best.index;
    return;
  }
  const float inv_t = 1.f / t;
  if (tid < parts) {
    const float s = piece_sum[r * parts + tid];
    scaled[tid] = s > 0.f ? s * expf((own_value - best.value) * inv_t) : 0.f;
  }
  __syncthreads();
  if (tid == 0) {
    float total = 0.f;
    for (int p = 0; p < parts; ++p) total += scaled[p];
    const float target = uniform_of(static_cast<uint64_t>(seeds[r]), static_cast<uint64_t>(counters[r])) * total;
    // the piece in which the cumulative weight passes the target; rounding may leave the target beyond the
    // last piece: then the last piece with weight
    float before = 0.f;
    int piece = -1, last = 0;
    for (int p = 0; p < parts; ++p) {
      if (!(scaled[p] > 0.f)) continue;
      last = p;
      if (before + scaled[p] > target) {
        piece = p;
        break;
      }
      before += scaled[p];
    }
    if (piece < 0) {
      piece = last;
      before -= scaled[last];
    }
    piece_s = piece;
    before_s = before;
    target_s = target;
  }
  __syncthreads();
  const float target = target_s;
  const int begin = piece_s * piece_len;
  const int end = min(vocab, begin + piece_len);
  const float* row = logits + static_cast<int64_t>(r) * vocab;
  // every thread owns a contiguous run of the piece
  const int per = (end - begin + SAMPLE_THREADS - 1) / SAMPLE_THREADS;
  const int mine_begin = min(end, begin + tid * per);
  const int mine_end = min(end, mine_begin + per);
  float mine = 0.f;
  for (int i = mine_begin; i < mine_end; ++i) mine += expf((row[i] - best.value) * inv_t);
  sums[tid] = mine;
  __syncthreads();
  if (tid == 0) {
    float running = before_s;
    int owner = 0;
    for (; owner < SAMPLE_THREADS - 1; ++owner) {
      if (running + sums[owner] > target) break;
      running += sums[owner];
    }
    const int b = min(end, begin + owner * per), e = min(end, b + per);
    int pick = -1;
    for (int i = b; i < e; ++i) {
      running += expf((row[i] - best.value) * inv_t);
      if (running > target) {
        pick = i;
        break;
      }
    }
    if (pick < 0) {
      // rounding left the target beyond the piece's end: its last token with weight
      pick = best.index;
      for (int i = end - 1; i >= begin; --i)
        if (expf((row[i] - best.value) * inv_t) > 0.f) {
          pick = i;
          break;
        }
    }
    out[r] = pick;
  }
}

// scratch: piece_value and piece_sum float [rows * parts], piece_index int32 [rows * parts], parts from
// distie_argmax_parts; may be null when that is 1
extern "C" int distie_sample(const float* logits, const float* temperature, const int64_t* seeds,
                             const int64_t* counters, int32_t* out, int rows, int vocab, float* piece_value,
                             int32_t* piece_index, float* piece_sum, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (vocab <= 0) return DISTIE_BAD_ARGUMENT;
  const int parts = distie_argmax_parts(rows, vocab);
  if (parts == 1) {
    sample_kernel<<<rows, SAMPLE_THREADS, 0, stream>>>(logits, temperature, seeds, counters, out, vocab);
    return launch_status();
  }
  if (piece_value == nullptr || piece_index == nullptr || piece_sum == nullptr || parts > SAMPLE_MAX_PARTS)
    return DISTIE_BAD_ARGUMENT;
  const int piece_len = (vocab + parts - 1) / parts;
  sample_pieces_kernel<<<dim3(parts, rows), SAMPLE_THREADS, 0, stream>>>(logits, temperature, piece_value, piece_index,
                                                                        piece_sum, vocab, piece_len);
  sample_pick_kernel<<<rows, SAMPLE_THREADS, 0, stream>>>(logits, temperature, seeds, counters, piece_value,
                                                          piece_index, piece_sum, out, parts, vocab, piece_len);
  return launch_status();
}
