// Large matrix products through hipBLASLt, with the plan of every shape kept: y[M, N] = x[M, K] . W[N, K]^T
// (+ bias), float32 sums, y with rows `ldy` elements apart. The operands are both bfloat16 (y in bfloat16 or
// float32) or both float32 (y in float32: products and sums in float32, the library's plain 32-bit compute type,
// no reduced-precision mode).
//
// The reference leaves these products to its library as well (torch.nn.functional.linear on cuBLAS:
// worker/src/inference/qwen2/model.py:60-75). Calling the library from here instead of through torch saves
// most of the host time of a call (descriptors and the choice of kernel are made once per shape), lets the
// output be a column block of a wider matrix, adds the bias in float32, and lets the engine time the library's
// candidate kernels itself for the shapes of a full portion.
//
// One device per process, one caller at a time (a mutex guards the table of plans). Outside the timing of
// candidates nothing here allocates device memory after `distie_lib_init`, so a call can be recorded into a graph
// once its shape has been seen.
#include "common.h"

#include <hipblaslt/hipblaslt.h>
#include <hipblaslt/hipblaslt-ext.hpp>

#include <cmath>
#include <mutex>
#include <unordered_map>
#include <vector>

#define DISTIE_LIB_UNSUPPORTED (-3)      // the library offers no kernel for this product: the caller takes another way
#define DISTIE_LIB_NOT_READY (-4)

namespace {

constexpr size_t WORKSPACE_BYTES = size_t(128) << 20;
constexpr int CANDIDATES = 16;           // of the library's own ranking, for a shape that is not timed
constexpr int TIMED_RUNS = 4;
constexpr size_t FLUSH_BYTES = size_t(384) << 20;      // more than the 256 MB of the memory-side cache
constexpr float WORTH_TIMING = 1.3f;     // a candidate whose first run takes this much longer than the best so far is dropped
constexpr size_t MAX_PLANS = 4096;       // beyond this many shapes the plans that were not timed are forgotten
constexpr int ROW_CLASS = 32;            // shapes that are not timed share the choice of kernel with the other row counts of their class

struct Key {
  int M, N, K, x_dtype, y_dtype, bias;
  int64_t ldy;
  bool operator==(const Key& o) const {
    return M == o.M && N == o.N && K == o.K && x_dtype == o.x_dtype && y_dtype == o.y_dtype && bias == o.bias && ldy == o.ldy;
  }
};
struct KeyHash {
  size_t operator()(const Key& k) const {
    uint64_t h = 1469598103934665603ull;
    for (uint64_t v : {uint64_t(k.M), uint64_t(k.N), uint64_t(k.K), uint64_t(k.x_dtype), uint64_t(k.y_dtype), uint64_t(k.bias), uint64_t(k.ldy)}) {
      h ^= v;
      h *= 1099511628211ull;
    }
    return size_t(h);
  }
};
struct Plan {
  hipblasLtMatmulDesc_t product = nullptr;
  hipblasLtMatrixLayout_t w = nullptr, x = nullptr, y = nullptr;
  hipblasLtMatmulAlgo_t algo;
  bool timed = false;
};

std::mutex guard;
hipblasLtHandle_t handle = nullptr;
void* workspace = nullptr;
int device_of_handle = -1;
std::unordered_map<Key, Plan, KeyHash> plans;
// the choice for a class of row counts (the key's M rounded up to ROW_CLASS): the library's first, or the kernel
// found by timing if a shape of the class was timed (the engine times the class's largest row count). A serving
// run meets a new row count in almost every step with a portion in it, and asking the library to rank its
// kernels costs more than the product of a short portion
std::unordered_map<Key, hipblasLtMatmulAlgo_t, KeyHash> class_choice;
std::unordered_map<Key, bool, KeyHash> class_timed;
long plans_made = 0, plans_timed = 0, choices_asked = 0, candidates_refused = 0;

bool ok(hipblasStatus_t s) { return s == HIPBLAS_STATUS_SUCCESS; }
hipDataType type_of(int dtype) { return dtype == DISTIE_F32 ? HIP_R_32F : HIP_R_16BF; }

void drop(Plan& p) {
  if (p.product) hipblasLtMatmulDescDestroy(p.product);
  if (p.w) hipblasLtMatrixLayoutDestroy(p.w);
  if (p.x) hipblasLtMatrixLayoutDestroy(p.x);
  if (p.y) hipblasLtMatrixLayoutDestroy(p.y);
  p = Plan();
}

// In the library's column-major terms: y^T [N x M, ld ldy] = W^T (stored K x N, ld K, transposed) . x^T (stored K x M, ld K).
int make_layouts(const Key& key, Plan& plan) {
  const hipDataType in_type = type_of(key.x_dtype), out_type = type_of(key.y_dtype);
  if (!ok(hipblasLtMatmulDescCreate(&plan.product, HIPBLAS_COMPUTE_32F, HIP_R_32F))) return DISTIE_LIB_UNSUPPORTED;
  const int32_t transposed = HIPBLAS_OP_T, plain = HIPBLAS_OP_N;
  bool fine = ok(hipblasLtMatmulDescSetAttribute(plan.product, HIPBLASLT_MATMUL_DESC_TRANSA, &transposed, sizeof(transposed))) &&
              ok(hipblasLtMatmulDescSetAttribute(plan.product, HIPBLASLT_MATMUL_DESC_TRANSB, &plain, sizeof(plain)));
  if (fine && key.bias) {
    const uint32_t epilogue = HIPBLASLT_EPILOGUE_BIAS;
    const int32_t bias_type = HIP_R_32F;
    fine = ok(hipblasLtMatmulDescSetAttribute(plan.product, HIPBLASLT_MATMUL_DESC_EPILOGUE, &epilogue, sizeof(epilogue))) &&
           ok(hipblasLtMatmulDescSetAttribute(plan.product, HIPBLASLT_MATMUL_DESC_BIAS_DATA_TYPE, &bias_type, sizeof(bias_type)));
  }
  fine = fine && ok(hipblasLtMatrixLayoutCreate(&plan.w, in_type, key.K, key.N, key.K)) &&
         ok(hipblasLtMatrixLayoutCreate(&plan.x, in_type, key.K, key.M, key.K)) &&
         ok(hipblasLtMatrixLayoutCreate(&plan.y, out_type, key.N, key.M, key.ldy));
  return fine ? 0 : DISTIE_LIB_UNSUPPORTED;
}

// the library's own ranking of its kernels for this product, best first
int ask_library(const Plan& plan, std::vector<hipblasLtMatmulHeuristicResult_t>& found) {
  hipblasLtMatmulPreference_t preference = nullptr;
  if (!ok(hipblasLtMatmulPreferenceCreate(&preference))) return DISTIE_LIB_UNSUPPORTED;
  const uint64_t room = WORKSPACE_BYTES;
  hipblasLtMatmulPreferenceSetAttribute(preference, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &room, sizeof(room));
  found.assign(CANDIDATES, hipblasLtMatmulHeuristicResult_t());
  int count = 0;
  const hipblasStatus_t s = hipblasLtMatmulAlgoGetHeuristic(handle, plan.product, plan.w, plan.x, plan.y, plan.y, preference,
                                                            CANDIDATES, found.data(), &count);
  hipblasLtMatmulPreferenceDestroy(preference);
  ++choices_asked;
  if (!ok(s) || count <= 0) return DISTIE_LIB_UNSUPPORTED;
  found.resize(count);
  return 0;
}

bool takes(const Plan& plan, hipblasLtMatmulAlgo_t& algo) {
  const float one = 1.f, zero = 0.f;
  size_t needs = 0;
  return ok(hipblaslt_ext::matmulIsAlgoSupported(handle, plan.product, &one, plan.w, plan.x, &zero, plan.y, plan.y, algo, needs)) &&
         needs <= WORKSPACE_BYTES;
}

hipblasStatus_t run(const Plan& plan, const hipblasLtMatmulAlgo_t& algo, const void* x, const void* w, const void* bias,
                    void* y, hipStream_t stream) {
  const float one = 1.f, zero = 0.f;
  if (bias != nullptr &&
      !ok(hipblasLtMatmulDescSetAttribute(plan.product, HIPBLASLT_MATMUL_DESC_BIAS_POINTER, &bias, sizeof(bias))))
    return HIPBLAS_STATUS_INVALID_VALUE;
  return hipblasLtMatmul(handle, plan.product, &one, w, plan.w, x, plan.x, &zero, y, plan.y, y, plan.y, &algo, workspace,
                         WORKSPACE_BYTES, stream);
}

// largest |got - want| and largest |want| over rows x columns (rows `ld` apart), as the bit patterns of the
// (non-negative) floats, which order as the floats do; a NaN anywhere makes the difference infinite
template <typename T>
__global__ void compare_kernel(const T* __restrict__ got, const T* __restrict__ want, int rows, int columns, int64_t ld,
                               uint32_t* __restrict__ worst) {
  float diff = 0.f, size = 0.f;
  for (int64_t i = blockIdx.x * int64_t(blockDim.x) + threadIdx.x; i < int64_t(rows) * columns; i += int64_t(gridDim.x) * blockDim.x) {
    const int64_t at = i / columns * ld + i % columns;
    const float g = to_float(got[at]), w = to_float(want[at]);
    const float d = fabsf(g - w);
    diff = (d == d) ? fmaxf(diff, d) : INFINITY;
    size = fmaxf(size, fabsf(w));
  }
  atomicMax(&worst[0], __float_as_uint(diff));
  atomicMax(&worst[1], __float_as_uint(size));
}

// What the timing of candidates needs beyond the product's own buffers, freed on every way out.
struct Bench {
  hipEvent_t begin = nullptr, end = nullptr;
  void* flush = nullptr;          // overwritten before every timed run: larger than the memory-side cache
  void* reference = nullptr;      // the result of the library's first choice
  uint32_t* worst = nullptr;
  ~Bench() {
    if (begin) hipEventDestroy(begin);
    if (end) hipEventDestroy(end);
    if (flush) hipFree(flush);
    if (reference) hipFree(reference);
    if (worst) hipFree(worst);
  }
};

// Time every kernel of the library that takes the product and keep the fastest whose result agrees with that of
// the library's own first choice. -> 0, or a status
int choose_by_timing(Plan& plan, const Key& key, const std::vector<hipblasLtMatmulHeuristicResult_t>& found, const void* x,
                     const void* w, const void* bias, void* y, hipStream_t stream) {
  // every kernel that takes this product, not only the first of the library's ranking (which is made for speed
  // of choice: at 2,048 x 37,888 x 3,584 the best of all kernels is 10 % faster than the best of the first 16)
  std::vector<hipblasLtMatmulAlgo_t> candidates;
  for (const auto& r : found) candidates.push_back(r.algo);
  {
    const hipDataType in_type = type_of(key.x_dtype), out_type = type_of(key.y_dtype);
    std::vector<hipblasLtMatmulHeuristicResult_t> all;
    if (ok(hipblaslt_ext::getAllAlgos(handle, hipblaslt_ext::GemmType::HIPBLASLT_GEMM, HIPBLAS_OP_T, HIPBLAS_OP_N,
                                      in_type, in_type, out_type, out_type, HIPBLAS_COMPUTE_32F, all)))
      for (auto& r : all)
        if (takes(plan, r.algo)) candidates.push_back(r.algo);
  }
  Bench bench;
  const size_t element = key.y_dtype == DISTIE_F32 ? 4 : 2;
  const size_t y_bytes = (size_t(key.M - 1) * key.ldy + key.N) * element;
  if (hipEventCreate(&bench.begin) != hipSuccess || hipEventCreate(&bench.end) != hipSuccess ||
      hipMalloc(&bench.reference, y_bytes) != hipSuccess || hipMalloc(reinterpret_cast<void**>(&bench.worst), 8) != hipSuccess)
    return DISTIE_LIB_NOT_READY;
  // Every timed run starts on cold caches, as the product will between its neighbours in a step. Timed back to
  // back on warm weights, the choice was less stable from run to run and no better (2,048-token prefill of the
  // 1.5B shape on one box: 9.39 and 10.0 ms warm, 9.36 and 9.22 cold; the library's own first 16 warm: 9.36).
  if (hipMalloc(&bench.flush, FLUSH_BYTES) != hipSuccess) bench.flush = nullptr;
  // The kernels beyond the library's ranking are not ones it would have picked itself: a candidate counts only
  // if its result is the first choice's up to rounding (sums in another order: an output rounded to bfloat16
  // may move by one step of its 8 bits, a float32 output by far less).
  if (!ok(run(plan, found[0].algo, x, w, bias, y, stream)) ||
      hipMemcpyAsync(bench.reference, y, y_bytes, hipMemcpyDeviceToDevice, stream) != hipSuccess ||
      hipStreamSynchronize(stream) != hipSuccess)
    return DISTIE_LIB_UNSUPPORTED;
  const float allowed = key.y_dtype == DISTIE_BF16 ? 1.f / 64 : (key.x_dtype == DISTIE_BF16 ? 1e-4f : 1e-5f);
  auto agrees = [&]() {
    if (hipMemsetAsync(bench.worst, 0, 8, stream) != hipSuccess) return false;
    if (key.y_dtype == DISTIE_F32)
      compare_kernel<float><<<256, 256, 0, stream>>>(static_cast<const float*>(y), static_cast<const float*>(bench.reference),
                                                     key.M, key.N, key.ldy, bench.worst);
    else
      compare_kernel<bf16_t><<<256, 256, 0, stream>>>(static_cast<const bf16_t*>(y), static_cast<const bf16_t*>(bench.reference),
                                                      key.M, key.N, key.ldy, bench.worst);
    float host[2] = {INFINITY, 0.f};
    if (hipMemcpyAsync(host, bench.worst, 8, hipMemcpyDeviceToHost, stream) != hipSuccess ||
        hipStreamSynchronize(stream) != hipSuccess)
      return false;
    return host[0] <= allowed * host[1];
  };
  auto timed = [&](const hipblasLtMatmulAlgo_t& algo, int runs, float& ms) {
    ms = 0.f;
    for (int r = 0; r < runs; ++r) {
      if (bench.flush != nullptr && hipMemsetAsync(bench.flush, r, FLUSH_BYTES, stream) != hipSuccess) return false;
      hipEventRecord(bench.begin, stream);
      const bool ran = ok(run(plan, algo, x, w, bias, y, stream));
      hipEventRecord(bench.end, stream);
      if (hipEventSynchronize(bench.end) != hipSuccess || !ran) return false;
      float one_run = 0.f;
      hipEventElapsedTime(&one_run, bench.begin, bench.end);
      ms += one_run / runs;
    }
    return true;
  };
  float best = -1.f;
  for (const auto& candidate : candidates) {
    float once = 0.f, ms = 0.f;
    if (!timed(candidate, 1, once)) continue;                               // a warm-up, and the run that is checked
    if (!agrees()) {
      ++candidates_refused;
      continue;
    }
    if (best > 0.f && once > WORTH_TIMING * best) continue;
    if (!timed(candidate, TIMED_RUNS, ms)) continue;
    if (best < 0.f || ms < best) {
      best = ms;
      plan.algo = candidate;
    }
  }
  return best < 0.f ? DISTIE_LIB_UNSUPPORTED : 0;
}

}  // namespace

// Once per process, with the device current: the library's handle and its workspace (128 MiB, kept until the
// process ends).
extern "C" int distie_lib_init(int device) {
  std::lock_guard<std::mutex> lock(guard);
  if (handle != nullptr) return device == device_of_handle ? 0 : DISTIE_BAD_ARGUMENT;
  hipError_t e = hipSetDevice(device);
  if (e != hipSuccess) return static_cast<int>(e);
  if (!ok(hipblasLtCreate(&handle))) {
    handle = nullptr;
    return DISTIE_LIB_NOT_READY;
  }
  e = hipMalloc(&workspace, WORKSPACE_BYTES);
  if (e != hipSuccess) {
    hipblasLtDestroy(handle);
    handle = nullptr;
    return static_cast<int>(e);
  }
  device_of_handle = device;
  return 0;
}

// plans made, and plans whose kernel was chosen by timing
extern "C" void distie_lib_counts(long* made, long* timed) {
  std::lock_guard<std::mutex> lock(guard);
  *made = plans_made;
  *timed = plans_timed;
}

// plans held now, times the library was asked to rank its kernels, timed candidates refused for a result that
// differed from the library's first choice
extern "C" void distie_lib_more_counts(long* held, long* asked, long* refused) {
  std::lock_guard<std::mutex> lock(guard);
  *held = static_cast<long>(plans.size());
  *asked = choices_asked;
  *refused = candidates_refused;
}

// y = x . W^T (+ bias). `x_dtype`: of x and W, `y_dtype`: of y. `bias`: float32 [N] or null. `tune` != 0: a shape not yet
// timed has every kernel of the library that takes it run on `stream` (which is waited for: not inside a capture) and
// keeps the fastest whose result agrees with that of the library's first choice (y is written by every candidate
// run, each time with the whole result). Which kernel wins can differ from process to process when two are about
// equally fast, and with it the rounding of a bfloat16 result: an engine that must repeat bit for bit leaves `tune`
// off. A shape that is not timed takes the library's first choice for its class of row counts (M rounded up to 32).
extern "C" int distie_lib_linear(const void* x, const void* w, const void* bias, void* y, int x_dtype, int y_dtype, int M,
                                 int N, int K, int64_t ldy, int tune, hipStream_t stream) {
  if (M < 1 || N < 1 || K < 1 || ldy < N || (y_dtype != DISTIE_F32 && y_dtype != DISTIE_BF16) ||
      (x_dtype != DISTIE_F32 && x_dtype != DISTIE_BF16) || (x_dtype == DISTIE_F32 && y_dtype != DISTIE_F32) ||
      x == nullptr || w == nullptr || y == nullptr)
    return DISTIE_BAD_ARGUMENT;
  std::lock_guard<std::mutex> lock(guard);
  if (handle == nullptr) return DISTIE_LIB_NOT_READY;
  const Key key{M, N, K, x_dtype, y_dtype, bias != nullptr ? 1 : 0, ldy};
  auto it = plans.find(key);
  if (it == plans.end() || (tune && !it->second.timed)) {
    if (it == plans.end()) {
      if (plans.size() >= MAX_PLANS) {
        // a long run with ever new row counts: forget the plans that cost nothing to make again
        for (auto p = plans.begin(); p != plans.end();) {
          if (p->second.timed) {
            ++p;
          } else {
            drop(p->second);
            p = plans.erase(p);
          }
        }
      }
      Plan fresh;
      const int made = make_layouts(key, fresh);
      if (made != 0) {
        drop(fresh);
        return made;
      }
      it = plans.emplace(key, fresh).first;
      ++plans_made;
    }
    Plan& plan = it->second;
    Key of_class = key;
    of_class.M = (M + ROW_CLASS - 1) / ROW_CLASS * ROW_CLASS;
    auto known = class_choice.find(of_class);
    std::vector<hipblasLtMatmulHeuristicResult_t> found;
    if (!tune && known != class_choice.end() && takes(plan, known->second)) {
      plan.algo = known->second;
    } else {
      const int asked = ask_library(plan, found);
      if (asked != 0) {
        drop(plan);
        plans.erase(it);
        return asked;
      }
      plan.algo = found[0].algo;
      if (class_timed.find(of_class) == class_timed.end()) class_choice[of_class] = plan.algo;
    }
    if (tune) {
      const int chosen = choose_by_timing(plan, key, found, x, w, bias, y, stream);
      if (chosen != 0) return chosen;
      plan.timed = true;
      ++plans_timed;
      class_choice[of_class] = plan.algo;
      class_timed[of_class] = true;
    }
  }
  const hipblasStatus_t s = run(it->second, it->second.algo, x, w, bias, y, stream);
  if (!ok(s)) return DISTIE_LIB_UNSUPPORTED;
  return launch_status();
}
