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
long plans_made = 0, plans_timed = 0;

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
int make_plan(const Key& key, Plan& plan, std::vector<hipblasLtMatmulHeuristicResult_t>& found) {
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
  if (!fine) return DISTIE_LIB_UNSUPPORTED;
  hipblasLtMatmulPreference_t preference = nullptr;
  if (!ok(hipblasLtMatmulPreferenceCreate(&preference))) return DISTIE_LIB_UNSUPPORTED;
  const uint64_t room = WORKSPACE_BYTES;
  hipblasLtMatmulPreferenceSetAttribute(preference, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &room, sizeof(room));
  found.assign(CANDIDATES, hipblasLtMatmulHeuristicResult_t());
  int count = 0;
  const hipblasStatus_t s = hipblasLtMatmulAlgoGetHeuristic(handle, plan.product, plan.w, plan.x, plan.y, plan.y, preference,
                                                            CANDIDATES, found.data(), &count);
  hipblasLtMatmulPreferenceDestroy(preference);
  if (!ok(s) || count <= 0) return DISTIE_LIB_UNSUPPORTED;
  found.resize(count);
  plan.algo = found[0].algo;
  return 0;
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

// y = x . W^T (+ bias). `x_dtype`: of x and W, `y_dtype`: of y. `bias`: float32 [N] or null. `tune` != 0: a shape not yet timed has the library's candidate
// kernels run TIMED_RUNS times each on `stream` (which is waited for: not inside a capture) and keeps the fastest;
// otherwise a new shape takes the library's first choice. The output is written by every candidate run, each
// time with the whole result.
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
  std::vector<hipblasLtMatmulHeuristicResult_t> found;
  if (it == plans.end() || (tune && !it->second.timed)) {
    Plan fresh;
    const int made = make_plan(key, fresh, found);
    if (made != 0) {
      drop(fresh);
      return made;
    }
    if (it != plans.end()) {
      drop(it->second);
      it->second = fresh;
    } else {
      it = plans.emplace(key, fresh).first;
      ++plans_made;
    }
    if (tune) {
      // every kernel of the library that takes this product, not only the first of its own ranking (which is
      // made for speed of choice: at 2,048 x 37,888 x 3,584 the best of all kernels is 10 % faster than the best
      // of the first 16)
      std::vector<hipblasLtMatmulAlgo_t> candidates;
      for (const auto& r : found) candidates.push_back(r.algo);
      {
        const hipDataType in_type = type_of(x_dtype), out_type = type_of(y_dtype);
        std::vector<hipblasLtMatmulHeuristicResult_t> all;
        if (ok(hipblaslt_ext::getAllAlgos(handle, hipblaslt_ext::GemmType::HIPBLASLT_GEMM, HIPBLAS_OP_T, HIPBLAS_OP_N,
                                          in_type, in_type, out_type, out_type, HIPBLAS_COMPUTE_32F, all))) {
          const float one = 1.f, zero = 0.f;
          for (auto& r : all) {
            size_t needs = 0;
            if (ok(hipblaslt_ext::matmulIsAlgoSupported(handle, it->second.product, &one, it->second.w, it->second.x, &zero,
                                                        it->second.y, it->second.y, r.algo, needs)) &&
                needs <= WORKSPACE_BYTES)
              candidates.push_back(r.algo);
          }
        }
      }
      hipEvent_t begin, end;
      if (hipEventCreate(&begin) != hipSuccess || hipEventCreate(&end) != hipSuccess) return DISTIE_LIB_NOT_READY;
      // Every timed run starts on cold caches, as the product will between its neighbours in a step: a buffer
      // larger than the memory-side cache is overwritten first. Timed back to back on warm weights, the choice
      // was less stable from run to run and no better (2,048-token prefill of the 1.5B shape on one box: 9.39 and
      // 10.0 ms warm, 9.36 and 9.22 cold; the library's own first 16 warm: 9.36; the 7B shape 27.6 / 27.5 / 29.6).
      void* flush = nullptr;
      if (hipMalloc(&flush, FLUSH_BYTES) != hipSuccess) flush = nullptr;
      auto timed = [&](const hipblasLtMatmulAlgo_t& algo, int runs, float& ms) {
        ms = 0.f;
        for (int r = 0; r < runs; ++r) {
          if (flush != nullptr && hipMemsetAsync(flush, r, FLUSH_BYTES, stream) != hipSuccess) return false;
          hipEventRecord(begin, stream);
          const bool ran = ok(run(it->second, algo, x, w, bias, y, stream));
          hipEventRecord(end, stream);
          if (hipEventSynchronize(end) != hipSuccess || !ran) return false;
          float one_run = 0.f;
          hipEventElapsedTime(&one_run, begin, end);
          ms += one_run / runs;
        }
        return true;
      };
      float best = -1.f;
      for (const auto& candidate : candidates) {
        float once = 0.f, ms = 0.f;
        if (!timed(candidate, 1, once)) continue;                               // a warm-up, and a check
        if (best > 0.f && once > WORTH_TIMING * best) continue;
        if (!timed(candidate, TIMED_RUNS, ms)) continue;
        if (best < 0.f || ms < best) {
          best = ms;
          it->second.algo = candidate;
        }
      }
      if (flush != nullptr) hipFree(flush);
      hipEventDestroy(begin);
      hipEventDestroy(end);
      if (best < 0.f) return DISTIE_LIB_UNSUPPORTED;
      it->second.timed = true;
      ++plans_timed;
    }
  }
  const hipblasStatus_t s = run(it->second, it->second.algo, x, w, bias, y, stream);
  if (!ok(s)) return DISTIE_LIB_UNSUPPORTED;
  return launch_status();
}
