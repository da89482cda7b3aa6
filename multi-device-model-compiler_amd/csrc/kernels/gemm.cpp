// GEMM with bias / activation / residual epilogue over hipBLASLt.
//
// Replaces mgpuMatmul and mgpuMatmulEx<T> (lib/Kernels/GPU/Ops.cu:57-120,
// 134-234).  Same row-major contract through the column-major operand swap of
// Ops.cu:83-85,178-183: out^T[N,M] = W^T[N,K] . in^T[K,M].  Differences:
//  * the whole plan (operation descriptor, layouts, chosen algorithm) is built
//    once per (shape, flags, type) and reused; the reference rebuilds all
//    descriptors on every call and caches only the heuristic result;
//  * fp16 / bf16 inputs accumulate in fp32 (HIPBLAS_COMPUTE_32F); the reference
//    asks for fp16 accumulation (Ops.cu:164-167);
//  * GELU is applied by an exact-erf kernel after a bias-only epilogue, because
//    the library's fused GELU is the tanh approximation;
//  * a call only enqueues: which of the two kernels serves a shape - the
//    library or the hand-written MFMA kernel of gemm_mfma.hip - comes from a
//    table decided offline (gemm_table.inc, written by `bench.py --tune-gemm`
//    from measurements on an MI355X) and, for shapes the table does not hold,
//    from a fixed rule; the library runs the heuristic's first algorithm.
//    MGPU_GEMM_KERNEL=library or =mfma in the environment overrides both.  A
//    caller who wants a shape measured on its own device asks for it
//    explicitly with tuneMatmulEx (mgpuMatmulExTune in the C ABI), outside any
//    stream capture: that call allocates scratch operands, times the
//    library's candidates and the hand-written kernel, and keeps the winner
//    for the rest of the process;
//  * the library's workspace is per caller stream (allocated on a stream's
//    first library GEMM outside a capture), so GEMMs on different streams never
//    share one; a stream first seen under capture gets an algorithm that needs
//    no workspace.
#include "common.hpp"
#include "mgpu_ops_internal.hpp"

#include <hipblaslt/hipblaslt.h>

#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <tuple>
#include <vector>

namespace mgpu {

namespace {

hipblasLtHandle_t ltHandle = nullptr;
constexpr size_t workspaceSize = 32u * 1024u * 1024u;
std::mutex planMutex;
std::map<hipStream_t, void *> workspaceOf; // per caller stream, see the header comment

bool isCapturing(hipStream_t s) {
  hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
  return hipStreamIsCapturing(s, &capture) != hipSuccess || capture != hipStreamCaptureStatusNone;
}

// The stream's workspace; null when it has none yet and none can be made now (capture).
void *workspaceFor(hipStream_t s) {
  auto it = workspaceOf.find(s);
  if (it != workspaceOf.end()) return it->second;
  if (isCapturing(s)) return nullptr;
  void *ws = nullptr;
  MGPU_CHECK_HIP(hipMalloc(&ws, workspaceSize));
  workspaceOf[s] = ws;
  return ws;
}

void checkBlas(hipblasStatus_t status, const char *where) {
  if (status != HIPBLAS_STATUS_SUCCESS)
    fail(std::string(where) + ": hipBLASLt API failed with status " + std::to_string((int)status));
}
#define MGPU_CHECK_BLAS(expr) checkBlas((expr), #expr)

struct Plan {
  hipblasLtMatmulDesc_t op = nullptr;
  hipblasLtMatrixLayout_t a = nullptr, b = nullptr, d = nullptr;
  hipblasLtMatmulAlgo_t algo;          // the heuristic's first answer (or the tuned one)
  size_t algoWorkspace = 0;
  hipblasLtMatmulAlgo_t algoNoWs;      // the first answer that needs no workspace
  bool hasNoWs = false;
  bool handWritten = false; // serve the shape with gemm_mfma.hip when the operands allow it
};

// Shapes decided offline: {type (1 fp16, 2 bf16), M, N, K, hasBias, act, hasResidual, hand-written kernel?}.
struct TableEntry {
  int dt;
  int64_t M, N, K;
  int hasBias, act, hasResidual, handWritten;
};
const TableEntry kTable[] = {
#include "gemm_table.inc"
};

// Which kernel serves a shape nobody measured: the hand-written one where it can pay -
// reductions up to 1024 deep, a GELU to fuse, or at most one 128-row tile per CU (its
// eight-wavefront form).  On long reductions over many tiles the library's steady state
// is ahead.
bool ruleSaysHandWritten(int64_t M, int64_t N, int64_t K, int act) {
  return K <= 1024 || act == ACT_GELU || (M / 128) * (N / 128) <= numComputeUnits();
}

// 0: measure, 1: always the library, 2: the hand-written kernel wherever it applies
int forcedKernel() {
  static const int mode = [] {
    const char *v = std::getenv("MGPU_GEMM_KERNEL");
    if (!v) return 0;
    if (!std::strcmp(v, "library")) return 1;
    if (!std::strcmp(v, "mfma")) return 2;
    return 0;
  }();
  return mode;
}

using Key = std::tuple<int64_t, int64_t, int64_t, int, int, int, int>;
std::map<Key, Plan> plans;

hipDataType dataType(DType dt) {
  switch (dt) {
  case DType::F32:
    return HIP_R_32F;
  case DType::F16:
    return HIP_R_16F;
  default:
    return HIP_R_16BF;
  }
}

void destroyPlan(Plan &p) {
  if (p.d) hipblasLtMatrixLayoutDestroy(p.d);
  if (p.b) hipblasLtMatrixLayoutDestroy(p.b);
  if (p.a) hipblasLtMatrixLayoutDestroy(p.a);
  if (p.op) hipblasLtMatmulDescDestroy(p.op);
  p = Plan{};
}

constexpr int kCandidates = 64; // heuristic answers asked for and screened
constexpr int kFinalists = 4;   // re-timed at length after the screening pass

// Times the candidates on scratch operands of the plan's shape (its own stream,
// its own buffers: the caller's data and stream are not touched) and returns
// the index of the fastest; 0 when nothing could be measured.  *handWritten
// says whether the hand-written kernel beat it (with the separate GELU pass
// counted on the library's side).
int fastestCandidate(const Plan &p, const hipblasLtMatmulHeuristicResult_t *results, int count, DType dt,
                     int64_t M, int64_t N, int64_t K, bool hasBias, int act, bool hasResidual,
                     bool *handWritten) {
  const size_t eb = dt == DType::F32 ? 4 : 2;
  void *in = nullptr, *w = nullptr, *out = nullptr, *bias = nullptr, *workspace = nullptr;
  hipStream_t s = nullptr;
  hipEvent_t e0 = nullptr, e1 = nullptr;
  int best = 0;
  const bool ready = hipMalloc(&in, (size_t)M * K * eb) == hipSuccess && hipMalloc(&w, (size_t)K * N * eb) == hipSuccess &&
                     hipMalloc(&out, (size_t)M * N * eb) == hipSuccess && hipMalloc(&bias, (size_t)N * eb) == hipSuccess &&
                     hipMalloc(&workspace, workspaceSize) == hipSuccess &&
                     hipStreamCreate(&s) == hipSuccess && hipEventCreate(&e0) == hipSuccess &&
                     hipEventCreate(&e1) == hipSuccess;
  if (ready) {
    // 0x3c bytes: 1.06 as fp16, 0.0115 as fp32, finite in every type
    (void)hipMemsetAsync(in, 0x3c, (size_t)M * K * eb, s);
    (void)hipMemsetAsync(w, 0x3c, (size_t)K * N * eb, s);
    (void)hipMemsetAsync(out, 0x3c, (size_t)M * N * eb, s);
    (void)hipMemsetAsync(bias, 0x3c, (size_t)N * eb, s);
    if (hasBias)
      (void)hipblasLtMatmulDescSetAttribute(p.op, HIPBLASLT_MATMUL_DESC_BIAS_POINTER, &bias, sizeof(bias));
    const float alpha = 1.0f, beta = hasResidual ? 1.0f : 0.0f;
    // reps launches of candidate c between two events, after one untimed launch; < 0 on failure
    auto timeCandidate = [&](int c, int reps) -> float {
      bool ok = true;
      for (int rep = 0; rep <= reps && ok; rep++) {
        if (rep == 1) (void)hipEventRecord(e0, s);
        ok = hipblasLtMatmul(ltHandle, p.op, &alpha, w, p.a, in, p.b, &beta, out, p.d, out, p.d, &results[c].algo,
                             workspace, workspaceSize, s) == HIPBLAS_STATUS_SUCCESS;
      }
      float ms = 0.0f;
      if (!ok || hipEventRecord(e1, s) != hipSuccess || hipEventSynchronize(e1) != hipSuccess ||
          hipEventElapsedTime(&ms, e0, e1) != hipSuccess)
        return -1.0f;
      return ms / reps;
    };
    // Screening: three launches each; the kFinalists fastest go on.
    std::vector<std::pair<float, int>> screened;
    for (int c = 0; c < count; c++) {
      if (results[c].state != HIPBLAS_STATUS_SUCCESS || results[c].workspaceSize > workspaceSize) continue;
      const float ms = timeCandidate(c, 3);
      if (ms >= 0.0f) screened.emplace_back(ms, c);
    }
    std::sort(screened.begin(), screened.end());
    // Final: twenty launches each.
    float bestMs = -1.0f;
    for (size_t i = 0; i < screened.size() && i < (size_t)kFinalists; i++) {
      const float ms = timeCandidate(screened[i].second, 20);
      if (ms >= 0.0f && (bestMs < 0.0f || ms < bestMs)) {
        bestMs = ms;
        best = screened[i].second;
      }
    }
    // The hand-written kernel on the same operands (`out` doubles as the residual).
    const void *biasArg = hasBias ? bias : nullptr, *resArg = hasResidual ? out : nullptr;
    if (bestMs >= 0.0f && gemmMfmaSupports(dt, in, w, biasArg, resArg, out, M, N, K)) {
      // Both paths in alternating runs of twenty launches, three runs each, so that
      // they meet the same clocks: a lone burst of a kernel that has the device to
      // itself for a millisecond runs faster than the same kernel in a layer.
      auto timeLoop = [&](auto &&launchOnce) -> float {
        try {
          launchOnce();
          (void)hipEventRecord(e0, s);
          for (int rep = 0; rep < 20; rep++) launchOnce();
        } catch (const std::exception &) {
          return -1.0f;
        }
        float ms = 0.0f;
        if (hipEventRecord(e1, s) != hipSuccess || hipEventSynchronize(e1) != hipSuccess ||
            hipEventElapsedTime(&ms, e0, e1) != hipSuccess)
          return -1.0f;
        return ms;
      };
      const float alpha1 = 1.0f, beta1 = hasResidual ? 1.0f : 0.0f;
      auto libraryOnce = [&] {
        if (hipblasLtMatmul(ltHandle, p.op, &alpha1, w, p.a, in, p.b, &beta1, out, p.d, out, p.d, &results[best].algo,
                            workspace, workspaceSize, s) != HIPBLAS_STATUS_SUCCESS)
          throw std::runtime_error("hipblasLtMatmul");
        if (act == ACT_GELU) {
          if (dt == DType::F16) geluInPlaceF16(out, (size_t)M * N, s);
          else geluInPlaceBF16(out, (size_t)M * N, s);
        }
      };
      auto mfmaOnce = [&] { gemmMfma(dt, in, w, biasArg, resArg, out, M, N, K, act, s); };
      float libraryMs = 0.0f, mfmaMs = 0.0f;
      bool ok = true;
      for (int round = 0; round < 3 && ok; round++) {
        const float l = timeLoop(libraryOnce), m = timeLoop(mfmaOnce);
        ok = l >= 0.0f && m >= 0.0f;
        libraryMs += l;
        mfmaMs += m;
      }
      // three per cent of margin: a tie goes to the library
      *handWritten = ok && mfmaMs < 0.97f * libraryMs;
    }
    (void)hipStreamSynchronize(s);
  }
  if (e0) (void)hipEventDestroy(e0);
  if (e1) (void)hipEventDestroy(e1);
  if (s) (void)hipStreamDestroy(s);
  for (void *ptr : {in, w, out, bias, workspace})
    if (ptr) (void)hipFree(ptr);
  (void)hipGetLastError();
  return best;
}

// Builds (once per shape, flags and type) the library's descriptors and picks its
// algorithms; decides which kernel serves the shape.  No measurement, no allocation
// beyond the library's host-side descriptors.  With `tune` the caller has asked for the
// measurement (tuneMatmulEx).
Plan &getPlan(DType dt, int64_t M, int64_t N, int64_t K, bool hasBias, int act, bool hasResidual, bool tune) {
  const bool relu = act == ACT_RELU;
  const Key key{M, N, K, (int)hasBias, act, (int)hasResidual, (int)dt};
  auto it = plans.find(key);
  if (it != plans.end() && !tune) return it->second;
  if (it != plans.end()) {
    destroyPlan(it->second);
    plans.erase(it);
  }

  Plan p;
  const hipDataType t = dataType(dt);
  MGPU_CHECK_BLAS(hipblasLtMatmulDescCreate(&p.op, HIPBLAS_COMPUTE_32F, HIP_R_32F));
  hipblasLtEpilogue_t epilogue = HIPBLASLT_EPILOGUE_DEFAULT;
  if (hasBias && relu)
    epilogue = HIPBLASLT_EPILOGUE_RELU_BIAS;
  else if (hasBias)
    epilogue = HIPBLASLT_EPILOGUE_BIAS;
  else if (relu)
    epilogue = HIPBLASLT_EPILOGUE_RELU;
  MGPU_CHECK_BLAS(hipblasLtMatmulDescSetAttribute(p.op, HIPBLASLT_MATMUL_DESC_EPILOGUE, &epilogue,
                                                  sizeof(epilogue)));
  if (hasBias) {
    const int32_t biasType = (int32_t)t;
    MGPU_CHECK_BLAS(hipblasLtMatmulDescSetAttribute(p.op, HIPBLASLT_MATMUL_DESC_BIAS_DATA_TYPE,
                                                    &biasType, sizeof(biasType)));
  }
  // Column-major view of the row-major operands: A = weight (N x K, ld N),
  // B = input (K x M, ld K), C/D = output (N x M, ld N).
  MGPU_CHECK_BLAS(hipblasLtMatrixLayoutCreate(&p.a, t, N, K, N));
  MGPU_CHECK_BLAS(hipblasLtMatrixLayoutCreate(&p.b, t, K, M, K));
  MGPU_CHECK_BLAS(hipblasLtMatrixLayoutCreate(&p.d, t, N, M, N));

  hipblasLtMatmulPreference_t pref = nullptr;
  MGPU_CHECK_BLAS(hipblasLtMatmulPreferenceCreate(&pref));
  const uint64_t ws = workspaceSize;
  MGPU_CHECK_BLAS(hipblasLtMatmulPreferenceSetAttribute(
      pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &ws, sizeof(ws)));
  hipblasLtMatmulHeuristicResult_t results[kCandidates] = {};
  int returned = 0;
  const hipblasStatus_t st = hipblasLtMatmulAlgoGetHeuristic(ltHandle, p.op, p.a, p.b, p.d, p.d,
                                                             pref, kCandidates, results, &returned);
  hipblasLtMatmulPreferenceDestroy(pref);
  if (st != HIPBLAS_STATUS_SUCCESS || returned == 0) {
    destroyPlan(p);
    fail("matmul: hipBLASLt has no algorithm for M=" + std::to_string(M) + " N=" +
         std::to_string(N) + " K=" + std::to_string(K));
  }
  p.algo = results[0].algo;
  p.algoWorkspace = results[0].workspaceSize;
  for (int c = 0; c < returned && !p.hasNoWs; c++)
    if (results[c].state == HIPBLAS_STATUS_SUCCESS && results[c].workspaceSize == 0) {
      p.algoNoWs = results[c].algo;
      p.hasNoWs = true;
    }

  // The kernel: the table, else the rule; a measurement only when asked for.
  const bool mfmaShape = (dt == DType::F16 || dt == DType::BF16) && M > 0 && M % 128 == 0 && (N % 128 == 0 || N % 96 == 0) && K % 32 == 0;
  p.handWritten = mfmaShape && ruleSaysHandWritten(M, N, K, act);
  for (const TableEntry &e : kTable)
    if (e.dt == (int)dt && e.M == M && e.N == N && e.K == K && e.hasBias == (int)hasBias && e.act == act &&
        e.hasResidual == (int)hasResidual)
      p.handWritten = mfmaShape && e.handWritten != 0;
  if (tune) {
    const int best = fastestCandidate(p, results, returned, dt, M, N, K, hasBias, act, hasResidual, &p.handWritten);
    p.algo = results[best].algo;
    p.algoWorkspace = results[best].workspaceSize;
  }
  if (forcedKernel()) p.handWritten = forcedKernel() == 2;
  return plans.emplace(key, p).first->second;
}

} // namespace

void gemmInit() {
  if (ltHandle) return;
  MGPU_CHECK_BLAS(hipblasLtCreate(&ltHandle));
}

void gemmDeinit() {
  std::lock_guard<std::mutex> lock(planMutex);
  for (auto &kv : plans) destroyPlan(kv.second);
  plans.clear();
  for (auto &kv : workspaceOf)
    if (kv.second) (void)hipFree(kv.second);
  workspaceOf.clear();
  if (ltHandle) hipblasLtDestroy(ltHandle);
  ltHandle = nullptr;
}

void matmulEx(DType dt, const void *input, const void *weight, const void *bias, void *output,
              const void *residual, int64_t M, int64_t N, int64_t K, bool hasBias, int act,
              bool hasResidual, hipStream_t stream) {
  if (M < 0 || N < 0 || K < 0) fail("matmul: negative shape");
  if (M == 0 || N == 0) return;
  if (K == 0) fail("matmul: K must be positive");
  if (!ltHandle) fail("matmul: gpuOpsInit() has not been called");
  if (!input || !weight || !output) fail("matmul: null pointer");
  if (hasBias && !bias) fail("matmul: hasBias set but bias is null");
  if (hasResidual && !residual) fail("matmul: hasResidual set but residual is null");
  if (act < ACT_NONE || act > ACT_GELU) fail("matmul: unknown activation");
  if (act != ACT_NONE && hasResidual)
    fail("matmul: an activation cannot be combined with a residual");

  std::lock_guard<std::mutex> lock(planMutex);
  const Plan &p = getPlan(dt, M, N, K, hasBias, act, hasResidual, false);
  if (p.handWritten && gemmMfmaSupports(dt, input, weight, hasBias ? bias : nullptr,
                                        hasResidual ? residual : nullptr, output, M, N, K)) {
    gemmMfma(dt, input, weight, hasBias ? bias : nullptr, hasResidual ? residual : nullptr, output, M, N, K, act,
             stream);
    return;
  }
  if (hasBias)
    MGPU_CHECK_BLAS(hipblasLtMatmulDescSetAttribute(p.op, HIPBLASLT_MATMUL_DESC_BIAS_POINTER, &bias,
                                                    sizeof(bias)));
  const float alpha = 1.0f, beta = hasResidual ? 1.0f : 0.0f;
  // The stream's own workspace; a stream first met under capture has none and runs the
  // first algorithm that does without.
  void *workspace = p.algoWorkspace ? workspaceFor(stream) : nullptr;
  const hipblasLtMatmulAlgo_t *algo = &p.algo;
  if (p.algoWorkspace && !workspace) {
    if (!p.hasNoWs) fail("matmul: the library needs a workspace for this shape; run it once on this stream before capturing");
    algo = &p.algoNoWs;
  }
  MGPU_CHECK_BLAS(hipblasLtMatmul(ltHandle, p.op, &alpha, weight, p.a, input, p.b, &beta,
                                  hasResidual ? residual : output, p.d, output, p.d, algo,
                                  workspace, workspace ? workspaceSize : 0, stream));
  if (act == ACT_GELU) {
    if (dt == DType::F16)
      geluInPlaceF16(output, (size_t)M * N, stream);
    else if (dt == DType::BF16)
      geluInPlaceBF16(output, (size_t)M * N, stream);
    else
      geluInPlaceF32(static_cast<float *>(output), (size_t)M * N, stream);
  }
}

// Measures, on this device and on scratch operands of the shape, the library's top
// candidates and the hand-written kernel, and keeps the faster path for the rest of the
// process.  Synchronous, allocates and frees device memory: never call it under stream
// capture or from a path that must only enqueue.  Returns true when the hand-written
// kernel was kept.
bool tuneMatmulEx(DType dt, int64_t M, int64_t N, int64_t K, bool hasBias, int act, bool hasResidual) {
  if (M <= 0 || N <= 0 || K <= 0) fail("tuneMatmulEx: bad shape");
  if (!ltHandle) fail("tuneMatmulEx: gpuOpsInit() has not been called");
  if (act < ACT_NONE || act > ACT_GELU || (act != ACT_NONE && hasResidual)) fail("tuneMatmulEx: bad epilogue");
  std::lock_guard<std::mutex> lock(planMutex);
  return getPlan(dt, M, N, K, hasBias, act, hasResidual, true).handWritten;
}

} // namespace mgpu
