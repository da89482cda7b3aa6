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
//    MGPU_GEMM_KERNEL=library or =mfma in the environment overrides both.
//    Nothing in this library measures anything: the tuner that writes the
//    table lives with the benchmark's launch loops;
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

// The stream's workspace; null when it has none yet and none can be made now (the stream
// is capturing, or the allocation failed).  Workspaces are kept per stream handle until
// gemmDeinit(); a caller that creates and destroys streams without end should run its
// GEMMs on a bounded set of them.
void *workspaceFor(hipStream_t s) {
  auto it = workspaceOf.find(s);
  if (it != workspaceOf.end()) return it->second;
  if (isCapturing(s)) return nullptr;
  void *ws = nullptr;
  if (hipMalloc(&ws, workspaceSize) != hipSuccess) { // out of memory, or another stream is capturing
    (void)hipGetLastError();
    return nullptr; // the caller falls back to an algorithm that needs no workspace; asked again next time
  }
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

// Shapes decided offline: {type (1 fp16, 2 bf16), M, N, K, hasBias, act, hasResidual, hand-written kernel
// (against the library, both on the ABI's [K, N] weight)?, the library on a K-major copy of the weight
// ahead of both?}.
struct TableEntry {
  int dt;
  int64_t M, N, K;
  int hasBias, act, hasResidual, handWritten, kMajorLibrary;
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

bool mfmaShape(DType dt, int64_t M, int64_t N, int64_t K) {
  return (dt == DType::F16 || dt == DType::BF16) && M > 0 && M % 128 == 0 && (N % 128 == 0 || N % 96 == 0) && K % 32 == 0;
}

const TableEntry *tableRow(DType dt, int64_t M, int64_t N, int64_t K, bool hasBias, int act, bool hasResidual) {
  for (const TableEntry &e : kTable)
    if (e.dt == (int)dt && e.M == M && e.N == N && e.K == K && e.hasBias == (int)hasBias && e.act == act &&
        e.hasResidual == (int)hasResidual)
      return &e;
  return nullptr;
}

using Key = std::tuple<int64_t, int64_t, int64_t, int, int, int, int, int>;
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

constexpr int kCandidates = 16; // heuristic answers looked through for one that needs no workspace

// Builds (once per shape, flags and type) the library's descriptors and picks its
// algorithms; decides which kernel serves the shape.  No measurement, no allocation
// beyond the library's host-side descriptors.
Plan &getPlan(DType dt, int64_t M, int64_t N, int64_t K, bool hasBias, int act, bool hasResidual, bool weightKMajor) {
  const bool relu = act == ACT_RELU;
  const Key key{M, N, K, (int)hasBias, act, (int)hasResidual, (int)dt, (int)weightKMajor};
  auto it = plans.find(key);
  if (it != plans.end()) return it->second;

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
  // Column-major view of the row-major operands: A = weight (N x K, ld N; a K-major weight is
  // the K x N matrix with ld K, transposed), B = input (K x M, ld K), C/D = output (N x M, ld N).
  if (weightKMajor) {
    const hipblasOperation_t transposed = HIPBLAS_OP_T;
    MGPU_CHECK_BLAS(hipblasLtMatmulDescSetAttribute(p.op, HIPBLASLT_MATMUL_DESC_TRANSA, &transposed, sizeof(transposed)));
    MGPU_CHECK_BLAS(hipblasLtMatrixLayoutCreate(&p.a, t, K, N, K));
  } else {
    MGPU_CHECK_BLAS(hipblasLtMatrixLayoutCreate(&p.a, t, N, K, N));
  }
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

  // The kernel: the table, else the rule.
  p.handWritten = mfmaShape(dt, M, N, K) && ruleSaysHandWritten(M, N, K, act);
  if (const TableEntry *e = tableRow(dt, M, N, K, hasBias, act, hasResidual)) p.handWritten = mfmaShape(dt, M, N, K) && e->handWritten != 0;
  if (forcedKernel()) p.handWritten = forcedKernel() == 2;
  if (weightKMajor) p.handWritten = false; // the hand-written kernel reads [K, N] weights only
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

bool gemmPrefersKMajor(DType dt, int64_t M, int64_t N, int64_t K, bool hasBias, int act, bool hasResidual) {
  if (forcedKernel()) return forcedKernel() == 1;
  if (const TableEntry *e = tableRow(dt, M, N, K, hasBias, act, hasResidual)) return e->kMajorLibrary != 0;
  // Nobody measured the shape: the library's kernels for K-major weights were ahead of its
  // kernels for [K, N] weights at every shape measured, so the copy pays wherever the library
  // would serve the shape anyway.
  return !(mfmaShape(dt, M, N, K) && ruleSaysHandWritten(M, N, K, act));
}

void matmulEx(DType dt, const void *input, const void *weight, const void *bias, void *output,
              const void *residual, int64_t M, int64_t N, int64_t K, bool hasBias, int act,
              bool hasResidual, hipStream_t stream, bool weightKMajor) {
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
  const Plan &p = getPlan(dt, M, N, K, hasBias, act, hasResidual, weightKMajor);
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
    if (!p.hasNoWs) fail("matmul: the library needs a workspace for this shape and none could be allocated now (stream capture or out of memory); run it once on this stream before capturing");
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

} // namespace mgpu
