// Timed launch loops for bench.py.  A compiled model calls the kernel library
// from C++ at a few hundred nanoseconds per call; a Python caller needs
// several microseconds per ctypes call, longer than the streaming kernels run.
// These loops make K calls of one C-ABI entry point from C++, rotating through
// `nsets` buffer sets, between two events recorded on the launch stream, and
// return the elapsed milliseconds.  Measurement plumbing only: nothing here is
// part of the kernel library, and every launch goes through the same entry
// point a model would call.
#include "mgpu_ops.h"

#include <hip/hip_runtime.h>

#include <cstdint>

namespace {
template <typename F> float timed(F &&launch, int steps, int warmup, hipStream_t stream) {
  for (int i = 0; i < warmup; i++) launch(i);
  if (hipStreamSynchronize(stream) != hipSuccess) return -1.0f;
  hipEvent_t e0, e1;
  if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) return -1.0f;
  (void)hipEventRecord(e0, stream);
  for (int i = 0; i < steps; i++) launch(i);
  (void)hipEventRecord(e1, stream);
  float ms = -1.0f;
  if (hipEventSynchronize(e1) != hipSuccess || hipEventElapsedTime(&ms, e0, e1) != hipSuccess) ms = -1.0f;
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  return ms;
}
} // namespace

extern "C" {

float mgpuBenchLayerNormF32(void *const *x, void *const *y, int nsets, const void *gamma, const void *beta,
                            float eps, int m, int n, int steps, int warmup, void *stream) {
  return timed(
      [&](int i) {
        mgpuLayerNormF32(static_cast<const float *>(x[i % nsets]), static_cast<const float *>(gamma),
                         static_cast<const float *>(beta), static_cast<float *>(y[i % nsets]), eps, m, n, stream);
      },
      steps, warmup, static_cast<hipStream_t>(stream));
}

float mgpuBenchLayerNormF16(void *const *x, void *const *y, int nsets, const void *gamma, const void *beta,
                            float eps, int m, int n, int steps, int warmup, void *stream) {
  return timed([&](int i) { mgpuLayerNormF16(x[i % nsets], gamma, beta, y[i % nsets], eps, m, n, stream); }, steps,
               warmup, static_cast<hipStream_t>(stream));
}

float mgpuBenchAddF32(void *const *a, void *const *b, void *const *c, int nsets, int64_t n, int steps, int warmup,
                      void *stream) {
  return timed(
      [&](int i) {
        mgpuAddF32(static_cast<const float *>(a[i % nsets]), static_cast<const float *>(b[i % nsets]),
                   static_cast<float *>(c[i % nsets]), n, stream);
      },
      steps, warmup, static_cast<hipStream_t>(stream));
}

float mgpuBenchFusedMHAF16(void *const *qkv, void *const *out, int nsets, const int32_t *seqlens, int B, int S,
                           int H, int D, float scale, int causal, int steps, int warmup, void *stream) {
  return timed(
      [&](int i) { mgpuFusedMHAF16(qkv[i % nsets], seqlens, out[i % nsets], B, S, H, D, scale, causal, stream); },
      steps, warmup, static_cast<hipStream_t>(stream));
}

float mgpuBenchBertEncoderLayerF16(const void *x, void *const *params, const int32_t *seqlens, void *out, int64_t B,
                                   int64_t S, int64_t d, int64_t ffn, int64_t H, float eps, int noAlloc, int steps,
                                   int warmup, void *stream) {
  auto *fn = noAlloc ? mgpuBertEncoderLayerF16NoAlloc : mgpuBertEncoderLayerF16;
  return timed(
      [&](int) {
        fn(x, params[0], params[1], params[2], params[3], params[4], params[5], params[6], params[7], params[8],
           params[9], params[10], params[11], seqlens, out, B, S, d, ffn, H, eps, stream);
      },
      steps, warmup, static_cast<hipStream_t>(stream));
}

} // extern "C"
