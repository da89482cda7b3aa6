// Timed launch loops for bench.py.  A compiled model calls the kernel library
// from C++ at a few hundred nanoseconds per call; a Python caller needs
// several microseconds per ctypes call, longer than the streaming kernels run.
// These loops make K calls of one C-ABI entry point from C++, rotating through
// `nsets` buffer sets, between two events recorded on the launch stream, and
// return the elapsed milliseconds.  Measurement plumbing only: nothing here is
// part of the kernel library, and every launch goes through the same entry
// point a model would call.
#include "mgpu_ops.h"

#include "bench_timed.hpp"

#include <hip/hip_runtime.h>

#include <cstdint>

using mgpu_bench::timed;

extern "C" {

float mgpuBenchLayerNormF32(void *const *x, void *const *y, int nsets, const void *gamma, const void *beta,
                            float eps, int m, int n, int steps, int warmup, void *stream) {
  return timed(
      [&](unsigned long i) {
        mgpuLayerNormF32(static_cast<const float *>(x[i % nsets]), static_cast<const float *>(gamma),
                         static_cast<const float *>(beta), static_cast<float *>(y[i % nsets]), eps, m, n, stream);
      },
      steps, warmup, static_cast<hipStream_t>(stream));
}

float mgpuBenchLayerNormF16(void *const *x, void *const *y, int nsets, const void *gamma, const void *beta,
                            float eps, int m, int n, int steps, int warmup, void *stream) {
  return timed([&](unsigned long i) { mgpuLayerNormF16(x[i % nsets], gamma, beta, y[i % nsets], eps, m, n, stream); }, steps,
               warmup, static_cast<hipStream_t>(stream));
}

float mgpuBenchAddF32(void *const *a, void *const *b, void *const *c, int nsets, int64_t n, int steps, int warmup,
                      void *stream) {
  return timed(
      [&](unsigned long i) {
        mgpuAddF32(static_cast<const float *>(a[i % nsets]), static_cast<const float *>(b[i % nsets]),
                   static_cast<float *>(c[i % nsets]), n, stream);
      },
      steps, warmup, static_cast<hipStream_t>(stream));
}

float mgpuBenchFusedMHAF16(void *const *qkv, void *const *out, int nsets, const int32_t *seqlens, int B, int S,
                           int H, int D, float scale, int causal, int steps, int warmup, void *stream) {
  return timed(
      [&](unsigned long i) { mgpuFusedMHAF16(qkv[i % nsets], seqlens, out[i % nsets], B, S, H, D, scale, causal, stream); },
      steps, warmup, static_cast<hipStream_t>(stream));
}

float mgpuBenchBertEncoderLayerF16(const void *x, void *const *params, const int32_t *seqlens, void *out, int64_t B,
                                   int64_t S, int64_t d, int64_t ffn, int64_t H, float eps, int noAlloc, int steps,
                                   int warmup, void *stream) {
  auto *fn = noAlloc ? mgpuBertEncoderLayerF16NoAlloc : mgpuBertEncoderLayerF16;
  return timed(
      [&](unsigned long) {
        fn(x, params[0], params[1], params[2], params[3], params[4], params[5], params[6], params[7], params[8],
           params[9], params[10], params[11], seqlens, out, B, S, d, ffn, H, eps, stream);
      },
      steps, warmup, static_cast<hipStream_t>(stream));
}

} // extern "C"
