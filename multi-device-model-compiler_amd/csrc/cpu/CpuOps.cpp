// CPU op library of the CPU runner: plain C++ / OpenMP, fp32 arithmetic.
// Semantics follow lib/Kernels/CPU/Ops.cpp:34-80 (matmul: out = in . W + bias,
// row major) and the GPU entry points of the same name for the rest.
#include "multi-device-model-compiler/Kernels/CPU/Ops.h"

#include <cmath>
#include <cstring>
#include <vector>
#ifdef _OPENMP
#include <omp.h>
#endif

static bool fastFlag = false;

void cpuOpsInit(bool fastMathFlag) { fastFlag = fastMathFlag; }
bool getOpsFastFlag() { return fastFlag; }
int cpuOpsNumThreads() {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

namespace {
inline float halfToFloat(uint16_t h) {
  const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1fu, man = h & 0x3ffu, bits;
  if (exp == 0) {
    if (man == 0) {
      bits = sign;
    } else {
      int e = -1;
      do {
        man <<= 1;
        e++;
      } while (!(man & 0x400u));
      bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3ffu) << 13);
    }
  } else if (exp == 31) {
    bits = sign | 0x7f800000u | (man << 13);
  } else {
    bits = sign | ((exp + 112u) << 23) | (man << 13);
  }
  float f;
  std::memcpy(&f, &bits, 4);
  return f;
}

inline uint16_t floatToHalf(float f) {
  uint32_t x;
  std::memcpy(&x, &f, 4);
  const uint32_t sign = (x >> 16) & 0x8000u;
  x &= 0x7fffffffu;
  if (x >= 0x7f800000u) return (uint16_t)(sign | 0x7c00u | (x > 0x7f800000u ? 0x200u : 0));
  if (x >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u); // rounds to inf
  if (x < 0x33000001u) return (uint16_t)sign;              // rounds to zero
  int exp = (int)(x >> 23) - 127;
  uint32_t man = (x & 0x7fffffu) | 0x800000u;
  int shift = exp >= -14 ? 13 : 13 + (-14 - exp);
  uint32_t kept = man >> shift, rem = man & ((1u << shift) - 1), half = 1u << (shift - 1);
  if (rem > half || (rem == half && (kept & 1))) kept++;
  uint32_t out = exp >= -14 ? (uint32_t)((exp + 15) << 10) + (kept - 1024u) : kept;
  return (uint16_t)(sign | out);
}
} // namespace

extern "C" {

void mcpuMatmul(float *input, float *weight, float *bias, float *output, int64_t M, int64_t N,
                int64_t K) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < M; i++) {
    float *o = output + i * N;
    for (int64_t j = 0; j < N; j++) o[j] = bias ? bias[j] : 0.0f;
    for (int64_t k = 0; k < K; k++) {
      const float a = input[i * K + k];
      const float *w = weight + k * N;
#pragma omp simd
      for (int64_t j = 0; j < N; j++) o[j] += a * w[j];
    }
  }
}

// NCHW fp32 convolution (cross-correlation) + bias + optional postAdd + optional
// ReLU; the CPU side of mgpuConv2d (reference: oneDNN convolution_forward with
// post-ops, lib/Kernels/CPU/Ops.cpp; Ops.h:24-29).  One output row at a time,
// the tap loop outermost so that the inner loop runs along the row.
void mcpuConv2d(float *input, float *weight, float *bias, float *output, float *postAdd, int64_t N,
                int64_t IC, int64_t H, int64_t W, int64_t OC, int64_t KH, int64_t KW, int64_t OH,
                int64_t OW, int64_t PHL, int64_t PWL, int64_t /*PHR*/, int64_t /*PWR*/, int64_t SH,
                int64_t SW, int64_t DH, int64_t DW, bool hasPostAdd, bool hasContainRelu) {
#pragma omp parallel for collapse(3) schedule(static)
  for (int64_t n = 0; n < N; n++)
    for (int64_t oc = 0; oc < OC; oc++)
      for (int64_t oh = 0; oh < OH; oh++) {
        float *row = output + ((n * OC + oc) * OH + oh) * OW;
        for (int64_t ow = 0; ow < OW; ow++) row[ow] = bias[oc];
        for (int64_t ic = 0; ic < IC; ic++)
          for (int64_t kh = 0; kh < KH; kh++) {
            const int64_t ih = oh * SH - PHL + kh * DH;
            if (ih < 0 || ih >= H) continue;
            const float *src = input + ((n * IC + ic) * H + ih) * W;
            for (int64_t kw = 0; kw < KW; kw++) {
              const float wv = weight[((oc * IC + ic) * KH + kh) * KW + kw];
              const int64_t off = kw * DW - PWL;
              // ow range with 0 <= ow*SW + off < W
              int64_t lo = off < 0 ? (-off + SW - 1) / SW : 0;
              int64_t hi = (W - 1 - off) >= 0 ? (W - 1 - off) / SW + 1 : 0;
              if (hi > OW) hi = OW;
#pragma omp simd
              for (int64_t ow = lo; ow < hi; ow++) row[ow] += wv * src[ow * SW + off];
            }
          }
        if (hasPostAdd) {
          const float *add = postAdd + ((n * OC + oc) * OH + oh) * OW;
          for (int64_t ow = 0; ow < OW; ow++) row[ow] += add[ow];
        }
        if (hasContainRelu)
          for (int64_t ow = 0; ow < OW; ow++) row[ow] = row[ow] > 0.0f ? row[ow] : 0.0f;
      }
}

// method 0: window maximum over the taps inside the image; 1: window sum over
// those taps divided by KH*KW (Ops.h:31-36).
void mcpuPool2d(float *input, float *output, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OH,
                int64_t OW, int64_t KH, int64_t KW, int64_t PHL, int64_t PWL, int64_t /*PHR*/,
                int64_t /*PWR*/, int64_t SH, int64_t SW, int64_t method) {
#pragma omp parallel for collapse(2) schedule(static)
  for (int64_t pl = 0; pl < N * C; pl++)
    for (int64_t oh = 0; oh < OH; oh++)
      for (int64_t ow = 0; ow < OW; ow++) {
        float acc = method ? 0.0f : -INFINITY;
        for (int64_t kh = 0; kh < KH; kh++) {
          const int64_t ih = oh * SH - PHL + kh;
          if (ih < 0 || ih >= H) continue;
          for (int64_t kw = 0; kw < KW; kw++) {
            const int64_t iw = ow * SW - PWL + kw;
            if (iw < 0 || iw >= W) continue;
            const float v = input[(pl * H + ih) * W + iw];
            acc = method ? acc + v : (v > acc ? v : acc);
          }
        }
        output[(pl * OH + oh) * OW + ow] = method ? acc / (float)(KH * KW) : acc;
      }
}

void mcpuAddF32(const float *a, const float *b, float *c, int64_t n) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; i++) c[i] = a[i] + b[i];
}

void mcpuLayerNormF32(const float *input, const float *gamma, const float *beta, float *output,
                      float eps, int32_t m, int32_t n) {
#pragma omp parallel for schedule(static)
  for (int32_t r = 0; r < m; r++) {
    const float *x = input + (int64_t)r * n;
    float *y = output + (int64_t)r * n;
    float sum = 0.0f;
#pragma omp simd reduction(+ : sum)
    for (int32_t i = 0; i < n; i++) sum += x[i];
    const float mean = sum / (float)n;
    float sq = 0.0f;
#pragma omp simd reduction(+ : sq)
    for (int32_t i = 0; i < n; i++) sq += (x[i] - mean) * (x[i] - mean);
    const float rstd = 1.0f / std::sqrt(sq / (float)n + eps);
#pragma omp simd
    for (int32_t i = 0; i < n; i++) y[i] = (x[i] - mean) * rstd * gamma[i] + beta[i];
  }
}

void mcpuFusedMHAF16(const void *qkvv, const int32_t *seqlens, void *outv, int32_t B, int32_t S,
                     int32_t H, int32_t D, float scale, int32_t causal) {
  const uint16_t *qkv = static_cast<const uint16_t *>(qkvv);
  uint16_t *out = static_cast<uint16_t *>(outv);
  const int64_t tok = 3LL * H * D;
#pragma omp parallel
  {
    std::vector<float> q((size_t)S * D), k((size_t)S * D), v((size_t)S * D), p(S), acc(D);
#pragma omp for collapse(2) schedule(dynamic)
    for (int32_t b = 0; b < B; b++)
      for (int32_t h = 0; h < H; h++) {
        int32_t len = seqlens ? seqlens[b] : S;
        len = len < 0 ? 0 : (len > S ? S : len);
        for (int32_t s = 0; s < S; s++) {
          const int64_t base = ((int64_t)b * S + s) * tok + (int64_t)h * D;
          for (int32_t d = 0; d < D; d++) {
            q[(size_t)s * D + d] = halfToFloat(qkv[base + d]);
            k[(size_t)s * D + d] = halfToFloat(qkv[base + (int64_t)H * D + d]);
            v[(size_t)s * D + d] = halfToFloat(qkv[base + 2LL * H * D + d]);
          }
        }
        for (int32_t i = 0; i < S; i++) {
          int32_t nk = len;
          if (causal && i + 1 < nk) nk = i + 1;
          uint16_t *o = out + ((int64_t)b * S + i) * H * D + (int64_t)h * D;
          if (nk <= 0) {
            for (int32_t d = 0; d < D; d++) o[d] = 0;
            continue;
          }
          float mx = -INFINITY;
          for (int32_t j = 0; j < nk; j++) {
            float dot = 0.0f;
#pragma omp simd reduction(+ : dot)
            for (int32_t d = 0; d < D; d++) dot += q[(size_t)i * D + d] * k[(size_t)j * D + d];
            p[j] = dot * scale;
            mx = p[j] > mx ? p[j] : mx;
          }
          float den = 0.0f;
          for (int32_t j = 0; j < nk; j++) {
            p[j] = std::exp(p[j] - mx);
            den += p[j];
          }
          for (int32_t d = 0; d < D; d++) acc[d] = 0.0f;
          for (int32_t j = 0; j < nk; j++) {
            const float pj = p[j];
#pragma omp simd
            for (int32_t d = 0; d < D; d++) acc[d] += pj * v[(size_t)j * D + d];
          }
          for (int32_t d = 0; d < D; d++) o[d] = floatToHalf(acc[d] / den);
        }
      }
  }
}

} // extern "C"
