// CPU op library of the CPU runner: plain C++ / OpenMP, fp32 arithmetic.
// Semantics follow lib/Kernels/CPU/Ops.cpp:34-80 (matmul: out = in . W + bias,
// row major) and the GPU entry points of the same name for the rest.
#include "multi-device-model-compiler/Kernels/CPU/Ops.h"

#include <cmath>
#include <cstddef>
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

// Thread count of the OpenMP loops below (the CPU baseline is timed at one
// thread and at all cores).
void mcpuSetNumThreads(int32_t n) {
#ifdef _OPENMP
  if (n > 0) omp_set_num_threads(n);
#else
  (void)n;
#endif
}
int32_t mcpuGetNumThreads(void) { return cpuOpsNumThreads(); }

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

// ---- 16-bit element types, fused epilogues and the layers --------------------
// CPU twins of the GPU entry points of the same name: fp32 arithmetic on the
// fp16 values the GPU path holds at the same point (every tensor that the GPU
// path stores as fp16 is rounded to fp16 here too), so that the two runners can
// be compared stage by stage.

void mcpuCastF32ToF16(void *dst, const float *src, size_t size) {
  uint16_t *d = static_cast<uint16_t *>(dst);
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < (int64_t)size; i++) d[i] = floatToHalf(src[i]);
}

void mcpuCastF16ToF32(float *dst, const void *src, size_t size) {
  const uint16_t *s = static_cast<const uint16_t *>(src);
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < (int64_t)size; i++) dst[i] = halfToFloat(s[i]);
}

} // extern "C"

namespace {

// One row: out = LayerNorm(x [+ residual]); `sum` (may be null) receives the
// rounded sum.  Statistics come from the un-rounded fp32 sums, the normalised
// value from the rounded one (the GPU kernel's dataflow, LayerNorm.cu:186-233).
template <bool HALF>
void layerNormRow(const void *xv, const void *rv, const void *gv, const void *bv, void *sumv, void *outv, float eps,
                  int64_t r, int32_t n, float *tmp) {
  auto load = [&](const void *p, int64_t i) {
    return HALF ? halfToFloat(static_cast<const uint16_t *>(p)[i]) : static_cast<const float *>(p)[i];
  };
  auto store = [&](void *p, int64_t i, float v) {
    if (HALF) static_cast<uint16_t *>(p)[i] = floatToHalf(v);
    else static_cast<float *>(p)[i] = v;
  };
  const int64_t base = r * n;
  float total = 0.0f;
  for (int32_t i = 0; i < n; i++) {
    tmp[i] = load(xv, base + i) + (rv ? load(rv, base + i) : 0.0f);
    total += tmp[i];
  }
  const float mean = total / (float)n;
  float sq = 0.0f;
  for (int32_t i = 0; i < n; i++) sq += (tmp[i] - mean) * (tmp[i] - mean);
  const float rstd = 1.0f / std::sqrt(sq / (float)n + eps);
  for (int32_t i = 0; i < n; i++) {
    float v = tmp[i];
    if (rv && HALF) v = halfToFloat(floatToHalf(v));
    if (sumv) store(sumv, base + i, v);
    const float g = gv ? load(gv, i) : 1.0f, b = bv ? load(bv, i) : 0.0f;
    store(outv, base + i, (v - mean) * rstd * g + b);
  }
}

template <bool HALF>
void layerNormRows(const void *x, const void *res, const void *g, const void *b, void *sum, void *out, float eps,
                   int32_t m, int32_t n) {
#pragma omp parallel
  {
    std::vector<float> tmp((size_t)(n > 0 ? n : 1));
#pragma omp for schedule(static)
    for (int32_t r = 0; r < m; r++) layerNormRow<HALF>(x, res, g, b, sum, out, eps, r, n, tmp.data());
  }
}

inline float geluErf(float x) { return 0.5f * x * std::erfc(-x * 0.70710678118654752440f); }

// out[M,N] = act(in[M,K] . w[K,N] + bias) + residual on fp32 buffers; four rows
// of the output share every weight row that streams by.
void gemmF32(const float *in, const float *w, const float *bias, const float *residual, float *out, int64_t M,
             int64_t N, int64_t K, int act) {
#pragma omp parallel for schedule(static)
  for (int64_t i0 = 0; i0 < M; i0 += 4) {
    const int64_t rows = M - i0 < 4 ? M - i0 : 4;
    float *o0 = out + i0 * N, *o1 = o0 + (rows > 1 ? N : 0), *o2 = o0 + (rows > 2 ? 2 * N : 0),
          *o3 = o0 + (rows > 3 ? 3 * N : 0);
    for (int64_t r = 0; r < rows; r++)
      for (int64_t j = 0; j < N; j++) out[(i0 + r) * N + j] = bias ? bias[j] : 0.0f;
    if (rows == 4) {
      for (int64_t k = 0; k < K; k++) {
        const float a0 = in[i0 * K + k], a1 = in[(i0 + 1) * K + k], a2 = in[(i0 + 2) * K + k], a3 = in[(i0 + 3) * K + k];
        const float *wr = w + k * N;
#pragma omp simd
        for (int64_t j = 0; j < N; j++) {
          const float wv = wr[j];
          o0[j] += a0 * wv;
          o1[j] += a1 * wv;
          o2[j] += a2 * wv;
          o3[j] += a3 * wv;
        }
      }
    } else {
      for (int64_t r = 0; r < rows; r++)
        for (int64_t k = 0; k < K; k++) {
          const float a = in[(i0 + r) * K + k];
          const float *wr = w + k * N;
          float *o = out + (i0 + r) * N;
#pragma omp simd
          for (int64_t j = 0; j < N; j++) o[j] += a * wr[j];
        }
    }
    for (int64_t r = 0; r < rows; r++) {
      float *o = out + (i0 + r) * N;
      if (act == 1)
        for (int64_t j = 0; j < N; j++) o[j] = o[j] > 0.0f ? o[j] : 0.0f;
      else if (act == 2)
        for (int64_t j = 0; j < N; j++) o[j] = geluErf(o[j]);
      if (residual)
        for (int64_t j = 0; j < N; j++) o[j] += residual[(i0 + r) * N + j];
    }
  }
}

std::vector<float> widen(const void *p, size_t n) {
  std::vector<float> f(p ? n : 0);
  if (p) mcpuCastF16ToF32(f.data(), p, n);
  return f;
}

void matmulExF16(const void *in, const void *w, const void *bias, void *out, const void *residual, int64_t M, int64_t N,
                 int64_t K, int act) {
  const std::vector<float> a = widen(in, (size_t)M * K), b = widen(w, (size_t)K * N), bi = widen(bias, (size_t)N),
                           res = widen(residual, (size_t)M * N);
  std::vector<float> o((size_t)M * N);
  gemmF32(a.data(), b.data(), bias ? bi.data() : nullptr, residual ? res.data() : nullptr, o.data(), M, N, K, act);
  mcpuCastF32ToF16(out, o.data(), (size_t)M * N);
}

} // namespace

extern "C" {

void mcpuLayerNormF16(const void *input, const void *gamma, const void *beta, void *output, float eps, int32_t m,
                      int32_t n) {
  layerNormRows<true>(input, nullptr, gamma, beta, nullptr, output, eps, m, n);
}
void mcpuAddResidualPreLayerNormF32(const float *input, const float *residual, const float *gamma, const float *beta,
                                    float *output, float *normed_output, float eps, int32_t m, int32_t n) {
  layerNormRows<false>(input, residual, gamma, beta, output, normed_output, eps, m, n);
}
void mcpuAddResidualPreLayerNormF16(const void *input, const void *residual, const void *gamma, const void *beta,
                                    void *output, void *normed_output, float eps, int32_t m, int32_t n) {
  layerNormRows<true>(input, residual, gamma, beta, output, normed_output, eps, m, n);
}

// hasRelu: 0 none, 1 ReLU, 2 GELU (erf form), as mgpuMatmulEx*.
void mcpuMatmulExF32(float *input, float *weight, float *bias, float *output, float *residual, int64_t M, int64_t N,
                     int64_t K, int32_t hasBias, int32_t hasRelu, int32_t hasResidual) {
  gemmF32(input, weight, hasBias ? bias : nullptr, hasResidual ? residual : nullptr, output, M, N, K, hasRelu);
}
void mcpuMatmulExF16(void *input, void *weight, void *bias, void *output, void *residual, int64_t M, int64_t N,
                     int64_t K, int32_t hasBias, int32_t hasRelu, int32_t hasResidual) {
  matmulExF16(input, weight, hasBias ? bias : nullptr, output, hasResidual ? residual : nullptr, M, N, K, hasRelu);
}

// Pre-LN layer with the reference's CPU signature (Kernels/CPU/Ops.h:38-43;
// lib/Kernels/CPU/LLM.cpp:176-538).  The arithmetic is that of the GPU layer of
// this build (and of the reference's GPU layer, LLM.cu:26-159): fp16 tensors
// between the stages, softmax scale 1/sqrt(d_head), causal mask when is_casual.
// The reference's own CPU graph applies neither the scale nor a mask
// (LLM.cpp:266-277); a CPU twin that is to be compared with the GPU runner
// cannot follow it there.
void mcpuLLMDecodingContextLayer(float *input, float *qkv, float *gemm_weight, float *gemm_bias, float *ffn1_weight,
                                 float *ffn1_bias, float *ffn2_weight, float *ffn2_bias, float *output, int64_t batch,
                                 int64_t seq_len, int64_t d_model, int64_t feed_forward_dim, int64_t head_num,
                                 bool norm_first, bool is_casual, bool is_relu) {
  const int64_t M = batch * seq_len, d = d_model, ffn = feed_forward_dim;
  if (M <= 0 || d <= 0 || ffn <= 0 || head_num <= 0 || d % head_num) return;
  auto half = [](const float *src, size_t n) {
    std::vector<uint16_t> h(n);
    mcpuCastF32ToF16(h.data(), src, n);
    return h;
  };
  const std::vector<uint16_t> x = half(input, (size_t)M * d), wqkv = half(qkv, (size_t)d * 3 * d),
                              wo = half(gemm_weight, (size_t)d * d), bo = half(gemm_bias, (size_t)d),
                              w1 = half(ffn1_weight, (size_t)d * ffn), b1 = half(ffn1_bias, (size_t)ffn),
                              w2 = half(ffn2_weight, (size_t)ffn * d), b2 = half(ffn2_bias, (size_t)d);
  std::vector<uint16_t> ln((size_t)M * d), packed((size_t)M * 3 * d), ctx((size_t)M * d), proj((size_t)M * d),
      y((size_t)M * d), f((size_t)M * ffn), o((size_t)M * d);
  const int64_t dh = d / head_num;
  const int act = is_relu ? 1 : 2;
  if (norm_first) { // y = x + proj(attention(LN(x))), out = y + ffn(LN(y))
    mcpuLayerNormF16(x.data(), nullptr, nullptr, ln.data(), 1e-5f, (int32_t)M, (int32_t)d);
    matmulExF16(ln.data(), wqkv.data(), nullptr, packed.data(), nullptr, M, 3 * d, d, 0);
    mcpuFusedMHAF16(packed.data(), nullptr, ctx.data(), (int32_t)batch, (int32_t)seq_len, (int32_t)head_num,
                    (int32_t)dh, 1.0f / std::sqrt((float)dh), is_casual ? 1 : 0);
    matmulExF16(ctx.data(), wo.data(), bo.data(), proj.data(), nullptr, M, d, d, 0);
    mcpuAddResidualPreLayerNormF16(proj.data(), x.data(), nullptr, nullptr, y.data(), ln.data(), 1e-5f, (int32_t)M,
                                   (int32_t)d);
    matmulExF16(ln.data(), w1.data(), b1.data(), f.data(), nullptr, M, ffn, d, act);
    matmulExF16(f.data(), w2.data(), b2.data(), o.data(), y.data(), M, d, ffn, 0);
  } else { // post-LN: h = LN(x + proj(attention(x))), out = LN(h + ffn(h))
    matmulExF16(x.data(), wqkv.data(), nullptr, packed.data(), nullptr, M, 3 * d, d, 0);
    mcpuFusedMHAF16(packed.data(), nullptr, ctx.data(), (int32_t)batch, (int32_t)seq_len, (int32_t)head_num,
                    (int32_t)dh, 1.0f / std::sqrt((float)dh), is_casual ? 1 : 0);
    matmulExF16(ctx.data(), wo.data(), bo.data(), proj.data(), nullptr, M, d, d, 0);
    mcpuAddResidualPreLayerNormF16(proj.data(), x.data(), nullptr, nullptr, ln.data(), y.data(), 1e-5f, (int32_t)M,
                                   (int32_t)d); // y = h; ln takes the rounded sum nobody reads
    matmulExF16(y.data(), w1.data(), b1.data(), f.data(), nullptr, M, ffn, d, act);
    matmulExF16(f.data(), w2.data(), b2.data(), proj.data(), nullptr, M, d, ffn, 0);
    mcpuAddResidualPreLayerNormF16(proj.data(), y.data(), nullptr, nullptr, ln.data(), o.data(), 1e-5f, (int32_t)M,
                                   (int32_t)d);
  }
  mcpuCastF16ToF32(output, o.data(), (size_t)M * d);
}

// Post-LN BERT encoder layer on fp16 tensors: CPU twin of mgpuBertEncoderLayerF16.
void mcpuBertEncoderLayerF16(const void *x, const void *wqkv, const void *bqkv, const void *wo, const void *bo,
                             const void *gamma1, const void *beta1, const void *w1, const void *b1, const void *w2,
                             const void *b2, const void *gamma2, const void *beta2, const int32_t *seqlens, void *out,
                             int64_t batch, int64_t seq_len, int64_t d_model, int64_t feed_forward_dim, int64_t head_num,
                             float eps) {
  const int64_t M = batch * seq_len, d = d_model, ffn = feed_forward_dim;
  if (M <= 0 || d <= 0 || ffn <= 0 || head_num <= 0 || d % head_num) return;
  std::vector<uint16_t> packed((size_t)M * 3 * d), ctx((size_t)M * d), proj((size_t)M * d), sum((size_t)M * d),
      h1((size_t)M * d), f((size_t)M * ffn);
  matmulExF16(x, wqkv, bqkv, packed.data(), nullptr, M, 3 * d, d, 0);
  const int64_t dh = d / head_num;
  mcpuFusedMHAF16(packed.data(), seqlens, ctx.data(), (int32_t)batch, (int32_t)seq_len, (int32_t)head_num, (int32_t)dh,
                  1.0f / std::sqrt((float)dh), 0);
  matmulExF16(ctx.data(), wo, bo, proj.data(), nullptr, M, d, d, 0);
  mcpuAddResidualPreLayerNormF16(proj.data(), x, gamma1, beta1, sum.data(), h1.data(), eps, (int32_t)M, (int32_t)d);
  matmulExF16(h1.data(), w1, b1, f.data(), nullptr, M, ffn, d, 2);
  matmulExF16(f.data(), w2, b2, proj.data(), nullptr, M, d, ffn, 0);
  mcpuAddResidualPreLayerNormF16(proj.data(), h1.data(), gamma2, beta2, sum.data(), out, eps, (int32_t)M, (int32_t)d);
}

} // extern "C"
