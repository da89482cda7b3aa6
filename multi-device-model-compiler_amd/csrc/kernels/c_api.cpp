// extern "C" layer of the kernel library (include/mgpu_ops.h) and the
// reference's C++ names (Kernels/GPU/Ops.h, Utils.h of this build).
//
// The C entry points catch the std::logic_error the C++ layer throws (after it
// has printed the message), remember the message for mgpuOpsTakeLastError() and
// return without launching: a C caller cannot unwind a C++ exception.
#include "mgpu_ops.h"

#include "common.hpp"
#include "mgpu_ops_internal.hpp"
#include "multi-device-model-compiler/Kernels/GPU/Ops.h"
#include "multi-device-model-compiler/Kernels/GPU/Utils.h"

#include <exception>
#include <string>

namespace {

thread_local std::string lastError;
thread_local std::string handedOut;
thread_local bool hasError = false;

template <typename F> void guarded(F &&f) noexcept {
  try {
    f();
  } catch (const std::exception &e) {
    lastError = e.what();
    hasError = true;
  } catch (...) {
    lastError = "unknown failure";
    hasError = true;
  }
}

inline hipStream_t S(mgpuStream_t s) { return reinterpret_cast<hipStream_t>(s); }

} // namespace

// ---- the reference's C++ names --------------------------------------------

void checkHipStatus(hipError_t status) { mgpu::checkHipStatus(status, "checkHipStatus"); }

void gpuLLMOpsInit() {
  mgpu::llmInit();
  mgpu::noAllocInit();
}
void gpuLLMOpsDeinit() { mgpu::llmDeinit(); }
extern "C" void mgpuLLMOpsCacheWeights(int32_t enable) {
  guarded([&] { mgpu::llmCacheWeights(enable != 0); });
}

void gpuOpsInit() {
  mgpu::gemmInit();
  gpuLLMOpsInit();
}

void gpuOpsDeinit() {
  mgpu::gemmDeinit();
  gpuLLMOpsDeinit();
}

template <typename T> struct DTypeOf;
template <> struct DTypeOf<float> { static constexpr mgpu::DType value = mgpu::DType::F32; };
template <> struct DTypeOf<half> { static constexpr mgpu::DType value = mgpu::DType::F16; };
template <> struct DTypeOf<hip_bfloat16> { static constexpr mgpu::DType value = mgpu::DType::BF16; };

template <typename T>
void mgpuMatmulEx(T *input, T *weight, T *bias, T *output, T *residual, int64_t M, int64_t N,
                  int64_t K, bool hasBias, bool hasRelu, bool hasResidual, hipStream_t stream) {
  mgpu::matmulEx(DTypeOf<T>::value, input, weight, bias, output, residual, M, N, K, hasBias,
                 hasRelu ? mgpu::ACT_RELU : mgpu::ACT_NONE, hasResidual, stream);
}
template void mgpuMatmulEx<half>(half *, half *, half *, half *, half *, int64_t, int64_t, int64_t,
                                 bool, bool, bool, hipStream_t);
template void mgpuMatmulEx<float>(float *, float *, float *, float *, float *, int64_t, int64_t,
                                  int64_t, bool, bool, bool, hipStream_t);

template <typename T>
void mgpuLayerNorm(const T *input, const T *gamma, const T *beta, T *output,
                   const float layernorm_eps, const int m, const int n, float * /*scale*/,
                   hipStream_t stream) {
  mgpu::layerNorm(DTypeOf<T>::value, input, nullptr, gamma, beta, nullptr, output, layernorm_eps, m,
                  n, stream);
}
template void mgpuLayerNorm<half>(const half *, const half *, const half *, half *, const float,
                                  const int, const int, float *, hipStream_t);
template void mgpuLayerNorm<float>(const float *, const float *, const float *, float *,
                                   const float, const int, const int, float *, hipStream_t);
template void mgpuLayerNorm<hip_bfloat16>(const hip_bfloat16 *, const hip_bfloat16 *,
                                          const hip_bfloat16 *, hip_bfloat16 *, const float,
                                          const int, const int, float *, hipStream_t);

template <typename T>
void mgpuAddResidualPreLayerNorm(const T *input, const T *residual, const T *gamma, const T *beta,
                                 T *output, T *normed_output, const float layernorm_eps, int m,
                                 int n, float * /*scale*/, hipStream_t stream) {
  if (!residual || !output) mgpu::fail("mgpuAddResidualPreLayerNorm: null pointer");
  mgpu::layerNorm(DTypeOf<T>::value, input, residual, gamma, beta, output, normed_output,
                  layernorm_eps, m, n, stream);
}
template void mgpuAddResidualPreLayerNorm<half>(const half *, const half *, const half *,
                                                const half *, half *, half *, const float, int,
                                                int, float *, hipStream_t);
template void mgpuAddResidualPreLayerNorm<float>(const float *, const float *, const float *,
                                                 const float *, float *, float *, const float, int,
                                                 int, float *, hipStream_t);
template void mgpuAddResidualPreLayerNorm<hip_bfloat16>(const hip_bfloat16 *, const hip_bfloat16 *,
                                                        const hip_bfloat16 *, const hip_bfloat16 *,
                                                        hip_bfloat16 *, hip_bfloat16 *, const float,
                                                        int, int, float *, hipStream_t);

template <typename T>
void mgpuAddFusedQKVBiasTranspose(T *q_buf, T *k_buf, T *v_buf, T *QKV, const T *qkv_bias,
                                  const int batch_size, const int seq_len, const int token_num,
                                  const int head_num, const int size_per_head, hipStream_t stream) {
  mgpu::addFusedQKVBiasTransposeF16(q_buf, k_buf, v_buf, QKV, qkv_bias, batch_size, seq_len,
                                    token_num, head_num, size_per_head, stream);
}
template void mgpuAddFusedQKVBiasTranspose<half>(half *, half *, half *, half *, const half *,
                                                 const int, const int, const int, const int,
                                                 const int, hipStream_t);

template <typename T>
void mgpuFusedMHA(const T *qkv, const int32_t *seqlens, T *out, int B, int S, int H, int D,
                  float scale, bool causal, hipStream_t stream) {
  mgpu::fusedMHA(DTypeOf<T>::value, qkv, seqlens, out, B, S, H, D, scale, causal, stream);
}
template void mgpuFusedMHA<half>(const half *, const int32_t *, half *, int, int, int, int, float,
                                 bool, hipStream_t);
template void mgpuFusedMHA<hip_bfloat16>(const hip_bfloat16 *, const int32_t *, hip_bfloat16 *, int,
                                         int, int, int, float, bool, hipStream_t);

template <>
void invokeCast<half, float>(half *dst, float const *const src, const size_t size,
                             hipStream_t stream) {
  mgpu::castF32ToF16(dst, src, size, stream);
}
template <>
void invokeCast<float, half>(float *dst, half const *const src, const size_t size,
                             hipStream_t stream) {
  mgpu::castF16ToF32(dst, src, size, stream);
}

// ---- C ABI -------------------------------------------------------------------

extern "C" {

void mgpuOpsInit(void) { guarded([] { gpuOpsInit(); }); }
void mgpuOpsDeinit(void) { guarded([] { gpuOpsDeinit(); }); }

const char *mgpuOpsTakeLastError(void) {
  if (!hasError) return nullptr;
  hasError = false;
  handedOut.swap(lastError);
  return handedOut.c_str();
}

void mgpuAddF32(const float *a, const float *b, float *c, int64_t n, mgpuStream_t stream) {
  guarded([&] { mgpu::addF32(a, b, c, n, S(stream)); });
}

void mgpuLayerNormF32(const float *input, const float *gamma, const float *beta, float *output,
                      float eps, int32_t m, int32_t n, mgpuStream_t stream) {
  guarded([&] {
    mgpu::layerNorm(mgpu::DType::F32, input, nullptr, gamma, beta, nullptr, output, eps, m, n, S(stream));
  });
}
void mgpuLayerNormF16(const void *input, const void *gamma, const void *beta, void *output,
                      float eps, int32_t m, int32_t n, mgpuStream_t stream) {
  guarded([&] {
    mgpu::layerNorm(mgpu::DType::F16, input, nullptr, gamma, beta, nullptr, output, eps, m, n, S(stream));
  });
}
void mgpuLayerNormBF16(const void *input, const void *gamma, const void *beta, void *output,
                       float eps, int32_t m, int32_t n, mgpuStream_t stream) {
  guarded([&] {
    mgpu::layerNorm(mgpu::DType::BF16, input, nullptr, gamma, beta, nullptr, output, eps, m, n, S(stream));
  });
}

static void addResidualLN(mgpu::DType dt, const void *input, const void *residual,
                          const void *gamma, const void *beta, void *output, void *normed,
                          float eps, int32_t m, int32_t n, mgpuStream_t stream) {
  guarded([&] {
    if ((!residual || !output) && m > 0 && n > 0)
      mgpu::fail("mgpuAddResidualPreLayerNorm: null pointer");
    mgpu::layerNorm(dt, input, residual, gamma, beta, output, normed, eps, m, n, S(stream));
  });
}
void mgpuCastLayerNormF32ToF16(const float *input, const void *gamma, const void *beta, void *castOut,
                               void *output, float eps, int32_t m, int32_t n, mgpuStream_t stream) {
  guarded([&] {
    if (!mgpu::castLayerNormF32ToF16(input, gamma, beta, castOut, output, eps, m, n, S(stream)))
      mgpu::fail("mgpuCastLayerNormF32ToF16: n must be a multiple of 8 up to 4096 and the operands 16-byte aligned");
  });
}
void mgpuAddResidualPreLayerNormF32(const float *input, const float *residual, const float *gamma,
                                    const float *beta, float *output, float *normed_output,
                                    float eps, int32_t m, int32_t n, mgpuStream_t stream) {
  addResidualLN(mgpu::DType::F32, input, residual, gamma, beta, output, normed_output, eps, m, n, stream);
}
void mgpuAddResidualPreLayerNormF16(const void *input, const void *residual, const void *gamma,
                                    const void *beta, void *output, void *normed_output, float eps,
                                    int32_t m, int32_t n, mgpuStream_t stream) {
  addResidualLN(mgpu::DType::F16, input, residual, gamma, beta, output, normed_output, eps, m, n, stream);
}
void mgpuAddResidualPreLayerNormBF16(const void *input, const void *residual, const void *gamma,
                                     const void *beta, void *output, void *normed_output,
                                     float eps, int32_t m, int32_t n, mgpuStream_t stream) {
  addResidualLN(mgpu::DType::BF16, input, residual, gamma, beta, output, normed_output, eps, m, n, stream);
}

void mgpuFusedMHAF16(const void *qkv, const int32_t *seqlens, void *out, int32_t B, int32_t S,
                     int32_t H, int32_t D, float scale, int32_t causal, mgpuStream_t stream) {
  guarded([&] {
    mgpu::fusedMHA(mgpu::DType::F16, qkv, seqlens, out, B, S, H, D, scale, causal != 0, reinterpret_cast<hipStream_t>(stream));
  });
}
void mgpuFusedMHABF16(const void *qkv, const int32_t *seqlens, void *out, int32_t B, int32_t S,
                      int32_t H, int32_t D, float scale, int32_t causal, mgpuStream_t stream) {
  guarded([&] {
    mgpu::fusedMHA(mgpu::DType::BF16, qkv, seqlens, out, B, S, H, D, scale, causal != 0, reinterpret_cast<hipStream_t>(stream));
  });
}

void mgpuFusedMHAF16CuSeqlens(const void *qkv, const int32_t *cu_seqlens, void *out, int32_t B, int32_t max_s,
                              int32_t H, int32_t D, float scale, int32_t causal, mgpuStream_t stream) {
  guarded([&] {
    mgpu::fusedMHACuSeqlens(mgpu::DType::F16, qkv, cu_seqlens, out, B, max_s, H, D, scale, causal != 0, S(stream));
  });
}
void mgpuFusedMHABF16CuSeqlens(const void *qkv, const int32_t *cu_seqlens, void *out, int32_t B, int32_t max_s,
                               int32_t H, int32_t D, float scale, int32_t causal, mgpuStream_t stream) {
  guarded([&] {
    mgpu::fusedMHACuSeqlens(mgpu::DType::BF16, qkv, cu_seqlens, out, B, max_s, H, D, scale, causal != 0, S(stream));
  });
}

void mgpuCastF32ToF16(void *dst, const float *src, size_t size, mgpuStream_t stream) {
  guarded([&] { mgpu::castF32ToF16(dst, src, size, S(stream)); });
}
void mgpuCastF16ToF32(float *dst, const void *src, size_t size, mgpuStream_t stream) {
  guarded([&] { mgpu::castF16ToF32(dst, src, size, S(stream)); });
}
void mgpuCastF32ToBF16(void *dst, const float *src, size_t size, mgpuStream_t stream) {
  guarded([&] { mgpu::castF32ToBF16(dst, src, size, S(stream)); });
}
void mgpuCastBF16ToF32(float *dst, const void *src, size_t size, mgpuStream_t stream) {
  guarded([&] { mgpu::castBF16ToF32(dst, src, size, S(stream)); });
}

void mgpuAddFusedQKVBiasTransposeF16(void *q_buf, void *k_buf, void *v_buf, void *QKV,
                                     const void *qkv_bias, int32_t batch_size, int32_t seq_len,
                                     int32_t token_num, int32_t head_num, int32_t size_per_head,
                                     mgpuStream_t stream) {
  guarded([&] {
    mgpu::addFusedQKVBiasTransposeF16(q_buf, k_buf, v_buf, QKV, qkv_bias, batch_size, seq_len,
                                      token_num, head_num, size_per_head, S(stream));
  });
}
void mgpuAddFusedQKVBiasTransposeBF16(void *q_buf, void *k_buf, void *v_buf, void *QKV,
                                      const void *qkv_bias, int32_t batch_size, int32_t seq_len,
                                      int32_t token_num, int32_t head_num, int32_t size_per_head,
                                      mgpuStream_t stream) {
  guarded([&] {
    mgpu::addFusedQKVBiasTranspose(mgpu::DType::BF16, q_buf, k_buf, v_buf, QKV, qkv_bias, batch_size, seq_len,
                                   token_num, head_num, size_per_head, S(stream));
  });
}

void mgpuMatmul(float *input, float *weight, float *bias, float *output, int64_t M, int64_t N,
                int64_t K, mgpuStream_t stream) {
  guarded([&] {
    mgpu::matmulEx(mgpu::DType::F32, input, weight, bias, output, nullptr, M, N, K, bias != nullptr,
                   mgpu::ACT_NONE, false, S(stream));
  });
}
void mgpuConv2d(float *input, float *weight, float *bias, float *output, float *postAdd, int64_t N,
                int64_t IC, int64_t H, int64_t W, int64_t OC, int64_t KH, int64_t KW, int64_t OH,
                int64_t OW, int64_t PHL, int64_t PWL, int64_t PHR, int64_t PWR, int64_t SH, int64_t SW,
                int64_t DH, int64_t DW, bool hasPostAdd, bool hasContainRelu, mgpuStream_t stream) {
  guarded([&] {
    mgpu::conv2d(input, weight, bias, output, postAdd, N, IC, H, W, OC, KH, KW, OH, OW, PHL, PWL, PHR, PWR,
                 SH, SW, DH, DW, hasPostAdd, hasContainRelu, S(stream));
  });
}
void mgpuPool2d(float *input, float *output, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OH,
                int64_t OW, int64_t KH, int64_t KW, int64_t PHL, int64_t PWL, int64_t PHR, int64_t PWR,
                int64_t SH, int64_t SW, int64_t method, mgpuStream_t stream) {
  guarded([&] {
    mgpu::pool2d(input, output, N, C, H, W, OH, OW, KH, KW, PHL, PWL, PHR, PWR, SH, SW, method, S(stream));
  });
}
void mgpuMatmulExF16(void *input, void *weight, void *bias, void *output, void *residual,
                     int64_t M, int64_t N, int64_t K, int32_t hasBias, int32_t hasRelu,
                     int32_t hasResidual, mgpuStream_t stream) {
  guarded([&] {
    mgpu::matmulEx(mgpu::DType::F16, input, weight, bias, output, residual, M, N, K, hasBias != 0,
                   hasRelu, hasResidual != 0, S(stream));
  });
}
void mgpuPackWeight16(void *packed, void *weight, int64_t K, int64_t N, mgpuStream_t stream) {
  guarded([&] {
    if (K < 0 || N < 0) mgpu::fail("mgpuPackWeight16: negative shape");
    if (packed == weight && K > 0 && N > 0) mgpu::fail("mgpuPackWeight16: packed and weight must be different arrays");
    mgpu::transpose16(packed, weight, K, N, S(stream));
  });
}
void mgpuMatmulExPackedF16(void *input, void *packedWeight, void *bias, void *output, void *residual,
                           int64_t M, int64_t N, int64_t K, int32_t hasBias, int32_t hasRelu,
                           int32_t hasResidual, mgpuStream_t stream) {
  guarded([&] {
    mgpu::matmulEx(mgpu::DType::F16, input, packedWeight, bias, output, residual, M, N, K, hasBias != 0,
                   hasRelu, hasResidual != 0, S(stream), true);
  });
}
void mgpuMatmulExPackedBF16(void *input, void *packedWeight, void *bias, void *output, void *residual,
                            int64_t M, int64_t N, int64_t K, int32_t hasBias, int32_t hasRelu,
                            int32_t hasResidual, mgpuStream_t stream) {
  guarded([&] {
    mgpu::matmulEx(mgpu::DType::BF16, input, packedWeight, bias, output, residual, M, N, K, hasBias != 0,
                   hasRelu, hasResidual != 0, S(stream), true);
  });
}
static void gemmMfmaChecked(mgpu::DType dt, void *input, void *weight, void *bias, void *output, void *residual,
                            int64_t M, int64_t N, int64_t K, int32_t hasBias, int32_t act, int32_t hasResidual,
                            hipStream_t stream) {
  if (!input || !weight || !output) mgpu::fail("gemmMfma: null pointer");
  if (hasBias && !bias) mgpu::fail("gemmMfma: hasBias set but bias is null");
  if (hasResidual && !residual) mgpu::fail("gemmMfma: hasResidual set but residual is null");
  if (act < mgpu::ACT_NONE || act > mgpu::ACT_GELU) mgpu::fail("gemmMfma: unknown activation");
  mgpu::gemmMfma(dt, input, weight, hasBias ? bias : nullptr, hasResidual ? residual : nullptr, output, M, N, K, act,
                 stream);
}
void mgpuGemmMfmaF16(void *input, void *weight, void *bias, void *output, void *residual, int64_t M, int64_t N,
                     int64_t K, int32_t hasBias, int32_t hasRelu, int32_t hasResidual, mgpuStream_t stream) {
  guarded([&] {
    gemmMfmaChecked(mgpu::DType::F16, input, weight, bias, output, residual, M, N, K, hasBias, hasRelu, hasResidual,
                    S(stream));
  });
}
void mgpuGemmMfmaBF16(void *input, void *weight, void *bias, void *output, void *residual, int64_t M, int64_t N,
                      int64_t K, int32_t hasBias, int32_t hasRelu, int32_t hasResidual, mgpuStream_t stream) {
  guarded([&] {
    gemmMfmaChecked(mgpu::DType::BF16, input, weight, bias, output, residual, M, N, K, hasBias, hasRelu, hasResidual,
                    S(stream));
  });
}
void mgpuMatmulExBF16(void *input, void *weight, void *bias, void *output, void *residual,
                      int64_t M, int64_t N, int64_t K, int32_t hasBias, int32_t hasRelu,
                      int32_t hasResidual, mgpuStream_t stream) {
  guarded([&] {
    mgpu::matmulEx(mgpu::DType::BF16, input, weight, bias, output, residual, M, N, K, hasBias != 0,
                   hasRelu, hasResidual != 0, S(stream));
  });
}
void mgpuMatmulExF32(float *input, float *weight, float *bias, float *output, float *residual,
                     int64_t M, int64_t N, int64_t K, int32_t hasBias, int32_t hasRelu,
                     int32_t hasResidual, mgpuStream_t stream) {
  guarded([&] {
    mgpu::matmulEx(mgpu::DType::F32, input, weight, bias, output, residual, M, N, K, hasBias != 0,
                   hasRelu, hasResidual != 0, S(stream));
  });
}

void mgpuLLMDecodingContextLayer(float *input, float *qkv, float *gemm_weight, float *gemm_bias,
                                 float *ffn1_weight, float *ffn1_bias, float *ffn2_weight,
                                 float *ffn2_bias, float *output, int64_t batch, int64_t seq_len,
                                 int64_t d_model, int64_t feed_forward_dim, int64_t head_num,
                                 bool norm_first, bool is_casual, bool is_relu,
                                 mgpuStream_t stream) {
  guarded([&] {
    mgpu::decodingContextLayer(input, qkv, gemm_weight, gemm_bias, ffn1_weight, ffn1_bias,
                               ffn2_weight, ffn2_bias, output, batch, seq_len, d_model,
                               feed_forward_dim, head_num, norm_first, is_casual, is_relu,
                               S(stream));
  });
}

void mgpuBertEncoderLayerF16(const void *x, const void *wqkv, const void *bqkv, const void *wo,
                             const void *bo, const void *gamma1, const void *beta1, const void *w1,
                             const void *b1, const void *w2, const void *b2, const void *gamma2,
                             const void *beta2, const int32_t *seqlens, void *out, int64_t batch,
                             int64_t seq_len, int64_t d_model, int64_t feed_forward_dim,
                             int64_t head_num, float eps, mgpuStream_t stream) {
  guarded([&] {
    mgpu::bertEncoderLayerF16(x, wqkv, bqkv, wo, bo, gamma1, beta1, w1, b1, w2, b2, gamma2, beta2,
                              seqlens, out, batch, seq_len, d_model, feed_forward_dim, head_num,
                              eps, S(stream));
  });
}

void mgpuBertEncoderLayerF16NoAlloc(const void *x, const void *wqkv, const void *bqkv, const void *wo,
                                    const void *bo, const void *gamma1, const void *beta1, const void *w1,
                                    const void *b1, const void *w2, const void *b2, const void *gamma2,
                                    const void *beta2, const int32_t *seqlens, void *out, int64_t batch,
                                    int64_t seq_len, int64_t d_model, int64_t feed_forward_dim,
                                    int64_t head_num, float eps, mgpuStream_t stream) {
  guarded([&] {
    mgpu::bertEncoderLayerF16NoAlloc(x, wqkv, bqkv, wo, bo, gamma1, beta1, w1, b1, w2, b2, gamma2, beta2,
                                     seqlens, out, batch, seq_len, d_model, feed_forward_dim, head_num,
                                     eps, S(stream));
  });
}

} // extern "C"
