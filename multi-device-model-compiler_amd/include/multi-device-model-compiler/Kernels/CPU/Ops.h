// CPU op library that CPU-side model libraries call; counterpart of the
// reference's include/multi-device-model-compiler/Kernels/CPU/Ops.h:11-43
// (oneDNN there, plain C++ with OpenMP here; fp32 arithmetic, 16-bit inputs
// widened).  It is the CPU device of the runners, separate from the GPU kernel
// library: nothing on the GPU path calls it.
#ifndef MULTI_DEVICE_MODEL_COMPILER_KERNELS_CPU_OPS_H_
#define MULTI_DEVICE_MODEL_COMPILER_KERNELS_CPU_OPS_H_

#include <cstddef>
#include <cstdint>

void cpuOpsInit(bool fastMathFlag = false); // reference Ops.h:11
bool getOpsFastFlag();                      // :14
int cpuOpsNumThreads();

extern "C" {
void mcpuSetNumThreads(int32_t n);
int32_t mcpuGetNumThreads(void);
// reference Ops.h:20-22
void mcpuMatmul(float *input, float *weight, float *bias, float *output, int64_t M, int64_t N,
                int64_t K);
// CPU twins of the GPU entry points of mgpu_ops.h that have no reference name.
void mcpuConv2d(float *input, float *weight, float *bias, float *output, float *postAdd, int64_t N,
                int64_t IC, int64_t H, int64_t W, int64_t OC, int64_t KH, int64_t KW, int64_t OH,
                int64_t OW, int64_t PHL, int64_t PWL, int64_t PHR, int64_t PWR, int64_t SH, int64_t SW,
                int64_t DH, int64_t DW, bool hasPostAdd, bool hasContainRelu);
void mcpuPool2d(float *input, float *output, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OH,
                int64_t OW, int64_t KH, int64_t KW, int64_t PHL, int64_t PWL, int64_t PHR, int64_t PWR,
                int64_t SH, int64_t SW, int64_t method /* 0 - max, 1 - avg */);
void mcpuAddF32(const float *a, const float *b, float *c, int64_t n);
void mcpuLayerNormF32(const float *input, const float *gamma, const float *beta, float *output,
                      float eps, int32_t m, int32_t n);
void mcpuFusedMHAF16(const void *qkv, const int32_t *seqlens, void *out, int32_t B, int32_t S,
                     int32_t H, int32_t D, float scale, int32_t causal);
void mcpuLayerNormF16(const void *input, const void *gamma, const void *beta, void *output, float eps,
                      int32_t m, int32_t n);
void mcpuAddResidualPreLayerNormF32(const float *input, const float *residual, const float *gamma,
                                    const float *beta, float *output, float *normed_output, float eps,
                                    int32_t m, int32_t n);
void mcpuAddResidualPreLayerNormF16(const void *input, const void *residual, const void *gamma,
                                    const void *beta, void *output, void *normed_output, float eps,
                                    int32_t m, int32_t n);
void mcpuCastF32ToF16(void *dst, const float *src, size_t size);
void mcpuCastF16ToF32(float *dst, const void *src, size_t size);
void mcpuMatmulExF32(float *input, float *weight, float *bias, float *output, float *residual, int64_t M,
                     int64_t N, int64_t K, int32_t hasBias, int32_t hasRelu, int32_t hasResidual);
void mcpuMatmulExF16(void *input, void *weight, void *bias, void *output, void *residual, int64_t M,
                     int64_t N, int64_t K, int32_t hasBias, int32_t hasRelu, int32_t hasResidual);
// reference Ops.h:38-43
void mcpuLLMDecodingContextLayer(float *input, float *qkv, float *gemm_weight, float *gemm_bias,
                                 float *ffn1_weight, float *ffn1_bias, float *ffn2_weight,
                                 float *ffn2_bias, float *output, int64_t batch, int64_t seq_len,
                                 int64_t d_model, int64_t feed_forward_dim, int64_t head_num,
                                 bool norm_first, bool is_casual, bool is_relu);
void mcpuBertEncoderLayerF16(const void *x, const void *wqkv, const void *bqkv, const void *wo,
                             const void *bo, const void *gamma1, const void *beta1, const void *w1,
                             const void *b1, const void *w2, const void *b2, const void *gamma2,
                             const void *beta2, const int32_t *seqlens, void *out, int64_t batch,
                             int64_t seq_len, int64_t d_model, int64_t feed_forward_dim,
                             int64_t head_num, float eps);
}

#endif
