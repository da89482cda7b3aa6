// C++ interface of the device kernel library, under the names and argument
// order of the reference's include/multi-device-model-compiler/Kernels/GPU/Ops.h
// (:15-74) with hipStream_t in place of cudaStream_t and hipError_t in place of
// cudaError_t.  The extern "C" entry points are declared in mgpu_ops.h; this
// header adds the reference's C++-linkage functions and templates, which are
// thin wrappers over the same kernels.  On failure they print the message and
// throw std::logic_error, like lib/Kernels/GPU/Ops.cu:21-41.
#ifndef MULTI_DEVICE_MODEL_COMPILER_KERNELS_GPU_OPS_H_
#define MULTI_DEVICE_MODEL_COMPILER_KERNELS_GPU_OPS_H_

#include <cstdint>

#include <hip/hip_bfloat16.h>
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include "mgpu_ops.h"

#define MLIR_GPU_OPS_EXPORT __attribute__((visibility("default")))

MLIR_GPU_OPS_EXPORT void gpuOpsInit();      // reference Ops.h:15
MLIR_GPU_OPS_EXPORT void gpuOpsDeinit();    // :16
MLIR_GPU_OPS_EXPORT void gpuLLMOpsInit();   // :17
MLIR_GPU_OPS_EXPORT void gpuLLMOpsDeinit(); // :18

// Counterpart of checkCudaStatus (:20): prints and throws on a failed status.
MLIR_GPU_OPS_EXPORT void checkHipStatus(hipError_t status);

// Instantiated for half and float (:51-55).
template <typename T>
MLIR_GPU_OPS_EXPORT void mgpuMatmulEx(T *input, T *weight, T *bias, T *output, T *residual,
                                      int64_t M, int64_t N, int64_t K, bool hasBias, bool hasRelu,
                                      bool hasResidual, hipStream_t stream);

// Instantiated for half (as in the reference, :57-61) and also float and
// hip_bfloat16.  `scale` is accepted and ignored (int8 mode is not on this path).
template <typename T>
MLIR_GPU_OPS_EXPORT void mgpuLayerNorm(const T *input, const T *gamma, const T *beta, T *output,
                                       const float layernorm_eps, const int m, const int n,
                                       float *scale, hipStream_t stream);

// :63-68
template <typename T>
MLIR_GPU_OPS_EXPORT void
mgpuAddResidualPreLayerNorm(const T *input, const T *residual, const T *gamma, const T *beta,
                            T *output, T *normed_output, const float layernorm_eps, int m, int n,
                            float *scale, hipStream_t stream);

// :70-74, instantiated for half.
template <typename T>
MLIR_GPU_OPS_EXPORT void
mgpuAddFusedQKVBiasTranspose(T *q_buf, T *k_buf, T *v_buf, T *QKV, const T *qkv_bias,
                             const int batch_size, const int seq_len, const int token_num,
                             const int head_num, const int size_per_head, hipStream_t stream);

// No counterpart in the reference's header: there attention is reachable only
// through the dispatcher object used inside lib/Kernels/GPU/LLM.cu:79-81.
// Instantiated for half and hip_bfloat16.
template <typename T>
MLIR_GPU_OPS_EXPORT void mgpuFusedMHA(const T *qkv, const int32_t *seqlens, T *out, int B, int S,
                                      int H, int D, float scale, bool causal, hipStream_t stream);

#endif
