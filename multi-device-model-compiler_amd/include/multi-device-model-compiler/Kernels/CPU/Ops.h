// CPU op library that CPU-side model libraries call; counterpart of the
// reference's include/multi-device-model-compiler/Kernels/CPU/Ops.h:11-43
// (oneDNN there, plain C++ with OpenMP here; fp32 arithmetic, 16-bit inputs
// widened).  It is the CPU device of the runners, separate from the GPU kernel
// library: nothing on the GPU path calls it.
#ifndef MULTI_DEVICE_MODEL_COMPILER_KERNELS_CPU_OPS_H_
#define MULTI_DEVICE_MODEL_COMPILER_KERNELS_CPU_OPS_H_

#include <cstdint>

void cpuOpsInit(bool fastMathFlag = false); // reference Ops.h:11
bool getOpsFastFlag();                      // :14
int cpuOpsNumThreads();

extern "C" {
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
}

#endif
