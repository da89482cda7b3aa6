// C++ entry points behind the extern "C" layer (c_api.cpp) and the template
// wrappers of Kernels/GPU/Ops.h.  All of them enqueue on `stream` and throw
// std::logic_error (after printing) on bad arguments or a failed launch.
#pragma once

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>

namespace mgpu {

enum class DType { F32 = 0, F16 = 1, BF16 = 2 };

void addF32(const float *a, const float *b, float *c, int64_t n, hipStream_t stream);

// residual may be null (plain LayerNorm); sumOut may be null (the rounded sum is then not written).
void layerNorm(DType dt, const void *input, const void *residual, const void *gamma,
               const void *beta, void *sumOut, void *normed, float eps, int m, int n,
               hipStream_t stream);

// castOut = fp16(input), normed = LayerNorm(castOut) in one pass over fp32 rows
// (n a multiple of 8 up to 4096, 16-byte aligned operands); false, with
// nothing enqueued, for other shapes.
bool castLayerNormF32ToF16(const float *input, const void *gamma, const void *beta, void *castOut, void *normed,
                           float eps, int m, int n, hipStream_t stream);

void fusedMHA(DType dt, const void *qkv, const int32_t *seqlens, void *out, int B, int S, int H,
              int D, float scale, bool causal, hipStream_t stream);

// The reference's form of the sequence lengths: B + 1 prefix sums over token
// rows packed back to back (qkv [total, 3, H, D], out [total, H * D]); maxS
// bounds the longest sequence.
void fusedMHACuSeqlens(DType dt, const void *qkv, const int32_t *cuSeqlens, void *out, int B, int maxS, int H,
                       int D, float scale, bool causal, hipStream_t stream);

void castF32ToF16(void *dst, const float *src, size_t size, hipStream_t stream);
void castF16ToF32(float *dst, const void *src, size_t size, hipStream_t stream);
void castF32ToBF16(void *dst, const float *src, size_t size, hipStream_t stream);
void castBF16ToF32(float *dst, const void *src, size_t size, hipStream_t stream);
// dst[c][r] = src[r][c] of a row-major rows x cols matrix (fp32 -> fp16; any 16-bit type, bit for bit)
void transposeCastF32ToF16(void *dst, const float *src, int64_t rows, int64_t cols, hipStream_t stream);
void transpose16(void *dst, const void *src, int64_t rows, int64_t cols, hipStream_t stream);
void fillF16(void *dst, size_t count, float value, hipStream_t stream);
void fillI32(int32_t *dst, size_t count, int32_t value, hipStream_t stream);

void addFusedQKVBiasTranspose(DType dt, void *q, void *k, void *v, void *qkv, const void *bias, int B, int S,
                              int tokens, int H, int D, hipStream_t stream);
void addFusedQKVBiasTransposeF16(void *q, void *k, void *v, void *qkv, const void *bias, int B,
                                 int S, int tokens, int H, int D, hipStream_t stream);

enum Activation { ACT_NONE = 0, ACT_RELU = 1, ACT_GELU = 2 };
void gemmInit();
void gemmDeinit();
// weightKMajor: the weight is stored [N, K] (each output column's K values contiguous) instead of
// the ABI's [K, N]; the layers' weight cache keeps such copies, which the library multiplies
// faster.  Always served by the library.
void matmulEx(DType dt, const void *input, const void *weight, const void *bias, void *output,
              const void *residual, int64_t M, int64_t N, int64_t K, bool hasBias, int act,
              bool hasResidual, hipStream_t stream, bool weightKMajor = false);
// Should a caller that can keep a K-major copy of the weight hand that one to matmulEx for this
// problem?  (The committed table, else: wherever the library would serve the shape.)
bool gemmPrefersKMajor(DType dt, int64_t M, int64_t N, int64_t K, bool hasBias, int act, bool hasResidual);

// Hand-written MFMA GEMM (gemm_mfma.hip): fp16 / bf16, M a multiple of 128, N of
// 128 or 96, K of 32, 16-byte aligned operands; bias and residual may be null.
bool gemmMfmaSupports(DType dt, const void *in, const void *weight, const void *bias, const void *residual,
                      const void *out, int64_t M, int64_t N, int64_t K);
void gemmMfma(DType dt, const void *in, const void *weight, const void *bias, const void *residual, void *out,
              int64_t M, int64_t N, int64_t K, int act, hipStream_t stream);

void conv2d(const float *input, const float *weight, const float *bias, float *output, const float *postAdd,
            int64_t N, int64_t IC, int64_t H, int64_t W, int64_t OC, int64_t KH, int64_t KW, int64_t OH,
            int64_t OW, int64_t PHL, int64_t PWL, int64_t PHR, int64_t PWR, int64_t SH, int64_t SW, int64_t DH,
            int64_t DW, bool hasPostAdd, bool relu, hipStream_t stream);
void pool2d(const float *input, float *output, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OH, int64_t OW,
            int64_t KH, int64_t KW, int64_t PHL, int64_t PWL, int64_t PHR, int64_t PWR, int64_t SH, int64_t SW,
            int64_t method, hipStream_t stream);

void llmInit();
void llmDeinit();
// Opt-in fp16 cache of the reference layer's fp32 weights (see llm.cpp); false also drops the copies.
void llmCacheWeights(bool enable);
void decodingContextLayer(float *input, float *qkv, float *gemm_weight, float *gemm_bias,
                          float *ffn1_weight, float *ffn1_bias, float *ffn2_weight,
                          float *ffn2_bias, float *output, int64_t batch, int64_t seq_len,
                          int64_t d_model, int64_t ffn, int64_t heads, bool norm_first,
                          bool causal, bool relu, hipStream_t stream);

void bertEncoderLayerF16(const void *x, const void *wqkv, const void *bqkv, const void *wo,
                         const void *bo, const void *gamma1, const void *beta1, const void *w1,
                         const void *b1, const void *w2, const void *b2, const void *gamma2,
                         const void *beta2, const int32_t *seqlens, void *out, int64_t B,
                         int64_t S, int64_t d, int64_t ffn, int64_t H, float eps,
                         hipStream_t stream);

// The same layer with every temporary in a fixed file-scope device array
// (layer_noalloc.hip): no allocation, no library GEMM; shapes beyond the array
// or outside the hand-written GEMM's tiling are an error.
void noAllocInit();
size_t noAllocScratchBytes();
void bertEncoderLayerF16NoAlloc(const void *x, const void *wqkv, const void *bqkv, const void *wo,
                                const void *bo, const void *gamma1, const void *beta1, const void *w1,
                                const void *b1, const void *w2, const void *b2, const void *gamma2,
                                const void *beta2, const int32_t *seqlens, void *out, int64_t B,
                                int64_t S, int64_t d, int64_t ffn, int64_t H, float eps,
                                hipStream_t stream);

void geluInPlaceF16(void *data, size_t n, hipStream_t stream);
void geluInPlaceBF16(void *data, size_t n, hipStream_t stream);
void geluInPlaceF32(float *data, size_t n, hipStream_t stream);

} // namespace mgpu
