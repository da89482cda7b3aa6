/*
 * mgpu_ops.h - C ABI of the device kernel library (libmgpu_hip_ops.so) for one
 * MI355X: LayerNorm, fused multi-head attention, elementwise add, casts,
 * GEMM with epilogue, and the transformer layers composed from them.
 *
 * Drop-in for the kernel library the reference's compiled models call by
 * symbol name (include/multi-device-model-compiler/Kernels/GPU/Ops.h:15-74,
 * Utils.h:6-8).  The reference exports only mgpuMatmul / mgpuConv2d /
 * mgpuPool2d / mgpuLLMDecodingContextLayer as `extern "C"` (Ops.h:22-49); its
 * LayerNorm, matmulEx, cast and QKV-transpose entry points are C++ templates
 * instantiated for `half` only, and it has no standalone entry point for
 * attention, fp32 LayerNorm or add (attention is reachable only through
 * lib/Kernels/GPU/LLM.cu:79-81, add only as a compiler-generated kernel).  This
 * header gives every one of them a plain C name with the element type in the
 * suffix; the C++ header Kernels/GPU/Ops.h of this build keeps the reference's
 * template names as thin wrappers over these.
 *
 * Conventions kept from the reference:
 *  - all data pointers are DEVICE pointers owned by the caller; the functions
 *    only enqueue work on `stream` (always the last argument) and return;
 *  - every function returns void.  The reference prints and throws
 *    std::logic_error on failure (lib/Kernels/GPU/Ops.cu:21-41); a C caller
 *    cannot catch that, so the extern "C" layer prints the message to stderr,
 *    records it, and returns without launching: query it with
 *    mgpuOpsTakeLastError().  The C++ template wrappers do throw.
 *  - 16-bit element types are passed as `const void *` holding IEEE binary16
 *    ("F16") or bfloat16 ("BF16") values.
 */
#ifndef MGPU_OPS_H_
#define MGPU_OPS_H_

#include <stdbool.h>
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void *mgpuStream_t; /* hipStream_t */

/* ---- library lifetime (Ops.h:15-18; Ops.cu:43-55; LLM.cu:14-24) ------- */
/* C names for gpuOpsInit()/gpuOpsDeinit(): create the hipBLASLt handle and look
 * up the fixed scratch array of mgpuBertEncoderLayerF16NoAlloc on the current
 * device.  Everything that depends on the caller's stream (the library's
 * workspace, the layers' arena, side stream and events) is created on the first
 * call that uses that stream and returned by the Deinit call. */
void mgpuOpsInit(void);
void mgpuOpsDeinit(void);
/* Returns the message of the most recent failure on the calling thread, or
 * NULL; the message stays valid until the next failing call.  Clears it. */
const char *mgpuOpsTakeLastError(void);

/* ---- elementwise add -------------------------------------------------- */
/* c[i] = a[i] + b[i], i < n, IEEE binary32, bit exact.  Replaces the kernel
 * the reference's pipeline generates for onnx.Add and launches through
 * mgpuLaunchKernel (lib/Pipelines/MLIRToGPU.cpp:94-135,
 * lib/Dialect/Device/IR/GPUOffloadingAttr.cpp:283-304); CPU twin
 * examples/add.ll:42-66. */
void mgpuAddF32(const float *a, const float *b, float *c, int64_t n, mgpuStream_t stream);

/* ---- LayerNorm -------------------------------------------------------- */
/* output[r,:] = (input[r,:] - mean_r) * rsqrt(var_r + eps) * gamma + beta for
 * m rows of n elements (biased variance, statistics in fp32).
 * Replaces mgpuLayerNorm<T> (Ops.h:57-61; lib/Kernels/GPU/LayerNorm.cu:410-436,
 * kernel :138-260).  `scale` of the reference signature (int8 quantisation,
 * unused on this path) is dropped.  gamma and beta must be non-null.  Unlike
 * the reference any n >= 1 is accepted (the reference needs n even). */
void mgpuLayerNormF32(const float *input, const float *gamma, const float *beta, float *output,
                      float eps, int32_t m, int32_t n, mgpuStream_t stream);
void mgpuLayerNormF16(const void *input, const void *gamma, const void *beta, void *output,
                      float eps, int32_t m, int32_t n, mgpuStream_t stream);
void mgpuLayerNormBF16(const void *input, const void *gamma, const void *beta, void *output,
                       float eps, int32_t m, int32_t n, mgpuStream_t stream);

/* castOut = fp16(input) and output = LayerNorm(castOut) in one pass over fp32
 * rows: the invokeCudaCast + mgpuLayerNorm pair that opens the reference's
 * layer (lib/Kernels/GPU/LLM.cu:37-52), with the arithmetic of the two calls
 * (the statistics come from the rounded copy).
 * n a multiple of 8 up to 4096 and 16-byte aligned operands, else an error. */
void mgpuCastLayerNormF32ToF16(const float *input, const void *gamma, const void *beta, void *castOut,
                               void *output, float eps, int32_t m, int32_t n, mgpuStream_t stream);

/* output = round(fp32(input) + fp32(residual)); normed_output = LayerNorm(output)
 * with the statistics taken from the un-rounded sums.  Replaces
 * mgpuAddResidualPreLayerNorm<T> (Ops.h:63-68; LayerNorm.cu:438-466). */
void mgpuAddResidualPreLayerNormF32(const float *input, const float *residual, const float *gamma,
                                    const float *beta, float *output, float *normed_output,
                                    float eps, int32_t m, int32_t n, mgpuStream_t stream);
void mgpuAddResidualPreLayerNormF16(const void *input, const void *residual, const void *gamma,
                                    const void *beta, void *output, void *normed_output,
                                    float eps, int32_t m, int32_t n, mgpuStream_t stream);
void mgpuAddResidualPreLayerNormBF16(const void *input, const void *residual, const void *gamma,
                                     const void *beta, void *output, void *normed_output,
                                     float eps, int32_t m, int32_t n, mgpuStream_t stream);

/* ---- fused multi-head attention -------------------------------------- */
/* out[b,i,h,:] = sum_j softmax_j(scale * <q[b,i,h,:], k[b,j,h,:]>) v[b,j,h,:]
 * qkv: packed [B, S, 3, H, D]; out: [B, S, H*D]; D is a multiple of 8 between 8
 * and 256 (64, 128 and 256 are the kernel's tile geometries; the other sizes,
 * among them 32, 40, 80, 144 and 160 of the reference's kernel list,
 * fused_multihead_attention_v2.h:4646-4673, run inside the next larger one).
 * seqlens: NULL, or B int32 valid key counts (keys j >= seqlens[b] are masked
 * out; all S query rows are produced).  causal != 0 also masks j > i.
 * No score matrix is written to memory.
 * Replaces FusedMHARunnerFP16v2::setup_causal_masked_fmha + run_causal_masked_fmha
 * (3rdparty/trt_fused_multihead_attention/qkvToContext.cu:162-199,306-315) as
 * called at lib/Kernels/GPU/LLM.cu:79-81.  The reference takes b+1 prefix sums
 * (fused_multihead_attention_v2.h:63-64); this takes per-sequence lengths over
 * a padded [B, S] layout, the ...CuSeqlens entry points below take the prefix sums. */
void mgpuFusedMHAF16(const void *qkv, const int32_t *seqlens, void *out, int32_t B, int32_t S,
                     int32_t H, int32_t D, float scale, int32_t causal, mgpuStream_t stream);
void mgpuFusedMHABF16(const void *qkv, const int32_t *seqlens, void *out, int32_t B, int32_t S,
                      int32_t H, int32_t D, float scale, int32_t causal, mgpuStream_t stream);

/* The same attention on the reference's own description of the sequences
 * (fused_multihead_attention_v2.h:63-64, filled at qkvToContext.cu:162-199):
 * cu_seqlens holds B + 1 int32 prefix sums over token rows packed back to back,
 * qkv is [total, 3, H, D] and out [total, H*D] with total = cu_seqlens[B];
 * sequence b owns rows cu_seqlens[b] .. cu_seqlens[b+1]-1, attends only inside
 * itself, and max_s bounds the longest sequence: the grid is sized by it, so a
 * sequence longer than max_s is cut to its first max_s keys and ITS OUTPUT ROWS
 * BEYOND max_s ARE NOT WRITTEN (the lengths live in device memory; the call
 * does not wait to read them, so it cannot reject such a sequence - pass the
 * true maximum).  With cu_seqlens = {0, S, 2S, ...} this is the dense call. */
void mgpuFusedMHAF16CuSeqlens(const void *qkv, const int32_t *cu_seqlens, void *out, int32_t B,
                              int32_t max_s, int32_t H, int32_t D, float scale, int32_t causal,
                              mgpuStream_t stream);
void mgpuFusedMHABF16CuSeqlens(const void *qkv, const int32_t *cu_seqlens, void *out, int32_t B,
                               int32_t max_s, int32_t H, int32_t D, float scale, int32_t causal,
                               mgpuStream_t stream);

/* ---- casts (Utils.h:6-8; lib/Kernels/GPU/Utils.cu:85-103) ------------- */
void mgpuCastF32ToF16(void *dst, const float *src, size_t size, mgpuStream_t stream);
void mgpuCastF16ToF32(float *dst, const void *src, size_t size, mgpuStream_t stream);
/* bfloat16 counterparts (16-bit patterns; round to nearest even, NaN kept quiet). */
void mgpuCastF32ToBF16(void *dst, const float *src, size_t size, mgpuStream_t stream);
void mgpuCastBF16ToF32(float *dst, const void *src, size_t size, mgpuStream_t stream);

/* ---- QKV bias + transpose (Ops.h:70-74; Transpose.cu:70-84) ----------- */
/* QKV [token,3,H,D] += bias[3,H,D] in place; q/k/v_buf receive [B,H,S,D]. */
void mgpuAddFusedQKVBiasTransposeF16(void *q_buf, void *k_buf, void *v_buf, void *QKV,
                                     const void *qkv_bias, int32_t batch_size, int32_t seq_len,
                                     int32_t token_num, int32_t head_num, int32_t size_per_head,
                                     mgpuStream_t stream);
void mgpuAddFusedQKVBiasTransposeBF16(void *q_buf, void *k_buf, void *v_buf, void *QKV,
                                      const void *qkv_bias, int32_t batch_size, int32_t seq_len,
                                      int32_t token_num, int32_t head_num, int32_t size_per_head,
                                      mgpuStream_t stream);

/* ---- GEMM ------------------------------------------------------------- */
/* output[M,N] = input[M,K] . weight[K,N] + bias[N], fp32, row major
 * (Ops.h:23-25; lib/Kernels/GPU/Ops.cu:57-120). */
void mgpuMatmul(float *input, float *weight, float *bias, float *output, int64_t M, int64_t N,
                int64_t K, mgpuStream_t stream);
/* ---- convolution and pooling (NCHW fp32) ------------------------------- */
/* output[N,OC,OH,OW] = act(conv(input[N,IC,H,W], weight[OC,IC,KH,KW]) + bias[OC] + postAdd),
 * act = ReLU when hasContainRelu, identity otherwise; postAdd [N,OC,OH,OW] is
 * read only when hasPostAdd.  Same argument list as the reference
 * (Ops.h:27-33; lib/Kernels/GPU/Ops.cu:238-335).  OH / OW must follow from
 * the other arguments; right / bottom padding is honoured. */
void mgpuConv2d(float *input, float *weight, float *bias, float *output, float *postAdd, int64_t N,
                int64_t IC, int64_t H, int64_t W, int64_t OC, int64_t KH, int64_t KW, int64_t OH,
                int64_t OW, int64_t PHL, int64_t PWL, int64_t PHR, int64_t PWR, int64_t SH, int64_t SW,
                int64_t DH, int64_t DW, bool hasPostAdd, bool hasContainRelu, mgpuStream_t stream);
/* output[N,C,OH,OW] = window maximum (method 0, padding ignored) or window
 * mean counting the padding as zeros (method 1) (Ops.h:35-41; Ops.cu:337-374). */
void mgpuPool2d(float *input, float *output, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OH,
                int64_t OW, int64_t KH, int64_t KW, int64_t PHL, int64_t PWL, int64_t PHR, int64_t PWR,
                int64_t SH, int64_t SW, int64_t method, mgpuStream_t stream);

/* output = act(input . weight + bias) + residual; replaces mgpuMatmulEx<T>
 * (Ops.h:51-55; Ops.cu:134-234).  hasRelu: 0 none, 1 ReLU; hasRelu == 2 selects
 * GELU (erf form), which the reference does not have.  fp32 accumulation. */
void mgpuMatmulExF16(void *input, void *weight, void *bias, void *output, void *residual,
                     int64_t M, int64_t N, int64_t K, int32_t hasBias, int32_t hasRelu,
                     int32_t hasResidual, mgpuStream_t stream);
void mgpuMatmulExF32(float *input, float *weight, float *bias, float *output, float *residual,
                     int64_t M, int64_t N, int64_t K, int32_t hasBias, int32_t hasRelu,
                     int32_t hasResidual, mgpuStream_t stream);
void mgpuMatmulExBF16(void *input, void *weight, void *bias, void *output, void *residual,
                      int64_t M, int64_t N, int64_t K, int32_t hasBias, int32_t hasRelu,
                      int32_t hasResidual, mgpuStream_t stream);

/* mgpuMatmulEx* only enqueue: which kernel serves a shape (the library's or the
 * hand-written MFMA kernel below) comes from a table decided offline and a
 * fixed rule, never from a measurement inside this library; MGPU_GEMM_KERNEL =
 * library | mfma in the environment overrides both.  The first library GEMM on
 * a stream allocates that stream's 32 MiB workspace (hipMalloc, outside stream
 * capture; a stream first seen under capture runs an algorithm that needs no
 * workspace). */

/* The weight pre-packed once, at model load (no counterpart in the reference, whose weight is
 * [K, N] row major in every call): mgpuPackWeight16 writes the K-major copy of a 16-bit weight,
 * packed[n * K + k] = weight[k * N + n], bit for bit (fp16 or bf16; a different array from
 * weight), and mgpuMatmulExPackedF16 / BF16 are mgpuMatmulExF16 / BF16 on such a copy.  The
 * GEMM library multiplies this layout 7-35 % faster at the shapes of the benchmark layers
 * (4096 x 2304 x 768: 19 against 29 us, against 22 on the hand-written kernel), so a caller
 * whose weights do not change packs them once.  Always the library's kernel; results differ
 * from mgpuMatmulEx* in the last bit (another summation order). */
void mgpuPackWeight16(void *packed, void *weight, int64_t K, int64_t N, mgpuStream_t stream);
void mgpuMatmulExPackedF16(void *input, void *packedWeight, void *bias, void *output, void *residual,
                           int64_t M, int64_t N, int64_t K, int32_t hasBias, int32_t hasRelu,
                           int32_t hasResidual, mgpuStream_t stream);
void mgpuMatmulExPackedBF16(void *input, void *packedWeight, void *bias, void *output, void *residual,
                            int64_t M, int64_t N, int64_t K, int32_t hasBias, int32_t hasRelu,
                            int32_t hasResidual, mgpuStream_t stream);

/* The hand-written MFMA kernel that serves mgpuMatmulExF16 / BF16 where it is
 * the faster path, callable by itself (no counterpart in the reference):
 * same arguments; M a multiple of 128, N of 128 or 96, K of 32, operands
 * 16-byte aligned, anything else is an error. */
void mgpuGemmMfmaF16(void *input, void *weight, void *bias, void *output, void *residual,
                     int64_t M, int64_t N, int64_t K, int32_t hasBias, int32_t hasRelu,
                     int32_t hasResidual, mgpuStream_t stream);
void mgpuGemmMfmaBF16(void *input, void *weight, void *bias, void *output, void *residual,
                      int64_t M, int64_t N, int64_t K, int32_t hasBias, int32_t hasRelu,
                      int32_t hasResidual, mgpuStream_t stream);

/* ---- transformer layers ----------------------------------------------- */
/* Transformer layer, fp32 in/out, fp16 compute; same signature as the reference
 * (Ops.h:43-48; lib/Kernels/GPU/LLM.cu:26-159).  norm_first = true is the reference's
 * pre-LN dataflow, y = x + proj(attention(LN(x))), out = y + ffn(LN(y)); norm_first =
 * false (declared but never read by the reference's bodies) is the post-LN ordering of
 * the same blocks, h = LN(x + proj(attention(x))), out = LN(h + ffn(h)).  Both
 * LayerNorms have gamma = 1, beta = 0, eps = 1e-5, as in the reference. */
void mgpuLLMDecodingContextLayer(float *input, float *qkv, float *gemm_weight, float *gemm_bias,
                                 float *ffn1_weight, float *ffn1_bias, float *ffn2_weight,
                                 float *ffn2_bias, float *output, int64_t batch, int64_t seq_len,
                                 int64_t d_model, int64_t feed_forward_dim, int64_t head_num,
                                 bool norm_first, bool is_casual, bool is_relu,
                                 mgpuStream_t stream);

/* Opt-in cache of the layers' weights; no counterpart in the reference, which casts all seven
 * fp32 weight and bias arrays of the layer above to fp16 on every call (LLM.cu:55-57,84-90,
 * 100-106,124-130: 300 MB of memory traffic per call at d_model 2048).  After
 * mgpuLLMOpsCacheWeights(1) an array is converted the first time its (address, shape) is seen
 * and the copy is reused by every later call; the caller promises not to change a cached array
 * in place.  The copies are fp16, and a weight matrix is kept transposed ([N, K], K contiguous)
 * where the GEMM library multiplies that layout faster; mgpuBertEncoderLayerF16, whose weights
 * are fp16 already, takes such transposed copies for the GEMMs that gain from them.  Results
 * stay within the layers' tolerances but are not bit-identical to the uncached path (another
 * GEMM kernel, another summation order).  mgpuLLMOpsCacheWeights(0) waits for the device, frees
 * the copies and returns to the default.  Calls under stream capture never use the cache.  The
 * first call that meets a new array allocates (hipMalloc) a copy of its size in fp16. */
void mgpuLLMOpsCacheWeights(int32_t enable);

/* Post-LN BERT encoder layer on fp16 tensors; no counterpart in the reference
 * (its only layer entry point is the pre-LN one above):
 *   qkv = x . wqkv + bqkv                 [M, 3d] read as [B,S,3,H,64]
 *   ctx = fused MHA(qkv, seqlens)         scale 1/8, no causal mask
 *   h1  = LayerNorm(ctx . wo + bo + x)    gamma1, beta1
 *   f   = GELU_erf(h1 . w1 + b1)
 *   out = LayerNorm(f . w2 + b2 + h1)     gamma2, beta2
 * Weights are row major [in, out]; seqlens may be NULL. */
void mgpuBertEncoderLayerF16(const void *x, const void *wqkv, const void *bqkv, const void *wo,
                             const void *bo, const void *gamma1, const void *beta1, const void *w1,
                             const void *b1, const void *w2, const void *b2, const void *gamma2,
                             const void *beta2, const int32_t *seqlens, void *out, int64_t batch,
                             int64_t seq_len, int64_t d_model, int64_t feed_forward_dim,
                             int64_t head_num, float eps, mgpuStream_t stream);

/* The same layer for callers that cannot allocate device memory (code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc);
 * no counterpart in the reference.  Same arguments and results as
 * mgpuBertEncoderLayerF16, but the call allocates nothing: its temporaries
 * live in a fixed 48 MiB device array inside the library (one copy per GPU,
 * held until the process ends) and all four GEMMs run on the hand-written MFMA
 * kernel.  Limits, each an error reported through mgpuOpsTakeLastError():
 *   batch*seq_len * (max(4*d_model, feed_forward_dim) + 2*d_model) * 2 bytes
 *   must fit in 48 MiB (BERT-base (32,128,768), ffn 3072: 36 MiB);
 *   batch*seq_len a multiple of 128, d_model and feed_forward_dim multiples
 *   of 128 (or 96) and of 32, operands 16-byte aligned.
 * A rejected call enqueues nothing.  The stream must belong to the device that
 * is current when the call is made (the array's address is that device's).
 * Every call on one GPU shares that GPU's array: calls that overlap in time on
 * different streams of one GPU race; calls on one stream are ordered. */
void mgpuBertEncoderLayerF16NoAlloc(const void *x, const void *wqkv, const void *bqkv, const void *wo,
                                    const void *bo, const void *gamma1, const void *beta1,
                                    const void *w1, const void *b1, const void *w2, const void *b2,
                                    const void *gamma2, const void *beta2, const int32_t *seqlens,
                                    void *out, int64_t batch, int64_t seq_len, int64_t d_model,
                                    int64_t feed_forward_dim, int64_t head_num, float eps,
                                    mgpuStream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* MGPU_OPS_H_ */
