// 2-D convolution and pooling on NCHW fp32 tensors.
//
// Replaces mgpuConv2d and mgpuPool2d (lib/Kernels/GPU/Ops.cu:238-335,337-374;
// declared in Ops.h:27-41), which wrap cudnnConvolutionBiasActivationForward and
// cudnnPoolingForward:
//   conv:  y = act(conv(x, w) + bias[oc] + postAdd),  act = ReLU or identity
//   pool:  max (padding ignored) or average that counts the padding
//          (CUDNN_POOLING_AVERAGE_COUNT_INCLUDE_PADDING, Ops.cu:347-349)
// The convolution is an explicit GEMM: an unfold kernel writes, per image, the
// [IC*KH*KW, OH*OW] matrix of input taps (1x1 / stride 1 / no padding needs
// none: the image already is that matrix), hipBLASLt multiplies it by the
// [OC, IC*KH*KW] filter matrix straight into the NCHW output, and one
// elementwise pass adds bias and postAdd and applies the activation.  Like the
// reference (CUDNN_TENSOR_OP_MATH_ALLOW_CONVERSION, Ops.cu:254-255) the
// products may run at reduced precision on the matrix cores.  Unlike it,
// asymmetric padding is honoured (the reference passes only PHL / PWL to cuDNN).
#include "common.hpp"
#include "mgpu_ops_internal.hpp"

namespace mgpu {

namespace {

struct ConvGeo {
  int IC, H, W, KH, KW, OH, OW, PHL, PWL, SH, SW, DH, DW;
};

// col[k, p] for one image: k = (ic*KH + kh)*KW + kw, p = oh*OW + ow.
__global__ __launch_bounds__(256) void unfold_kernel(const float *__restrict__ x, float *__restrict__ col,
                                                     ConvGeo g, int64_t total) {
  const int64_t P = (int64_t)g.OH * g.OW;
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += stride) {
    const int64_t p = i % P, k = i / P;
    const int ow = (int)(p % g.OW), oh = (int)(p / g.OW);
    const int kw = (int)(k % g.KW), kh = (int)((k / g.KW) % g.KH), ic = (int)(k / ((int64_t)g.KW * g.KH));
    const int ih = oh * g.SH - g.PHL + kh * g.DH, iw = ow * g.SW - g.PWL + kw * g.DW;
    float v = 0.0f;
    if (ih >= 0 && ih < g.H && iw >= 0 && iw < g.W) v = x[((int64_t)ic * g.H + ih) * g.W + iw];
    col[i] = v;
  }
}

// y[n, c, p] = act(y + bias[c] + add[n, c, p])
__global__ __launch_bounds__(256) void conv_epilogue_kernel(float *__restrict__ y, const float *__restrict__ bias,
                                                            const float *__restrict__ add, int64_t P, int64_t OC,
                                                            int64_t total, bool relu) {
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += stride) {
    float v = y[i] + bias[(i / P) % OC];
    if (add) v += add[i];
    // cuDNN's ReLU with CUDNN_NOT_PROPAGATE_NAN maps NaN to 0, as fmaxf does
    y[i] = relu ? fmaxf(v, 0.0f) : v;
  }
}

__global__ __launch_bounds__(256) void pool_kernel(const float *__restrict__ x, float *__restrict__ y, int64_t planes,
                                                   int H, int W, int OH, int OW, int KH, int KW, int PHL, int PWL,
                                                   int SH, int SW, bool average) {
  const int64_t total = planes * OH * OW;
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += stride) {
    const int ow = (int)(i % OW), oh = (int)((i / OW) % OH);
    const float *plane = x + (i / ((int64_t)OW * OH)) * H * W;
    float acc = average ? 0.0f : -INFINITY;
    for (int kh = 0; kh < KH; kh++) {
      const int ih = oh * SH - PHL + kh;
      if (ih < 0 || ih >= H) continue;
      for (int kw = 0; kw < KW; kw++) {
        const int iw = ow * SW - PWL + kw;
        if (iw < 0 || iw >= W) continue;
        const float v = plane[(int64_t)ih * W + iw];
        acc = average ? acc + v : fmaxf(acc, v);
      }
    }
    y[i] = average ? acc / (float)(KH * KW) : acc;
  }
}

unsigned blocksFor(int64_t items) {
  int64_t blocks = (items + 255) / 256;
  if (blocks > kMaxStreamBlocks) blocks = kMaxStreamBlocks;
  return (unsigned)(blocks > 0 ? blocks : 1);
}

bool fitsInt(int64_t v) { return v >= 0 && v <= 0x7fffffff; }

} // namespace

void conv2d(const float *input, const float *weight, const float *bias, float *output, const float *postAdd,
            int64_t N, int64_t IC, int64_t H, int64_t W, int64_t OC, int64_t KH, int64_t KW, int64_t OH,
            int64_t OW, int64_t PHL, int64_t PWL, int64_t PHR, int64_t PWR, int64_t SH, int64_t SW, int64_t DH,
            int64_t DW, bool hasPostAdd, bool relu, hipStream_t stream) {
  if (N < 0 || IC <= 0 || H <= 0 || W <= 0 || OC <= 0 || KH <= 0 || KW <= 0 || OH < 0 || OW < 0)
    fail("mgpuConv2d: bad shape");
  if (PHL < 0 || PWL < 0 || PHR < 0 || PWR < 0 || SH <= 0 || SW <= 0 || DH <= 0 || DW <= 0)
    fail("mgpuConv2d: bad padding, stride or dilation");
  const int64_t spanH = H + PHL + PHR - DH * (KH - 1) - 1, spanW = W + PWL + PWR - DW * (KW - 1) - 1;
  if (spanH < 0 || spanW < 0 || OH != spanH / SH + 1 || OW != spanW / SW + 1)
    fail("mgpuConv2d: output size does not follow from input, kernel, padding, stride and dilation");
  if (N == 0) return;
  if (!input || !weight || !bias || !output) fail("mgpuConv2d: null pointer");
  if (hasPostAdd && !postAdd) fail("mgpuConv2d: hasPostAdd set but postAdd is null");
  const int64_t K = IC * KH * KW, P = OH * OW;
  for (int64_t v : {IC, H, W, OC, KH, KW, OH, OW, PHL, PWL, SH, SW, DH, DW, K, P})
    if (!fitsInt(v)) fail("mgpuConv2d: dimension too large");

  const bool direct = KH == 1 && KW == 1 && SH == 1 && SW == 1 && PHL == 0 && PWL == 0 && PHR == 0 && PWR == 0;
  float *col = nullptr;
  if (!direct) MGPU_CHECK_HIP(hipMallocAsync(reinterpret_cast<void **>(&col), (size_t)(K * P) * sizeof(float), stream));
  const ConvGeo g{(int)IC, (int)H, (int)W, (int)KH, (int)KW, (int)OH, (int)OW, (int)PHL, (int)PWL,
                  (int)SH, (int)SW, (int)DH, (int)DW};
  for (int64_t n = 0; n < N; n++) {
    const float *image = input + n * IC * H * W;
    if (!direct) {
      unfold_kernel<<<dim3(blocksFor(K * P)), dim3(256), 0, stream>>>(image, col, g, K * P);
      MGPU_CHECK_LAUNCH("unfold_kernel");
    }
    // out_n [OC, P] = filter [OC, K] . taps [K, P]
    matmulEx(DType::F32, weight, direct ? image : col, nullptr, output + n * OC * P, nullptr, OC, P, K, false,
             ACT_NONE, false, stream);
  }
  if (col) MGPU_CHECK_HIP(hipFreeAsync(col, stream));
  conv_epilogue_kernel<<<dim3(blocksFor(N * OC * P)), dim3(256), 0, stream>>>(
      output, bias, hasPostAdd ? postAdd : nullptr, P, OC, N * OC * P, relu);
  MGPU_CHECK_LAUNCH("conv_epilogue_kernel");
}

void pool2d(const float *input, float *output, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OH, int64_t OW,
            int64_t KH, int64_t KW, int64_t PHL, int64_t PWL, int64_t PHR, int64_t PWR, int64_t SH, int64_t SW,
            int64_t method, hipStream_t stream) {
  if (N < 0 || C < 0 || H <= 0 || W <= 0 || OH < 0 || OW < 0 || KH <= 0 || KW <= 0) fail("mgpuPool2d: bad shape");
  if (PHL < 0 || PWL < 0 || PHR < 0 || PWR < 0 || SH <= 0 || SW <= 0) fail("mgpuPool2d: bad padding or stride");
  if (method != 0 && method != 1) fail("mgpuPool2d: method is 0 (max) or 1 (average)");
  const int64_t spanH = H + PHL + PHR - KH, spanW = W + PWL + PWR - KW;
  if (spanH < 0 || spanW < 0 || OH != spanH / SH + 1 || OW != spanW / SW + 1)
    fail("mgpuPool2d: output size does not follow from input, kernel, padding and stride");
  if (PHL >= KH || PWL >= KW || PHR >= KH || PWR >= KW) fail("mgpuPool2d: padding must be smaller than the window");
  if (N == 0 || C == 0) return;
  if (!input || !output) fail("mgpuPool2d: null pointer");
  for (int64_t v : {H, W, OH, OW, KH, KW, PHL, PWL, SH, SW})
    if (!fitsInt(v)) fail("mgpuPool2d: dimension too large");
  pool_kernel<<<dim3(blocksFor(N * C * OH * OW)), dim3(256), 0, stream>>>(
      input, output, N * C, (int)H, (int)W, (int)OH, (int)OW, (int)KH, (int)KW, (int)PHL, (int)PWL, (int)SH, (int)SW,
      method == 1);
  MGPU_CHECK_LAUNCH("pool_kernel");
}

} // namespace mgpu
