// 2-D convolution and pooling on NCHW fp32 tensors.
//
// Replaces mgpuConv2d and mgpuPool2d (lib/Kernels/GPU/Ops.cu:238-335,337-374;
// declared in Ops.h:27-41), which wrap cudnnConvolutionBiasActivationForward and
// cudnnPoolingForward:
//   conv:  y = act(conv(x, w) + bias[oc] + postAdd),  act = ReLU or identity
//   pool:  max (padding ignored) or average that counts the padding
//          (CUDNN_POOLING_AVERAGE_COUNT_INCLUDE_PADDING, Ops.cu:347-349)
// The convolution is an implicit GEMM on the fp32 matrix cores
// (v_mfma_f32_32x32x2_f32: true fp32 products, fp32 accumulation):
//   y[n][oc, p] = sum_k w[oc, k] * taps[k, p],  k = (ic, kh, kw), p = (oh, ow)
// A 256-thread block owns 64 output channels x 128 (or 64) output pixels of one
// image; its 4 wavefronts sit 2 x 2 over that tile, 32 channels x 64 (32)
// pixels each.  The tap matrix is never written to memory: per chunk of 32
// taps the block gathers its [32, pixels] slice from the image into LDS (zero
// for padding and for taps past the end; a thread keeps one pixel and walks
// a run of consecutive taps, so global reads run along image rows and the
// (ic, kh, kw) decomposition costs one division per chunk) next to the
// [64, 32] filter slice - both through registers, fetched one chunk ahead of
// the MFMAs that use them - and every lane feeds the MFMAs with one filter
// value and one tap value per instruction.  The accumulator layout puts 32 consecutive pixels of
// one channel in the 32 lanes of a register, so the epilogue (bias, postAdd,
// ReLU) writes whole 128-byte runs of the NCHW output: one pass over the
// output, none over an intermediate.  Unlike the reference, asymmetric padding
// is honoured (it passes only PHL / PWL to cuDNN).
#include "common.hpp"
#include "mgpu_ops_internal.hpp"

namespace mgpu {

namespace {

struct ConvGeo {
  int IC, H, W, KH, KW, OH, OW, PHL, PWL, SH, SW, DH, DW;
};

typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int kConvOC = 64; // output channels per block

template <int TP, int KC> // output pixels per block (128 or 64), taps staged per step
__global__ __launch_bounds__(256) void conv_mfma_kernel(const float *__restrict__ x, const float *__restrict__ w,
                                                        const float *__restrict__ bias, const float *__restrict__ add,
                                                        float *__restrict__ y, ConvGeo g, int OC, int K, int P,
                                                        int pTiles, bool relu) {
  constexpr int PJ = TP / 64; // 32-pixel accumulators per wavefront
  // +1: the 32 lanes of a filter read sit 33 words apart, one bank each
  __shared__ float filt[kConvOC][KC + 1];
  __shared__ float taps[KC][TP];

  const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
  const int l32 = lane % 32, hl = lane / 32;
  const int wm = wave / 2, wp = wave % 2;
  const int n = blockIdx.x / pTiles;
  const int p0 = (blockIdx.x % pTiles) * TP;
  const int oc0 = blockIdx.y * kConvOC;
  // block-uniform bases; everything a lane adds to them fits 32 bits (checked by the caller)
  const float *image = x + (int64_t)n * g.IC * g.H * g.W;
  const float *wtile = w + (int64_t)oc0 * K;

  // this thread's pixel for the gathers (fixed: 256 is a multiple of TP)
  const int gp = p0 + tid % TP;
  const bool gpValid = gp < P;
  const int goh = gpValid ? gp / g.OW : 0, gow = gpValid ? gp % g.OW : 0;
  // a pixel past the end gets a first row above the image for every tap: it gathers zeros
  const int ih0 = gpValid ? goh * g.SH - g.PHL : -g.KH * g.DH - 1, iw0 = gow * g.SW - g.PWL;

  f32x16 acc[PJ];
#pragma unroll
  for (int j = 0; j < PJ; j++)
#pragma unroll
    for (int i = 0; i < 16; i++) acc[j][i] = 0.0f;

  // Each chunk is fetched into registers one step ahead of its use, so the
  // global loads of chunk c+1 are in flight while the MFMAs of chunk c run.
  constexpr int FR = kConvOC * KC / 256; // filter values per thread and chunk
  constexpr int TR = KC * TP / 256;      // consecutive taps per thread and chunk
  const int tk0 = (tid / TP) * TR;            // first tap of this thread inside a chunk
  float fv[FR], tv[TR];
  auto fetch = [&](int k0) {
#pragma unroll
    for (int i = 0; i < FR; i++) { // consecutive threads along k
      const int e = tid + 256 * i;
      const int ocl = e / KC, kl = e % KC;
      // Unconditional loads from a clamped address, the value selected afterwards:
      // a load under a branch would have to land before the next one is issued.
      const bool live = oc0 + ocl < OC && k0 + kl < K;
      const float val = wtile[live ? (uint32_t)(ocl * K + k0 + kl) : 0u];
      fv[i] = live ? val : 0.0f;
    }
    // One division per chunk; from there the tap index walks like an odometer
    // and the image offset follows it with additions only.
    int k = k0 + tk0;
    int kw = k % g.KW, kh = (k / g.KW) % g.KH;
    int ih = ih0 + kh * g.DH, iw = iw0 + kw * g.DW;
    int off = ((k / (g.KW * g.KH)) * g.H + ih) * g.W + iw;
#pragma unroll
    for (int i = 0; i < TR; i++) {
      const bool inside = (unsigned)ih < (unsigned)g.H && (unsigned)iw < (unsigned)g.W && k < K;
      const float val = image[inside ? (uint32_t)off : 0u];
      tv[i] = inside ? val : 0.0f;
      k++;
      iw += g.DW;
      off += g.DW;
      if (++kw == g.KW) {
        kw = 0;
        iw = iw0;
        ih += g.DH;
        off += g.DH * g.W - g.KW * g.DW;
        if (++kh == g.KH) {
          kh = 0;
          ih = ih0;
          off += (g.H - g.KH * g.DH) * g.W;
        }
      }
    }
  };

  fetch(0);
  for (int k0 = 0; k0 < K; k0 += KC) {
    __syncthreads(); // everybody is done with the previous chunk
#pragma unroll
    for (int i = 0; i < FR; i++) {
      const int e = tid + 256 * i;
      filt[e / KC][e % KC] = fv[i];
    }
#pragma unroll
    for (int i = 0; i < TR; i++) taps[tk0 + i][tid % TP] = tv[i];
    __syncthreads();
    if (k0 + KC < K) fetch(k0 + KC);
#pragma unroll
    for (int kk = 0; kk < KC; kk += 2) {
      const float a = filt[32 * wm + l32][kk + hl];
#pragma unroll
      for (int j = 0; j < PJ; j++) {
        const float b = taps[kk + hl][wp * (TP / 2) + 32 * j + l32];
        acc[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc[j], 0, 0, 0);
      }
    }
  }

  // accumulator register r of lane l: channel 8*(r/4) + 4*(l/32) + r%4, pixel l%32
  const int ocl0 = 32 * wm + 4 * hl;        // channel of register 0 inside the tile
  const bool fullOc = oc0 + kConvOC <= OC; // uniform: no channel test inside a full tile
  const int64_t tileBase = ((int64_t)n * OC + oc0) * P + p0;
  float *ytile = y + tileBase;
  const float *atile = add ? add + tileBase : nullptr;
  const float *btile = bias + oc0;
#pragma unroll
  for (int j = 0; j < PJ; j++) {
    const int pl = wp * (TP / 2) + 32 * j + l32;
    if (p0 + pl >= P) continue;
#pragma unroll
    for (int r = 0; r < 16; r++) {
      constexpr int kRow[16] = {0, 1, 2, 3, 8, 9, 10, 11, 16, 17, 18, 19, 24, 25, 26, 27};
      const int ocl = ocl0 + kRow[r];
      if (!fullOc && oc0 + ocl >= OC) continue;
      const uint32_t off = (uint32_t)ocl * (uint32_t)P + (uint32_t)pl;
      float v = acc[j][r] + btile[ocl];
      if (atile) v += atile[off];
      // cuDNN's ReLU with CUDNN_NOT_PROPAGATE_NAN maps NaN to 0, as fmaxf does
      ytile[off] = relu ? fmaxf(v, 0.0f) : v;
    }
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
  for (int64_t v : {IC, H, W, OC, KH, KW, OH, OW, PHL, PWL, SH, SW, DH, DW, K, P, IC * H * W + (KH * DH + 1) * W + KW * DW})
    if (!fitsInt(v)) fail("mgpuConv2d: dimension too large");

  if (OH == 0 || OW == 0) return;
  const ConvGeo g{(int)IC, (int)H, (int)W, (int)KH, (int)KW, (int)OH, (int)OW, (int)PHL, (int)PWL,
                  (int)SH, (int)SW, (int)DH, (int)DW};
  const int64_t ocTiles = (OC + kConvOC - 1) / kConvOC;
  if (ocTiles > 65535) fail("mgpuConv2d: too many output channels for one launch");
  // 128-pixel tiles unless that leaves fewer than two blocks per compute unit
  const bool wide = N * ((P + 127) / 128) * ocTiles >= 512;
  const int64_t pTiles = wide ? (P + 127) / 128 : (P + 63) / 64;
  if (!fitsInt(N * pTiles)) fail("mgpuConv2d: too many output tiles for one launch");
  // lane offsets inside a block's filter and output tiles are 32-bit
  if (!fitsInt(kConvOC * K + K) || !fitsInt((kConvOC + 1) * P)) fail("mgpuConv2d: dimension too large");
  const dim3 grid((unsigned)(N * pTiles), (unsigned)ocTiles);
  const float *add = hasPostAdd ? postAdd : nullptr;
  if (wide)
    conv_mfma_kernel<128, 32><<<grid, dim3(256), 0, stream>>>(input, weight, bias, add, output, g, (int)OC, (int)K,
                                                              (int)P, (int)pTiles, relu);
  else
    conv_mfma_kernel<64, 32><<<grid, dim3(256), 0, stream>>>(input, weight, bias, add, output, g, (int)OC, (int)K,
                                                             (int)P, (int)pTiles, relu);
  MGPU_CHECK_LAUNCH("conv_mfma_kernel");
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
