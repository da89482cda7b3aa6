// mgpuBertEncoderLayerF16NoAlloc: the post-LN BERT encoder layer of
// bertEncoderLayerF16 (llm.cpp) for callers that cannot allocate device memory
// (code under HIP graph capture, tight serving loops, harnesses that forbid
// hipMalloc).  The reference has no such entry point.
//
// The temporaries of the layer (packed QKV, attention context, projection,
// residual sum, first LayerNorm output, FFN activation) live in one file-scope
// device array of kNoAllocScratchBytes instead of an arena from
// hipMallocAsync.  Every device the library runs on holds its own copy of the
// array until the process ends; its address on a device is looked up once, with
// that device current, through hipGetSymbolAddress and only that address is
// ever handed to kernels, memsets or copies (the array's name in host code is
// a host-side stand-in, not a device address).
//
// All four GEMMs run on the hand-written MFMA kernel (gemm_mfma.hip): the
// library path would bring a workspace and allocating plan set-up with it.
// Nothing in the call allocates, frees or synchronises.
//
// Every call on a device shares that device's array: calls on different
// streams of one device that overlap in time race on it.  Calls on one stream
// are ordered by the stream.  Nothing has to start at zero: every temporary is
// written in full before it is read.
#include "common.hpp"
#include "mgpu_ops_internal.hpp"

#include <cmath>
#include <mutex>

namespace mgpu {

namespace {

constexpr size_t kNoAllocScratchBytes = size_t(48) << 20; // 48 MiB: (32,128,768) with ffn 3072 needs 36 MiB

static __device__ __align__(256) unsigned char scratch[kNoAllocScratchBytes];

constexpr int kMaxDevices = 64;
void *scratchAddress[kMaxDevices] = {};
std::mutex scratchAddressMutex;

// Address of `scratch` on the current device, looked up on first use there.  The caller's
// stream must belong to the current device (as for every entry point of this library: the
// kernels are launched on the stream, the scratch address is the current device's).
unsigned char *scratchOnCurrentDevice() {
  int dev = -1;
  MGPU_CHECK_HIP(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices) fail("mgpuBertEncoderLayerF16NoAlloc: device ordinal out of range");
  std::lock_guard<std::mutex> lock(scratchAddressMutex);
  if (!scratchAddress[dev]) {
    void *ptr = nullptr;
    MGPU_CHECK_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    if (!ptr) fail("mgpuBertEncoderLayerF16NoAlloc: the scratch array has no address on this device");
    scratchAddress[dev] = ptr;
  }
  return static_cast<unsigned char *>(scratchAddress[dev]);
}

inline size_t roundUp256(size_t bytes) { return (bytes + 255) & ~size_t(255); }

} // namespace

// Called by gpuLLMOpsInit for the device current at that time, so that the
// first layer call on it does not pay the lookup (and the lazy load of the
// code object it triggers) inside a capture.
void noAllocInit() { (void)scratchOnCurrentDevice(); }

size_t noAllocScratchBytes() { return kNoAllocScratchBytes; }

void bertEncoderLayerF16NoAlloc(const void *x, const void *wqkv, const void *bqkv, const void *wo, const void *bo,
                                const void *gamma1, const void *beta1, const void *w1, const void *b1, const void *w2,
                                const void *b2, const void *gamma2, const void *beta2, const int32_t *seqlens,
                                void *out, int64_t B, int64_t S, int64_t d, int64_t ffn, int64_t H, float eps,
                                hipStream_t stream) {
  const char *name = "mgpuBertEncoderLayerF16NoAlloc";
  if (B < 0 || S < 0 || d <= 0 || ffn <= 0 || H <= 0) fail(std::string(name) + ": bad shape");
  if (d % H || d / H < 8 || d / H > 256 || (d / H) % 8)
    fail(std::string(name) + ": d_model / head_num must be a multiple of 8 between 8 and 256");
  if (B == 0 || S == 0) return;
  if (!x || !wqkv || !bqkv || !wo || !bo || !gamma1 || !beta1 || !w1 || !b1 || !w2 || !b2 || !gamma2 || !beta2 || !out)
    fail(std::string(name) + ": null pointer");
  const int64_t M = B * S;
  if (M > 0x7fffffff) fail(std::string(name) + ": shape too large");
  constexpr size_t h = 2; // bytes per fp16

  // Layout: [ qkv (3d) | ctx (d) ] shares its bytes with the FFN activation
  // (ffn wide), which is written only after both are dead; then the
  // projection (reused for the FFN2 output) and the first LayerNorm output.
  // (The rounded residual sums have no reader and are not written.)
  const size_t qkvBytes = roundUp256((size_t)M * 3 * d * h), rowBytes = roundUp256((size_t)M * d * h);
  const size_t ffnBytes = roundUp256((size_t)M * ffn * h);
  const size_t headBytes = qkvBytes + rowBytes > ffnBytes ? qkvBytes + rowBytes : ffnBytes;
  const size_t need = headBytes + 2 * rowBytes;
  if (need > kNoAllocScratchBytes)
    fail(std::string(name) + ": the layer needs " + std::to_string(need) + " bytes of temporaries, the fixed scratch holds " +
         std::to_string(kNoAllocScratchBytes) + " (batch * seq_len * (max(4 * d_model, feed_forward_dim) + 2 * d_model) * 2)");

  unsigned char *base = scratchOnCurrentDevice();
  void *qkv = base, *ctx = base + qkvBytes, *f = base;
  void *proj = base + headBytes, *h1 = base + headBytes + rowBytes;

  // Everything that can reject the call is checked before the first launch, so that a rejected
  // call enqueues nothing (under capture: leaves no partial graph).
  struct Gemm {
    const void *in, *w, *bias;
    void *o;
    int64_t N, K;
    int act;
  };
  const Gemm gemms[4] = {{x, wqkv, bqkv, qkv, 3 * d, d, ACT_NONE},
                         {ctx, wo, bo, proj, d, d, ACT_NONE},
                         {h1, w1, b1, f, ffn, d, ACT_GELU},
                         {f, w2, b2, proj, d, ffn, ACT_NONE}};
  for (const Gemm &g : gemms)
    if (!gemmMfmaSupports(DType::F16, g.in, g.w, g.bias, nullptr, g.o, M, g.N, g.K))
      fail(std::string(name) + ": batch * seq_len must be a multiple of 128, every GEMM width a multiple of 128 or 96, "
                               "every depth a multiple of 32, and the operands 16-byte aligned");
  if (!aligned16(x) || !aligned16(out) || !aligned16(gamma1) || !aligned16(beta1) || !aligned16(gamma2) || !aligned16(beta2))
    fail(std::string(name) + ": x, out and the LayerNorm vectors must be 16-byte aligned");
  auto gemm = [&](const Gemm &g) { gemmMfma(DType::F16, g.in, g.w, g.bias, nullptr, g.o, M, g.N, g.K, g.act, stream); };

  gemm(gemms[0]);
  fusedMHA(DType::F16, qkv, seqlens, ctx, (int)B, (int)S, (int)H, (int)(d / H), 1.0f / sqrtf((float)(d / H)), false,
           stream);
  gemm(gemms[1]);
  layerNorm(DType::F16, proj, x, gamma1, beta1, nullptr, h1, eps, (int)M, (int)d, stream);
  gemm(gemms[2]);
  gemm(gemms[3]);
  layerNorm(DType::F16, proj, h1, gamma2, beta2, nullptr, out, eps, (int)M, (int)d, stream);
}

} // namespace mgpu
