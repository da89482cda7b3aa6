// Launcher of the fused multi-head attention kernel (fmha_kernel.hpp): picks the tile
// geometry and the instantiation for a head size and a mask, checks the operands.
//
// Replaces the dispatcher of the reference's cubin kernels, FusedMHARunnerFP16v2
// (3rdparty/trt_fused_multihead_attention/qkvToContext.cu:162-199,306-315;
// fused_multihead_attention_v2.h:5278-5377), called at lib/Kernels/GPU/LLM.cu:79-81.
#include "fmha_kernel.hpp"
#include "mgpu_ops_internal.hpp"

namespace mgpu {

namespace {

using namespace fmha_detail;

// Compute units of the current device (asked once per device).
int deviceComputeUnits() {
  static int cached[64]; // 0 = not asked yet
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  int v = __atomic_load_n(&cached[dev], __ATOMIC_RELAXED);
  if (v == 0) {
    if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || v <= 0) v = 256;
    __atomic_store_n(&cached[dev], v, __ATOMIC_RELAXED);
  }
  return v;
}

// dHead: head dimension in memory; D: the tile geometry it runs in (dHead == D, or a
// smaller multiple of 8 with the PAD instantiation).
template <typename T, int D, int NQ, bool PAD>
void launch(const void *qkv, const int32_t *seqlens, const int32_t *cuSeqlens, void *out, int B, int S, int H,
            int dHead, float scale, bool causal, hipStream_t stream) {
  constexpr int BM = 128 * NQ;
  const int nQB = (S + BM - 1) / BM;
  // Causal query blocks go in pairs of equal total work - block i with block nQB - 1 - i in one work
  // item - when there are exactly four of them (449 <= S <= 512), the head dimension is 64 or 128 (at
  // 256 the loop over the pair does not fit the registers of two wavefronts per SIMD) and the halved
  // grid still gives every CU two blocks.  Everywhere else handing the blocks out longest first (below)
  // measured as fast or faster than pairing: b16 s768 h12 d128 49.9 against 60.8 us, b2 s4096 h16 d64 84.8
  // against 92.3, b16 s640 h16 d64 28.8 against 30.6; at four blocks pairing wins by 4-12 %.
  const bool pair = causal && D <= 128 && nQB == 4 && (int64_t)B * H * 2 >= 2 * (int64_t)deviceComputeUnits();
  const int64_t blocks = (int64_t)B * H * (pair ? (nQB + 1) / 2 : nQB);
  // what the kernel is told: 1 = paired; 2 = unpaired causal blocks longest first (once compute units
  // hold more than one block); 0 = query blocks in index order
  const int order = pair ? 1 : (causal && blocks > deviceComputeUnits()) ? 2 : 0;
  if (blocks > 0x7fffffffLL) fail("fusedMHA: problem too large for one launch");
  const float c = scale * 1.44269504088896340736f;
  const auto *in = static_cast<const uint16_t *>(qkv);
  auto *o = static_cast<uint16_t *>(out);
  const dim3 grid((unsigned)blocks), block(256);
  if (causal) {
    // (the causal kernel exists with one 32-query block per wavefront only)
    if constexpr (NQ == 1)
      fmha_fwd_kernel<T, D, NQ, true, false, PAD><<<grid, block, 0, stream>>>(in, seqlens, cuSeqlens, o, S, H, nQB, c, order, (int)blocks, dHead, nullptr);
    else
      fail("fusedMHA: internal dispatch error");
  } else {
    fmha_fwd_kernel<T, D, NQ, false, false, PAD><<<grid, block, 0, stream>>>(in, seqlens, cuSeqlens, o, S, H, nQB, c, order, (int)blocks, dHead, nullptr);
  }
  MGPU_CHECK_LAUNCH("fmha_fwd_kernel");
}

template <typename T>
void launchForHeadDim(const void *qkv, const int32_t *seqlens, const int32_t *cuSeqlens, void *out, int B, int S, int H,
                      int dHead, float scale, bool causal, hipStream_t stream) {
  // One 32-query block per wavefront, except on long unmasked-or-padded sequences at
  // head_dim 64: with 64 queries per wavefront every K / V operand read from LDS feeds
  // two MFMAs and a block of 256 queries shares each tile load, which measured 3-10 %
  // faster from S = 2048 on (b16 s2048 h12, b4 s4096 h16, b1 s16384 h8) - but at 229
  // VGPRs only two wavefronts fit a SIMD, so the 256-query blocks must fill both block
  // slots of every CU, and at S = 512 or 1024 prologue and epilogue of the fewer, larger
  // blocks cost more than the loop gains (b32 s512 h12: 9 % slower).
  const bool wideBlocks = dHead == 64 && !causal && S >= 2048 &&
                          (int64_t)B * H * ((S + 255) / 256) >= 2 * (int64_t)deviceComputeUnits();
  if (wideBlocks) launch<T, 64, 2, false>(qkv, seqlens, cuSeqlens, out, B, S, H, dHead, scale, causal, stream);
  else if (dHead == 64) launch<T, 64, 1, false>(qkv, seqlens, cuSeqlens, out, B, S, H, dHead, scale, causal, stream);
  else if (dHead == 128) launch<T, 128, 1, false>(qkv, seqlens, cuSeqlens, out, B, S, H, dHead, scale, causal, stream);
  else if (dHead == 256) launch<T, 256, 1, false>(qkv, seqlens, cuSeqlens, out, B, S, H, dHead, scale, causal, stream);
  else if (dHead < 64) launch<T, 64, 1, true>(qkv, seqlens, cuSeqlens, out, B, S, H, dHead, scale, causal, stream);
  else if (dHead < 128) launch<T, 128, 1, true>(qkv, seqlens, cuSeqlens, out, B, S, H, dHead, scale, causal, stream);
  else launch<T, 256, 1, true>(qkv, seqlens, cuSeqlens, out, B, S, H, dHead, scale, causal, stream);
}

} // namespace

namespace {
void fusedMHAChecked(DType dt, const void *qkv, const int32_t *seqlens, const int32_t *cuSeqlens, void *out, int B,
                     int S, int H, int D, float scale, bool causal, hipStream_t stream) {
  if (B < 0 || S < 0 || H < 0) fail("fusedMHA: negative shape");
  // 64, 128 and 256 are the tile geometries; the other head sizes of the reference's
  // dispatcher (32, 40, 80, 144, 160; fused_multihead_attention_v2.h:4646-4673) and any
  // other multiple of 8 run in the next larger geometry with the filler masked out.
  if (D < 8 || D > 256 || D % 8) fail("fusedMHA: head_dim must be a multiple of 8 between 8 and 256");
  if (B == 0 || S == 0 || H == 0) return;
  if (!qkv || !out) fail("fusedMHA: null pointer");
  if (!aligned16(qkv) || !aligned16(out)) fail("fusedMHA: qkv and out must be 16-byte aligned");
  if (!(scale > 0.0f) || !(scale < INFINITY)) fail("fusedMHA: softmax scale must be positive and finite");
  if ((int64_t)S * 3 * H * D * 2 > 0x7fffffffLL) fail("fusedMHA: one sequence of QKV must stay below 2 GiB");
  if (dt == DType::F16) launchForHeadDim<_Float16>(qkv, seqlens, cuSeqlens, out, B, S, H, D, scale, causal, stream);
  else if (dt == DType::BF16) launchForHeadDim<bf16_t>(qkv, seqlens, cuSeqlens, out, B, S, H, D, scale, causal, stream);
  else fail("fusedMHA: element type must be fp16 or bf16");
}
} // namespace

void fusedMHA(DType dt, const void *qkv, const int32_t *seqlens, void *out, int B, int S, int H,
              int D, float scale, bool causal, hipStream_t stream) {
  fusedMHAChecked(dt, qkv, seqlens, nullptr, out, B, S, H, D, scale, causal, stream);
}

void fusedMHACuSeqlens(DType dt, const void *qkv, const int32_t *cuSeqlens, void *out, int B, int maxS, int H,
                       int D, float scale, bool causal, hipStream_t stream) {
  if (!cuSeqlens && B > 0 && maxS > 0 && H > 0) fail("fusedMHA: cu_seqlens is null");
  fusedMHAChecked(dt, qkv, nullptr, cuSeqlens, out, B, maxS, H, D, scale, causal, stream);
}

} // namespace mgpu
