// The attention kernel with clock stamps, for bench.py --fmha-phases: the TRACE
// instantiation of the product's kernel template (csrc/kernels/fmha_kernel.hpp), fp16,
// head_dim 64, no masks, launched with the product's own grid and arguments.
// Measurement plumbing only: nothing here is part of the kernel library.
#include "fmha_kernel.hpp"

#include <hip/hip_runtime.h>

#include <cstdint>

extern "C" {

// stamps receives ten uint64 per block (device memory; blocks = B * H * ceil(S / 128)), all
// from wavefront 0 of the block: the shader clock at block entry, when the first K/V tile has
// landed, after the last tile, after the output stores were issued; the device-wide
// constant-rate clock at entry and exit; and the shader clocks, summed over the block's tiles,
// spent waiting for a tile to land, in the score MFMAs, in the softmax and in the P.V MFMAs.
// Returns the number of blocks, or -1 on a bad argument or a failed launch.
int64_t mgpuBenchFusedMHAF16Profile(const void *qkv, void *out, int32_t B, int32_t S, int32_t H, float scale,
                                    uint64_t *stamps, void *stream) {
  if (B <= 0 || S <= 0 || H <= 0 || !qkv || !out || !stamps) return -1;
  if (((uintptr_t)qkv | (uintptr_t)out) & 15) return -1;
  const int nQB = (S + 127) / 128;
  const int64_t blocks = (int64_t)B * H * nQB;
  if (blocks > 0x7fffffffLL || (int64_t)S * 3 * H * 64 * 2 > 0x7fffffffLL) return -1;
  mgpu::fmha_detail::fmha_fwd_kernel<_Float16, 64, 1, false, true>
      <<<dim3((unsigned)blocks), dim3(256), 0, static_cast<hipStream_t>(stream)>>>(
          static_cast<const uint16_t *>(qkv), nullptr, nullptr, static_cast<uint16_t *>(out), S, H, nQB,
          scale * 1.44269504088896340736f, 0, (int)blocks, 64, stamps);
  return hipGetLastError() == hipSuccess ? blocks : -1;
}

} // extern "C"
