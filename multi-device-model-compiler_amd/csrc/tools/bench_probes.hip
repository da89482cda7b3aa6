// Ceiling probes for bench.py --ceilings: what this device delivers to the
// simplest possible kernel of each kind, so that the fractions of the nameplate
// peaks reported for the product kernels can be read against what is reachable.
//   * a plain device copy (one 16-byte vector per lane, one block per 256
//     vectors: the geometry of the library's streaming kernels);
//   * the same copy at the grid and byte count of the headline LayerNorm
//     configuration: the cost of launching, filling and draining 1024 blocks;
//   * a loop of register-fed v_mfma_f32_32x32x16_f16 on four independent
//     accumulators, with the shader clock read inside the kernel.
// Measurement plumbing only: nothing here is part of the kernel library.
#include <hip/hip_runtime.h>

#include <cstdint>

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

__global__ __launch_bounds__(256) void probe_copy_kernel(const u32x4 *__restrict__ src, u32x4 *__restrict__ dst,
                                                          size_t vectors) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i < vectors) __builtin_nontemporal_store(src[i], dst + i);
}

// iters x 4 MFMAs per wavefront; stamps[2 * block] = shader clocks, [2 * block + 1] = constant-rate clocks
// spent by wavefront 0 of the block.
__global__ __launch_bounds__(256) void probe_mfma_kernel(float *__restrict__ sink, uint64_t *__restrict__ stamps,
                                                          int iters) {
  f16x8 a, b;
  for (int i = 0; i < 8; i++) {
    a[i] = (_Float16)(0.001f * (float)(threadIdx.x % 7 + i));
    b[i] = (_Float16)(0.002f * (float)(threadIdx.x % 5 + i));
  }
  f32x16 c0 = {}, c1 = {}, c2 = {}, c3 = {};
  const uint64_t t0 = clock64(), w0 = wall_clock64();
  for (int it = 0; it < iters; it++) {
    c0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c0, 0, 0, 0);
    c1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c1, 0, 0, 0);
    c2 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c2, 0, 0, 0);
    c3 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c3, 0, 0, 0);
  }
  float s = 0.0f;
  for (int i = 0; i < 16; i++) s += c0[i] + c1[i] + c2[i] + c3[i];
  const uint64_t t1 = clock64(), w1 = wall_clock64();
  if (s == 12345.678f) sink[0] = s; // keeps the accumulators alive
  if (threadIdx.x == 0) {
    stamps[2 * blockIdx.x] = t1 - t0;
    stamps[2 * blockIdx.x + 1] = w1 - w0;
  }
}

template <typename F> float timed(F &&launch, int steps, int warmup, hipStream_t stream) {
  for (int i = 0; i < warmup; i++) launch(i);
  if (hipStreamSynchronize(stream) != hipSuccess) return -1.0f;
  hipEvent_t e0, e1;
  if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) return -1.0f;
  (void)hipEventRecord(e0, stream);
  for (int i = 0; i < steps; i++) launch(i);
  (void)hipEventRecord(e1, stream);
  float ms = -1.0f;
  if (hipEventSynchronize(e1) != hipSuccess || hipEventElapsedTime(&ms, e0, e1) != hipSuccess) ms = -1.0f;
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  return hipGetLastError() == hipSuccess ? ms : -1.0f;
}

} // namespace

extern "C" {

// Milliseconds for `steps` copies of `bytes` (a multiple of 16) from src[i % nsets] to dst[i % nsets].
float mgpuProbeCopy(void *const *src, void *const *dst, int nsets, size_t bytes, int steps, int warmup, void *stream) {
  const size_t vectors = bytes / 16;
  const unsigned blocks = (unsigned)((vectors + 255) / 256);
  hipStream_t s = static_cast<hipStream_t>(stream);
  return timed(
      [&](int i) {
        probe_copy_kernel<<<dim3(blocks), dim3(256), 0, s>>>(static_cast<const u32x4 *>(src[i % nsets]),
                                                             static_cast<u32x4 *>(dst[i % nsets]), vectors);
      },
      steps, warmup, s);
}

// One launch of `blocks` blocks of four wavefronts, iters x 4 MFMAs each.  Returns the milliseconds
// of the launch; *shaderClocks / *constClocks receive the clocks wavefront 0 of block 0 spent in the
// loop (shader clock and the constant-rate clock); stamps must hold 2 * blocks uint64.
float mgpuProbeMfma(void *sink, void *stamps, int blocks, int iters, uint64_t *shaderClocks, uint64_t *constClocks,
                    void *stream) {
  hipStream_t s = static_cast<hipStream_t>(stream);
  const float ms = timed(
      [&](int) {
        probe_mfma_kernel<<<dim3(blocks), dim3(256), 0, s>>>(static_cast<float *>(sink), static_cast<uint64_t *>(stamps),
                                                            iters);
      },
      1, 1, s);
  uint64_t host[2] = {0, 0};
  if (hipMemcpy(host, stamps, sizeof(host), hipMemcpyDeviceToHost) != hipSuccess) return -1.0f;
  *shaderClocks = host[0];
  *constClocks = host[1];
  return ms;
}

// Rate of the constant clock behind wall_clock64(), in kHz (0 if the runtime does not say).
int mgpuProbeWallClockKHz(void) {
  int dev = 0, khz = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 0;
  if (hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, dev) != hipSuccess) return 0;
  return khz;
}

} // extern "C"
