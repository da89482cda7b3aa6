// Ceiling probes for bench.py --ceilings: what this device delivers to the
// simplest possible kernel of each kind, so that the fractions of the nameplate
// peaks reported for the product kernels can be read against what is reachable.
//   * a plain device copy (one 16-byte vector per lane, one block per 256
//     vectors: the geometry of the library's streaming kernels);
//   * the same copy at the grid and byte count of the headline LayerNorm
//     configuration: the cost of launching, filling and draining 1024 blocks;
//   * a loop of register-fed v_mfma_f32_32x32x16_f16 on four independent
//     accumulators, with the shader clock read inside the kernel;
//   * the instruction mix of one 64-key tile of the attention kernel at head_dim
//     64 (16 MFMAs; per score one fma, one exp2, one add, half a convert; 8
//     ds_read_b128 and 16 ds_read_b64_tr_b16 whose results nobody waits for),
//     once finely interleaved and once in the kernel's phases (scores, softmax,
//     P.V), with no barrier, no tile loads and no wait on LDS data: what a SIMD
//     can issue for that mix, in shader clocks per tile.
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

// MODE 0: MFMAs spread evenly through the softmax instructions; 1: eight MFMAs, the
// softmax, eight MFMAs, each phase fed by the one before (the product kernel's order).
template <int MODE> __global__ __launch_bounds__(256) void probe_fmha_mix_kernel(float *__restrict__ sink,
                                                                                 uint64_t *__restrict__ stamps, int tiles) {
  __shared__ __attribute__((aligned(1024))) unsigned char smem[16384];
  for (int i = threadIdx.x; i < 4096; i += 256) reinterpret_cast<uint32_t *>(smem)[i] = i;
  __syncthreads();
  const uint32_t lbase =
      (uint32_t)(uintptr_t)((__attribute__((address_space(3))) unsigned char *)smem) + (threadIdx.x % 64) * 16;
  typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
  float a[8];
  for (int i = 0; i < 8; i++) a[i] = 0.5f + 0.001f * (float)(threadIdx.x + i);
  f16x8 ma, mb;
  for (int i = 0; i < 8; i++) {
    ma[i] = (_Float16)0.01f;
    mb[i] = (_Float16)0.02f;
  }
  f32x16 c0 = {}, c1 = {};
  u32x4 ra = {0, 0, 0, 0};
  u32x2 rb = {0, 0};
  auto softmax8 = [&](int r) { // the softmax instructions of 8 scores
#pragma unroll
    for (int i = 0; i < 8; i++) {
      asm volatile("v_fma_f32 %0, %0, %0, %0\n v_exp_f32 %0, %0\n v_add_f32 %1, %1, %0" : "+v"(a[i]), "+v"(a[(i + 1) & 7]));
      if (i & 1) asm volatile("v_cvt_pk_f16_f32 %0, %0, %1" : "+v"(a[i]) : "v"(a[i - 1]));
      if (MODE == 0) {
        if (i == 0 || i == 4) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(ra) : "v"(lbase), "i"(r * 2048 + i * 128));
        if (i & 1) {
          asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(rb) : "v"(lbase), "i"(r * 2048 + i * 64));
          if (i & 2) c0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(ma, mb, c0, 0, 0, 0);
          else c1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(ma, mb, c1, 0, 0, 0);
        }
      }
    }
  };
  const uint64_t t0 = clock64();
  for (int t = 0; t < tiles; t++) {
    if (MODE == 1) {
#pragma unroll
      for (int r = 0; r < 8; r++) {
        asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(ra) : "v"(lbase), "i"(r * 1024));
        if (r & 1) c0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(ma, mb, c0, 0, 0, 0);
        else c1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(ma, mb, c1, 0, 0, 0);
      }
      a[0] += c0[0]; // the softmax starts from the scores
      a[1] += c1[0];
    }
#pragma unroll
    for (int r = 0; r < 4; r++) softmax8(r);
    if (MODE == 1) {
      ma[0] = (_Float16)a[0]; // P.V starts from the softmax
#pragma unroll
      for (int r = 0; r < 8; r++) {
        asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(rb) : "v"(lbase), "i"(r * 1024));
        asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(rb) : "v"(lbase), "i"(r * 1024 + 512));
        if (r & 1) c0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(ma, mb, c0, 0, 0, 0);
        else c1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(ma, mb, c1, 0, 0, 0);
      }
    }
  }
  asm volatile("s_waitcnt lgkmcnt(0)");
  const uint64_t t1 = clock64();
  float s = (float)(ra[0] + rb[0]);
  for (int i = 0; i < 8; i++) s += a[i];
  for (int i = 0; i < 16; i++) s += c0[i] + c1[i];
  if (s == 12345.678f) sink[0] = s;
  if (threadIdx.x == 0) stamps[blockIdx.x] = t1 - t0;
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

// Mean shader clocks per tile and wavefront of the attention instruction mix (mode 0 interleaved,
// 1 in phases) with `blocks` blocks of four wavefronts; stamps must hold `blocks` uint64.  < 0 on failure.
double mgpuProbeFmhaMix(void *sink, void *stamps, int blocks, int tiles, int mode, void *stream) {
  hipStream_t s = static_cast<hipStream_t>(stream);
  for (int rep = 0; rep < 2; rep++) {
    if (mode == 0) probe_fmha_mix_kernel<0><<<dim3(blocks), dim3(256), 0, s>>>(static_cast<float *>(sink), static_cast<uint64_t *>(stamps), tiles);
    else probe_fmha_mix_kernel<1><<<dim3(blocks), dim3(256), 0, s>>>(static_cast<float *>(sink), static_cast<uint64_t *>(stamps), tiles);
  }
  if (hipStreamSynchronize(s) != hipSuccess || hipGetLastError() != hipSuccess) return -1.0;
  uint64_t *host = new uint64_t[blocks];
  double mean = -1.0;
  if (hipMemcpy(host, stamps, sizeof(uint64_t) * blocks, hipMemcpyDeviceToHost) == hipSuccess) {
    double total = 0.0;
    for (int i = 0; i < blocks; i++) total += (double)host[i];
    mean = total / blocks / tiles;
  }
  delete[] host;
  return mean;
}

// Rate of the constant clock behind wall_clock64(), in kHz (0 if the runtime does not say).
int mgpuProbeWallClockKHz(void) {
  int dev = 0, khz = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 0;
  if (hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, dev) != hipSuccess) return 0;
  return khz;
}

} // extern "C"
