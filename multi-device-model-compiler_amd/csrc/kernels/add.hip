// Elementwise fp32 add at the HBM roofline.
//
// Replaces the kernel the reference's pipeline generates for onnx.Add
// (1200 blocks x 1024 threads, one scalar element per thread:
// include/multi-device-model-compiler/Dialect/Device/Transform/Passes.td:86-89)
// with 128-bit loads and non-temporal 128-bit stores, one vector per lane and one
// block per 256 vectors (the grid is sized to the array, not to the machine: blocks
// are dispatched in index order, so the device sweeps one window of memory at a time).
// One IEEE add per element: bit exact with examples/add.ll:42-66.
#include "common.hpp"
#include "mgpu_ops_internal.hpp"

namespace mgpu {

typedef float float4v __attribute__((ext_vector_type(4)));

// Each block walks UNROLL * 256 float4 per array per trip; all 2*UNROLL loads
// of a trip are issued before the first add.  Measured on MI355X at the
// (3,640,640) shape: plain loads + non-temporal stores with one vector per lane
// and one block per 256 vectors is the fastest combination (non-temporal LOADS
// cost about 10 %, more vectors per lane do not help at this size).
//
// Everything the kernel needs arrives as an explicit argument (the grid's stride included,
// instead of gridDim): the explicit arguments are preloaded into SGPRs, the grid dimensions
// would cost a load from the kernarg segment on the path to the first data load.
template <int UNROLL>
__global__ __launch_bounds__(256) void add_f32_vec4_kernel(const float4v *__restrict__ a,
                                                           const float4v *__restrict__ b,
                                                           float4v *__restrict__ c, int64_t n4, int64_t stride) {
  for (int64_t base = (int64_t)blockIdx.x * 256 * UNROLL + threadIdx.x; base < n4; base += stride) {
    float4v va[UNROLL], vb[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; u++) {
      const int64_t i = base + (int64_t)u * 256;
      if (i < n4) {
        va[u] = a[i];
        vb[u] = b[i];
      }
    }
#pragma unroll
    for (int u = 0; u < UNROLL; u++) {
      const int64_t i = base + (int64_t)u * 256;
      if (i < n4) __builtin_nontemporal_store(va[u] + vb[u], c + i);
    }
  }
}

// Tail (n % 4 elements) and the fallback for pointers that are not 16-byte
// aligned.
__global__ __launch_bounds__(256) void add_f32_scalar_kernel(const float *__restrict__ a,
                                                             const float *__restrict__ b,
                                                             float *__restrict__ c, int64_t begin,
                                                             int64_t n) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = begin + (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
    c[i] = a[i] + b[i];
}

void addF32(const float *a, const float *b, float *c, int64_t n, hipStream_t stream) {
  if (n < 0) fail("mgpuAddF32: negative element count");
  if (n == 0) return;
  if (!a || !b || !c) fail("mgpuAddF32: null pointer");
  if (aligned16(a) && aligned16(b) && aligned16(c) && n >= 4) {
    constexpr int UNROLL = 1;
    const int64_t n4 = n / 4;
    int64_t blocks = (n4 + 256 * UNROLL - 1) / (256 * UNROLL);
    const int64_t cap = kMaxStreamBlocks;
    if (blocks > cap) blocks = cap;
    add_f32_vec4_kernel<UNROLL><<<dim3((unsigned)blocks), dim3(256), 0, stream>>>(
        reinterpret_cast<const float4v *>(a), reinterpret_cast<const float4v *>(b),
        reinterpret_cast<float4v *>(c), n4, blocks * 256 * UNROLL);
    MGPU_CHECK_LAUNCH("add_f32_vec4_kernel");
    if (n % 4) {
      add_f32_scalar_kernel<<<dim3(1), dim3(64), 0, stream>>>(a, b, c, n4 * 4, n);
      MGPU_CHECK_LAUNCH("add_f32_scalar_kernel");
    }
  } else {
    int64_t blocks = (n + 255) / 256;
    const int64_t cap = kMaxStreamBlocks;
    if (blocks > cap) blocks = cap;
    add_f32_scalar_kernel<<<dim3((unsigned)blocks), dim3(256), 0, stream>>>(a, b, c, 0, n);
    MGPU_CHECK_LAUNCH("add_f32_scalar_kernel");
  }
}

} // namespace mgpu
