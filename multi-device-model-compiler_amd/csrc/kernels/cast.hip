// fp32 <-> fp16 casts, constant fills and the QKV bias + head transpose.
//
// Casts replace cudaCastFloat2Half / cudaCastHalf2Float
// (lib/Kernels/GPU/Utils.cu:38-103): the reference stages every value through
// shared memory with a fixed <<<256,256>>> launch; a cast has no reuse, so here
// each lane converts 8 elements between registers with 128-bit accesses on the
// wide side and the grid is sized to the array.  Round to nearest even.
// The transpose replaces add_fusedQKV_bias_transpose_kernel
// (lib/Kernels/GPU/Transpose.cu:5-84).
#include "common.hpp"
#include "mgpu_ops_internal.hpp"
#include "types.hpp"

namespace mgpu {

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

__global__ __launch_bounds__(256) void cast_f32_to_f16_vec8_kernel(f16x8 *__restrict__ dst,
                                                                   const f32x4 *__restrict__ src,
                                                                   size_t n8) {
  const size_t stride = (size_t)gridDim.x * 256;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n8; i += stride) {
    const f32x4 lo = src[2 * i];
    const f32x4 hi = src[2 * i + 1];
    f16x8 o;
#pragma unroll
    for (int e = 0; e < 4; e++) {
      o[e] = (_Float16)lo[e];
      o[4 + e] = (_Float16)hi[e];
    }
    __builtin_nontemporal_store(o, dst + i);
  }
}

__global__ __launch_bounds__(256) void cast_f16_to_f32_vec8_kernel(f32x4 *__restrict__ dst,
                                                                   const f16x8 *__restrict__ src,
                                                                   size_t n8) {
  const size_t stride = (size_t)gridDim.x * 256;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n8; i += stride) {
    const f16x8 v = src[i];
    f32x4 lo, hi;
#pragma unroll
    for (int e = 0; e < 4; e++) {
      lo[e] = (float)v[e];
      hi[e] = (float)v[4 + e];
    }
    __builtin_nontemporal_store(lo, dst + 2 * i);
    __builtin_nontemporal_store(hi, dst + 2 * i + 1);
  }
}

template <typename TO, typename TI>
__global__ __launch_bounds__(256) void cast_scalar_kernel(TO *__restrict__ dst,
                                                          const TI *__restrict__ src, size_t begin,
                                                          size_t n) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t i = begin + (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
    dst[i] = (TO)src[i];
}

template <typename T>
__global__ __launch_bounds__(256) void fill_kernel(T *__restrict__ dst, size_t n, T value) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) dst[i] = value;
}

unsigned gridFor(size_t items, int perBlock) {
  size_t blocks = (items + perBlock - 1) / perBlock;
  const size_t cap = (size_t)kMaxStreamBlocks;
  if (blocks > cap) blocks = cap;
  if (blocks == 0) blocks = 1;
  return (unsigned)blocks;
}

// One 16-byte vector (8 halves of one head row) per lane per trip:
// QKV [token, 3, H, D] (+ bias [3, H, D]) -> q/k/v [B, H, S, D], and the
// biased value is written back into QKV like the reference does
// (Transpose.cu:41-44).
__global__ __launch_bounds__(256) void qkv_bias_transpose_f16_kernel(
    _Float16 *__restrict__ q, _Float16 *__restrict__ k, _Float16 *__restrict__ v,
    _Float16 *__restrict__ qkv, const _Float16 *__restrict__ bias, int S, int tokens, int H,
    int D) {
  const int dv = D / 8; // vectors per head row
  const size_t total = (size_t)tokens * 3 * H * dv;
  const size_t stride = (size_t)gridDim.x * 256;
  _Float16 *const dst[3] = {q, k, v};
  for (size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x; idx < total; idx += stride) {
    const int d0 = (int)(idx % dv) * 8;
    size_t r = idx / dv;
    const int head = (int)(r % H);
    r /= H;
    const int which = (int)(r % 3);
    const int token = (int)(r / 3);
    const int b = token / S, s = token % S;
    f16x8 *src = reinterpret_cast<f16x8 *>(qkv + (((size_t)token * 3 + which) * H + head) * D + d0);
    f16x8 val = *src;
    if (bias) {
      const f16x8 bv = *reinterpret_cast<const f16x8 *>(bias + ((size_t)which * H + head) * D + d0);
#pragma unroll
      for (int e = 0; e < 8; e++) val[e] = (_Float16)((float)val[e] + (float)bv[e]);
      *src = val;
    }
    *reinterpret_cast<f16x8 *>(dst[which] + (((size_t)b * H + head) * S + s) * D + d0) = val;
  }
}

} // namespace

void castF32ToF16(void *dst, const float *src, size_t size, hipStream_t stream) {
  if (size == 0) return;
  if (!dst || !src) fail("castF32ToF16: null pointer");
  auto *d = static_cast<_Float16 *>(dst);
  size_t done = 0;
  if (aligned16(dst) && aligned16(src) && size >= 8) {
    const size_t n8 = size / 8;
    cast_f32_to_f16_vec8_kernel<<<dim3(gridFor(n8, 256)), dim3(256), 0, stream>>>(
        reinterpret_cast<f16x8 *>(d), reinterpret_cast<const f32x4 *>(src), n8);
    MGPU_CHECK_LAUNCH("cast_f32_to_f16_vec8_kernel");
    done = n8 * 8;
  }
  if (done < size) {
    cast_scalar_kernel<_Float16, float><<<dim3(gridFor(size - done, 256)), dim3(256), 0, stream>>>(
        d, src, done, size);
    MGPU_CHECK_LAUNCH("cast_scalar_kernel");
  }
}

void castF16ToF32(float *dst, const void *src, size_t size, hipStream_t stream) {
  if (size == 0) return;
  if (!dst || !src) fail("castF16ToF32: null pointer");
  auto *s = static_cast<const _Float16 *>(src);
  size_t done = 0;
  if (aligned16(dst) && aligned16(src) && size >= 8) {
    const size_t n8 = size / 8;
    cast_f16_to_f32_vec8_kernel<<<dim3(gridFor(n8, 256)), dim3(256), 0, stream>>>(
        reinterpret_cast<f32x4 *>(dst), reinterpret_cast<const f16x8 *>(s), n8);
    MGPU_CHECK_LAUNCH("cast_f16_to_f32_vec8_kernel");
    done = n8 * 8;
  }
  if (done < size) {
    cast_scalar_kernel<float, _Float16><<<dim3(gridFor(size - done, 256)), dim3(256), 0, stream>>>(
        dst, s, done, size);
    MGPU_CHECK_LAUNCH("cast_scalar_kernel");
  }
}

void fillF16(void *dst, size_t count, float value, hipStream_t stream) {
  if (count == 0) return;
  fill_kernel<_Float16><<<dim3(gridFor(count, 256)), dim3(256), 0, stream>>>(
      static_cast<_Float16 *>(dst), count, (_Float16)value);
  MGPU_CHECK_LAUNCH("fill_kernel");
}

void fillI32(int32_t *dst, size_t count, int32_t value, hipStream_t stream) {
  if (count == 0) return;
  fill_kernel<int32_t><<<dim3(gridFor(count, 256)), dim3(256), 0, stream>>>(dst, count, value);
  MGPU_CHECK_LAUNCH("fill_kernel");
}

void addFusedQKVBiasTransposeF16(void *q, void *k, void *v, void *qkv, const void *bias, int B,
                                 int S, int tokens, int H, int D, hipStream_t stream) {
  if (B < 0 || S < 0 || tokens < 0 || H < 0 || D < 0) fail("addFusedQKVBiasTranspose: negative shape");
  if (tokens == 0 || H == 0 || D == 0) return;
  if (tokens != B * S) fail("addFusedQKVBiasTranspose: token_num must equal batch_size * seq_len");
  if (D % 8) fail("addFusedQKVBiasTranspose: size_per_head must be a multiple of 8");
  if (!q || !k || !v || !qkv) fail("addFusedQKVBiasTranspose: null pointer");
  if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(qkv) || (bias && !aligned16(bias)))
    fail("addFusedQKVBiasTranspose: pointers must be 16-byte aligned");
  const size_t total = (size_t)tokens * 3 * H * (D / 8);
  qkv_bias_transpose_f16_kernel<<<dim3(gridFor(total, 256)), dim3(256), 0, stream>>>(
      static_cast<_Float16 *>(q), static_cast<_Float16 *>(k), static_cast<_Float16 *>(v),
      static_cast<_Float16 *>(qkv), static_cast<const _Float16 *>(bias), S, tokens, H, D);
  MGPU_CHECK_LAUNCH("qkv_bias_transpose_f16_kernel");
}

} // namespace mgpu

// ---- exact (erf) GELU, in place -------------------------------------------
namespace mgpu {

namespace {

__device__ __forceinline__ float gelu_erf(float x) {
  return 0.5f * x * (1.0f + erff(x * 0.70710678118654752440f));
}

__global__ __launch_bounds__(256) void gelu_f16_vec8_kernel(f16x8 *__restrict__ data, size_t n8) {
  const size_t stride = (size_t)gridDim.x * 256;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n8; i += stride) {
    f16x8 v = data[i];
#pragma unroll
    for (int e = 0; e < 8; e++) v[e] = (_Float16)gelu_erf((float)v[e]);
    data[i] = v;
  }
}

template <typename T>
__global__ __launch_bounds__(256) void gelu_scalar_kernel(T *__restrict__ data, size_t begin,
                                                          size_t n) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t i = begin + (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
    data[i] = (T)gelu_erf((float)data[i]);
}

} // namespace

void geluInPlaceF16(void *data, size_t n, hipStream_t stream) {
  if (n == 0) return;
  auto *d = static_cast<_Float16 *>(data);
  size_t done = 0;
  if (aligned16(data) && n >= 8) {
    const size_t n8 = n / 8;
    gelu_f16_vec8_kernel<<<dim3(gridFor(n8, 256)), dim3(256), 0, stream>>>(
        reinterpret_cast<f16x8 *>(d), n8);
    MGPU_CHECK_LAUNCH("gelu_f16_vec8_kernel");
    done = n8 * 8;
  }
  if (done < n) {
    gelu_scalar_kernel<_Float16><<<dim3(gridFor(n - done, 256)), dim3(256), 0, stream>>>(d, done, n);
    MGPU_CHECK_LAUNCH("gelu_scalar_kernel");
  }
}

void geluInPlaceF32(float *data, size_t n, hipStream_t stream) {
  if (n == 0) return;
  gelu_scalar_kernel<float><<<dim3(gridFor(n, 256)), dim3(256), 0, stream>>>(data, 0, n);
  MGPU_CHECK_LAUNCH("gelu_scalar_kernel");
}

} // namespace mgpu
