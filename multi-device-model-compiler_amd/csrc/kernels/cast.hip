// fp32 <-> fp16 / bf16 casts, constant fills, the QKV bias + head transpose and GELU.
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

// T is the 16-bit type (_Float16 or bf16_t); its vectors travel as 16 raw bytes.
// (The grid's stride is an explicit argument: explicit arguments are preloaded into SGPRs,
// gridDim would be a load from the kernarg segment in front of the first data load.)
template <typename T>
__global__ __launch_bounds__(256) void cast_f32_to_h_vec8_kernel(u32x4 *__restrict__ dst,
                                                                 const f32x4 *__restrict__ src, size_t n8,
                                                                 size_t stride) {
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n8; i += stride) {
    const f32x4 lo = src[2 * i];
    const f32x4 hi = src[2 * i + 1];
    const float v[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    __builtin_nontemporal_store(ElemTraits<T>::pack(v), dst + i);
  }
}

template <typename T>
__global__ __launch_bounds__(256) void cast_h_to_f32_vec8_kernel(f32x4 *__restrict__ dst,
                                                                 const u32x4 *__restrict__ src, size_t n8,
                                                                 size_t stride) {
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n8; i += stride) {
    float v[8];
    ElemTraits<T>::unpack(src[i], v);
    __builtin_nontemporal_store(f32x4{v[0], v[1], v[2], v[3]}, dst + 2 * i);
    __builtin_nontemporal_store(f32x4{v[4], v[5], v[6], v[7]}, dst + 2 * i + 1);
  }
}

template <typename TO, typename TI>
__global__ __launch_bounds__(256) void cast_scalar_kernel(TO *__restrict__ dst,
                                                          const TI *__restrict__ src, size_t begin,
                                                          size_t n) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t i = begin + (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
    dst[i] = ElemTraits<TO>::fromFloat(ElemTraits<TI>::toFloat(src[i]));
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
template <typename T>
__global__ __launch_bounds__(256) void qkv_bias_transpose_kernel(T *__restrict__ q, T *__restrict__ k,
                                                                 T *__restrict__ v, T *__restrict__ qkv,
                                                                 const T *__restrict__ bias, int S, int tokens,
                                                                 int H, int D) {
  const int dv = D / 8; // vectors per head row
  const size_t total = (size_t)tokens * 3 * H * dv;
  const size_t stride = (size_t)gridDim.x * 256;
  T *const dst[3] = {q, k, v};
  for (size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x; idx < total; idx += stride) {
    const int d0 = (int)(idx % dv) * 8;
    size_t r = idx / dv;
    const int head = (int)(r % H);
    r /= H;
    const int which = (int)(r % 3);
    const int token = (int)(r / 3);
    const int b = token / S, s = token % S;
    u32x4 *src = reinterpret_cast<u32x4 *>(qkv + (((size_t)token * 3 + which) * H + head) * D + d0);
    u32x4 val = *src;
    if (bias) {
      float x[8], bv[8];
      ElemTraits<T>::unpack(val, x);
      ElemTraits<T>::unpack(*reinterpret_cast<const u32x4 *>(bias + ((size_t)which * H + head) * D + d0), bv);
#pragma unroll
      for (int e = 0; e < 8; e++) x[e] += bv[e];
      val = ElemTraits<T>::pack(x);
      *src = val;
    }
    *reinterpret_cast<u32x4 *>(dst[which] + (((size_t)b * H + head) * S + s) * D + d0) = val;
  }
}

} // namespace

namespace {

template <typename T>
void castFromF32(void *dst, const float *src, size_t size, hipStream_t stream, const char *what) {
  if (size == 0) return;
  if (!dst || !src) fail(std::string(what) + ": null pointer");
  auto *d = static_cast<T *>(dst);
  size_t done = 0;
  if (aligned16(dst) && aligned16(src) && size >= 8) {
    const size_t n8 = size / 8;
    const unsigned blocks = gridFor(n8, 256);
    cast_f32_to_h_vec8_kernel<T><<<dim3(blocks), dim3(256), 0, stream>>>(
        reinterpret_cast<u32x4 *>(d), reinterpret_cast<const f32x4 *>(src), n8, (size_t)blocks * 256);
    MGPU_CHECK_LAUNCH("cast_f32_to_h_vec8_kernel");
    done = n8 * 8;
  }
  if (done < size) {
    cast_scalar_kernel<T, float><<<dim3(gridFor(size - done, 256)), dim3(256), 0, stream>>>(d, src, done, size);
    MGPU_CHECK_LAUNCH("cast_scalar_kernel");
  }
}

template <typename T>
void castToF32(float *dst, const void *src, size_t size, hipStream_t stream, const char *what) {
  if (size == 0) return;
  if (!dst || !src) fail(std::string(what) + ": null pointer");
  auto *s = static_cast<const T *>(src);
  size_t done = 0;
  if (aligned16(dst) && aligned16(src) && size >= 8) {
    const size_t n8 = size / 8;
    const unsigned blocks = gridFor(n8, 256);
    cast_h_to_f32_vec8_kernel<T><<<dim3(blocks), dim3(256), 0, stream>>>(
        reinterpret_cast<f32x4 *>(dst), reinterpret_cast<const u32x4 *>(s), n8, (size_t)blocks * 256);
    MGPU_CHECK_LAUNCH("cast_h_to_f32_vec8_kernel");
    done = n8 * 8;
  }
  if (done < size) {
    cast_scalar_kernel<float, T><<<dim3(gridFor(size - done, 256)), dim3(256), 0, stream>>>(dst, s, done, size);
    MGPU_CHECK_LAUNCH("cast_scalar_kernel");
  }
}


// dst[c][r] = T(src[r][c]) for a row-major rows x cols matrix: 64 x 64 tiles through LDS (one
// padding column against bank conflicts), coalesced on both sides.  Runs once per weight array
// (the weight cache of the layers), so it is written for clarity, not for the last GB/s.
template <typename TO, typename TI>
__global__ __launch_bounds__(256) void transpose_cast_kernel(TO *__restrict__ dst, const TI *__restrict__ src,
                                                             int64_t rows, int64_t cols) {
  __shared__ float tile[64][65];
  const int64_t r0 = (int64_t)blockIdx.y * 64, c0 = (int64_t)blockIdx.x * 64;
  const int tx = threadIdx.x % 64, ty = threadIdx.x / 64;
  for (int i = ty; i < 64; i += 4)
    if (r0 + i < rows && c0 + tx < cols) tile[i][tx] = (float)src[(r0 + i) * cols + c0 + tx];
  __syncthreads();
  for (int i = ty; i < 64; i += 4)
    if (c0 + i < cols && r0 + tx < rows) dst[(c0 + i) * rows + r0 + tx] = (TO)tile[tx][i];
}

} // namespace

void castF32ToF16(void *dst, const float *src, size_t size, hipStream_t stream) {
  castFromF32<_Float16>(dst, src, size, stream, "castF32ToF16");
}
void castF16ToF32(float *dst, const void *src, size_t size, hipStream_t stream) {
  castToF32<_Float16>(dst, src, size, stream, "castF16ToF32");
}
void castF32ToBF16(void *dst, const float *src, size_t size, hipStream_t stream) {
  castFromF32<bf16_t>(dst, src, size, stream, "castF32ToBF16");
}
void castBF16ToF32(float *dst, const void *src, size_t size, hipStream_t stream) {
  castToF32<bf16_t>(dst, src, size, stream, "castBF16ToF32");
}

void transposeCastF32ToF16(void *dst, const float *src, int64_t rows, int64_t cols, hipStream_t stream) {
  if (rows <= 0 || cols <= 0) return;
  if (!dst || !src) fail("transposeCastF32ToF16: null pointer");
  const dim3 grid((unsigned)((cols + 63) / 64), (unsigned)((rows + 63) / 64));
  if ((rows + 63) / 64 > 65535) fail("transposeCastF32ToF16: more than 4194240 rows");
  transpose_cast_kernel<_Float16, float><<<grid, dim3(256), 0, stream>>>(static_cast<_Float16 *>(dst), src, rows, cols);
  MGPU_CHECK_LAUNCH("transpose_cast_kernel");
}
void transpose16(void *dst, const void *src, int64_t rows, int64_t cols, hipStream_t stream) {
  if (rows <= 0 || cols <= 0) return;
  if (!dst || !src) fail("transpose16: null pointer");
  const dim3 grid((unsigned)((cols + 63) / 64), (unsigned)((rows + 63) / 64));
  if ((rows + 63) / 64 > 65535) fail("transpose16: more than 4194240 rows");
  // as 16-bit patterns (exact through the tile's floats): fp16 and bf16 alike, NaN payloads kept
  transpose_cast_kernel<uint16_t, uint16_t><<<grid, dim3(256), 0, stream>>>(static_cast<uint16_t *>(dst),
                                                                        static_cast<const uint16_t *>(src), rows, cols);
  MGPU_CHECK_LAUNCH("transpose_cast_kernel");
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

void addFusedQKVBiasTranspose(DType dt, void *q, void *k, void *v, void *qkv, const void *bias, int B, int S,
                              int tokens, int H, int D, hipStream_t stream) {
  if (B < 0 || S < 0 || tokens < 0 || H < 0 || D < 0) fail("addFusedQKVBiasTranspose: negative shape");
  if (tokens == 0 || H == 0 || D == 0) return;
  if (tokens != B * S) fail("addFusedQKVBiasTranspose: token_num must equal batch_size * seq_len");
  if (D % 8) fail("addFusedQKVBiasTranspose: size_per_head must be a multiple of 8");
  if (!q || !k || !v || !qkv) fail("addFusedQKVBiasTranspose: null pointer");
  if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(qkv) || (bias && !aligned16(bias)))
    fail("addFusedQKVBiasTranspose: pointers must be 16-byte aligned");
  const size_t total = (size_t)tokens * 3 * H * (D / 8);
  if (dt == DType::F16) {
    qkv_bias_transpose_kernel<_Float16><<<dim3(gridFor(total, 256)), dim3(256), 0, stream>>>(
        static_cast<_Float16 *>(q), static_cast<_Float16 *>(k), static_cast<_Float16 *>(v),
        static_cast<_Float16 *>(qkv), static_cast<const _Float16 *>(bias), S, tokens, H, D);
  } else if (dt == DType::BF16) {
    qkv_bias_transpose_kernel<bf16_t><<<dim3(gridFor(total, 256)), dim3(256), 0, stream>>>(
        static_cast<bf16_t *>(q), static_cast<bf16_t *>(k), static_cast<bf16_t *>(v),
        static_cast<bf16_t *>(qkv), static_cast<const bf16_t *>(bias), S, tokens, H, D);
  } else {
    fail("addFusedQKVBiasTranspose: element type must be fp16 or bf16");
  }
  MGPU_CHECK_LAUNCH("qkv_bias_transpose_kernel");
}

void addFusedQKVBiasTransposeF16(void *q, void *k, void *v, void *qkv, const void *bias, int B,
                                 int S, int tokens, int H, int D, hipStream_t stream) {
  addFusedQKVBiasTranspose(DType::F16, q, k, v, qkv, bias, B, S, tokens, H, D, stream);
}

} // namespace mgpu

// ---- exact (erf) GELU, in place -------------------------------------------
namespace mgpu {

namespace {

__device__ __forceinline__ float gelu_erf(float x) {
  return 0.5f * x * (1.0f + erff(x * 0.70710678118654752440f));
}

template <typename T>
__global__ __launch_bounds__(256) void gelu_h_vec8_kernel(u32x4 *__restrict__ data, size_t n8) {
  const size_t stride = (size_t)gridDim.x * 256;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n8; i += stride) {
    float v[8];
    ElemTraits<T>::unpack(data[i], v);
#pragma unroll
    for (int e = 0; e < 8; e++) v[e] = gelu_erfc(v[e]);
    data[i] = ElemTraits<T>::pack(v);
  }
}

template <typename T>
__global__ __launch_bounds__(256) void gelu_scalar_kernel(T *__restrict__ data, size_t begin,
                                                          size_t n) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t i = begin + (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
  {
    const float x = ElemTraits<T>::toFloat(data[i]);
    // fp32 results keep the library erf; the 16-bit types take the same formula as their vector kernel
    data[i] = ElemTraits<T>::fromFloat(sizeof(T) == 4 ? gelu_erf(x) : gelu_erfc(x));
  }
}

} // namespace

namespace {
template <typename T> void geluInPlaceH(void *data, size_t n, hipStream_t stream) {
  if (n == 0) return;
  auto *d = static_cast<T *>(data);
  size_t done = 0;
  if (aligned16(data) && n >= 8) {
    const size_t n8 = n / 8;
    gelu_h_vec8_kernel<T><<<dim3(gridFor(n8, 256)), dim3(256), 0, stream>>>(reinterpret_cast<u32x4 *>(d), n8);
    MGPU_CHECK_LAUNCH("gelu_h_vec8_kernel");
    done = n8 * 8;
  }
  if (done < n) {
    gelu_scalar_kernel<T><<<dim3(gridFor(n - done, 256)), dim3(256), 0, stream>>>(d, done, n);
    MGPU_CHECK_LAUNCH("gelu_scalar_kernel");
  }
}
} // namespace

void geluInPlaceF16(void *data, size_t n, hipStream_t stream) { geluInPlaceH<_Float16>(data, n, stream); }
void geluInPlaceBF16(void *data, size_t n, hipStream_t stream) { geluInPlaceH<bf16_t>(data, n, stream); }

void geluInPlaceF32(float *data, size_t n, hipStream_t stream) {
  if (n == 0) return;
  gelu_scalar_kernel<float><<<dim3(gridFor(n, 256)), dim3(256), 0, stream>>>(data, 0, n);
  MGPU_CHECK_LAUNCH("gelu_scalar_kernel");
}

} // namespace mgpu
