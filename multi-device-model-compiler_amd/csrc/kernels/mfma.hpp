// Operand types and the two matrix instructions shared by the MFMA kernels of
// this library (v_mfma_f32_32x32x16_{f16,bf16}), plus the transposing LDS read
// and the lane-half exchange of gfx950.
//
// Operand lane layout of the 32x32x16 instructions: lane l supplies row (A) or
// column (B) l % 32 and k-slots 8 * (l / 32) .. +7; the 32x32 accumulator gives
// lane l column l % 32 and rows 8 * (i / 4) + 4 * (l / 32) + i % 4 for register i.
#pragma once

#include "types.hpp"

namespace mgpu {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef short i16x4 __attribute__((ext_vector_type(4)));
typedef unsigned char __attribute__((address_space(3))) lds_u8; // a byte in LDS

template <typename T> struct Mma;
template <> struct Mma<_Float16> {
  using v8 = f16x8;
  using v4 = f16x4;
  __device__ static __forceinline__ f32x16 run(v8 a, v8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
  __device__ static __forceinline__ _Float16 narrow(float f) { return (_Float16)f; }
  __device__ static __forceinline__ float widen(_Float16 h) { return (float)h; }
  __device__ static __forceinline__ v4 readTr(const lds_u8 *p) {
    return __builtin_bit_cast(v4, __builtin_amdgcn_ds_read_tr16_b64_v4i16((i16x4 __attribute__((address_space(3))) *)p));
  }
};
template <> struct Mma<bf16_t> {
  using v8 = bf16x8;
  using v4 = bf16x4;
  __device__ static __forceinline__ f32x16 run(v8 a, v8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
  __device__ static __forceinline__ __bf16 narrow(float f) { return (__bf16)f; }
  __device__ static __forceinline__ float widen(__bf16 h) { return (float)h; }
  __device__ static __forceinline__ v4 readTr(const lds_u8 *p) {
    return __builtin_bit_cast(v4, __builtin_amdgcn_ds_read_tr16_b64_v4i16((i16x4 __attribute__((address_space(3))) *)p));
  }
};

// Exchange with lane l ^ 32: v_permlane32_swap hands every lane the value of
// the lower half in r[0] and of the upper half in r[1].
__device__ __forceinline__ float halves_max(float v) {
  const uint32_t u = __builtin_bit_cast(uint32_t, v);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return fmaxf(__builtin_bit_cast(float, (uint32_t)r[0]), __builtin_bit_cast(float, (uint32_t)r[1]));
}
__device__ __forceinline__ float halves_sum(float v) {
  const uint32_t u = __builtin_bit_cast(uint32_t, v);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return __builtin_bit_cast(float, (uint32_t)r[0]) + __builtin_bit_cast(float, (uint32_t)r[1]);
}

} // namespace mgpu
