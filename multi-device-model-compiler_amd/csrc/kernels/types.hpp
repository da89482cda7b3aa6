// Element traits for the 128-bit vectorised kernels: how many elements one
// 16-byte vector holds and how it widens to / narrows from fp32 (narrowing is
// round to nearest even, once).
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

namespace mgpu {

// 16 raw bytes: the unit every vectorised load and store moves.
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// bfloat16 travels as its 16 bit pattern; the kernels only ever widen it to
// fp32 or narrow fp32 to it.
struct bf16_t {
  uint16_t bits;
};

__device__ __forceinline__ float bf16_to_float(uint16_t b) {
  return __builtin_bit_cast(float, (uint32_t)b << 16);
}

__device__ __forceinline__ uint16_t float_to_bf16(float f) {
  uint32_t u = __builtin_bit_cast(uint32_t, f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u); // quiet NaN
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

template <typename T> struct ElemTraits;

template <> struct ElemTraits<float> {
  static constexpr int kVec = 4;
  __device__ static __forceinline__ float toFloat(float v) { return v; }
  __device__ static __forceinline__ float fromFloat(float v) { return v; }
  __device__ static __forceinline__ void unpack(const u32x4 &raw, float (&out)[4]) {
    // Copy the lanes out first: __builtin_bit_cast applied directly to a
    // vector-element lvalue reads element 0 whichever element is named.
    const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
    for (int i = 0; i < 4; i++) out[i] = __builtin_bit_cast(float, w[i]);
  }
  __device__ static __forceinline__ u32x4 pack(const float (&in)[4]) {
    u32x4 r;
    r.x = __builtin_bit_cast(uint32_t, in[0]);
    r.y = __builtin_bit_cast(uint32_t, in[1]);
    r.z = __builtin_bit_cast(uint32_t, in[2]);
    r.w = __builtin_bit_cast(uint32_t, in[3]);
    return r;
  }
};

template <> struct ElemTraits<_Float16> {
  static constexpr int kVec = 8;
  typedef _Float16 half2v __attribute__((ext_vector_type(2)));
  __device__ static __forceinline__ float toFloat(_Float16 v) { return (float)v; }
  __device__ static __forceinline__ _Float16 fromFloat(float v) { return (_Float16)v; }
  __device__ static __forceinline__ void unpack(const u32x4 &raw, float (&out)[8]) {
    const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const half2v h = __builtin_bit_cast(half2v, w[i]);
      out[2 * i] = (float)h[0];
      out[2 * i + 1] = (float)h[1];
    }
  }
  __device__ static __forceinline__ u32x4 pack(const float (&in)[8]) {
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
      half2v h;
      h[0] = (_Float16)in[2 * i];
      h[1] = (_Float16)in[2 * i + 1];
      w[i] = __builtin_bit_cast(uint32_t, h);
    }
    return u32x4{w[0], w[1], w[2], w[3]};
  }
};

template <> struct ElemTraits<bf16_t> {
  static constexpr int kVec = 8;
  __device__ static __forceinline__ float toFloat(bf16_t v) { return bf16_to_float(v.bits); }
  __device__ static __forceinline__ bf16_t fromFloat(float v) { return bf16_t{float_to_bf16(v)}; }
  __device__ static __forceinline__ void unpack(const u32x4 &raw, float (&out)[8]) {
    const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
    for (int i = 0; i < 4; i++) {
      out[2 * i] = __builtin_bit_cast(float, w[i] << 16);
      out[2 * i + 1] = __builtin_bit_cast(float, w[i] & 0xffff0000u);
    }
  }
  __device__ static __forceinline__ u32x4 pack(const float (&in)[8]) {
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; i++)
      w[i] = (uint32_t)float_to_bf16(in[2 * i]) | ((uint32_t)float_to_bf16(in[2 * i + 1]) << 16);
    return u32x4{w[0], w[1], w[2], w[3]};
  }
};

} // namespace mgpu
