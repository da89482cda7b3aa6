// Shared helpers of the device kernel library: error convention, launch
// geometry and cross-lane reductions for 64-wide wavefronts.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <stdexcept>
#include <string>

namespace mgpu {

// Error convention of the kernel library: print, then throw std::logic_error
// (reference: lib/Kernels/GPU/Ops.cu:21-41).  The extern "C" layer catches it.
[[noreturn]] inline void fail(const std::string &what) {
  std::fprintf(stderr, "mgpu ops: %s\n", what.c_str());
  throw std::logic_error(what);
}

inline void checkHipStatus(hipError_t status, const char *where) {
  if (status != hipSuccess) {
    (void)hipGetLastError();
    fail(std::string(where) + ": HIP API failed with status " +
         std::to_string(static_cast<int>(status)) + ": " + hipGetErrorString(status));
  }
}

#define MGPU_CHECK_HIP(expr) ::mgpu::checkHipStatus((expr), #expr)
#define MGPU_CHECK_LAUNCH(name) ::mgpu::checkHipStatus(hipGetLastError(), name)

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Streaming kernels get one block per block-sized piece of the array rather
// than a grid sized to the machine with a stride loop: blocks are dispatched
// in index order, so at any moment the whole device works on one contiguous
// window of memory, which the HBM controllers serve faster (6.4 against
// 4.5-5.7 TB/s measured on a 1 GiB copy).  The stride loop only takes over
// beyond this many blocks.
constexpr int64_t kMaxStreamBlocks = int64_t(1) << 22;

inline int numComputeUnits() {
  static int cus = [] {
    int dev = 0, v = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || v <= 0)
      v = 256;
    return v;
  }();
  return cus;
}

// GELU in its exact (erf) form, x * Phi(x), for fp16 / bf16 results.  Phi comes
// from the complementary error function in the Chebyshev-fitted form
// erfc(z) = t * exp(-z^2 + P(t)), t = 1 / (1 + z / 2) (Numerical Recipes'
// erfcc, fractional error below 1.2e-7 for every z >= 0): about 18
// instructions, and accurate on the negative tail, where 1 + erf(x / sqrt 2)
// cancels (relative error of x * Phi(x) in fp32 below 3e-6 for x > -5 against
// 5e-2 for the erf form).
__device__ __forceinline__ float gelu_erfc(float x) {
  const float z = fabsf(x) * 0.70710678118654752440f;
  const float t = __builtin_amdgcn_rcpf(fmaf(0.5f, z, 1.0f));
  float p = 0.17087277f;
  p = fmaf(p, t, -0.82215223f);
  p = fmaf(p, t, 1.48851587f);
  p = fmaf(p, t, -1.13520398f);
  p = fmaf(p, t, 0.27886807f);
  p = fmaf(p, t, -0.18628806f);
  p = fmaf(p, t, 0.09678418f);
  p = fmaf(p, t, 0.37409196f);
  p = fmaf(p, t, 1.00002368f);
  p = fmaf(p, t, -1.26551223f);
  const float halfErfc = 0.5f * t * __builtin_amdgcn_exp2f((p - z * z) * 1.44269504088896340736f);
  return x * (x > 0.0f ? 1.0f - halfErfc : halfErfc);
}

// ---- cross-lane sums on a 64-wide wavefront ------------------------------
// DPP moves inside a row of 16 lanes (no LDS traffic), then lane exchanges
// across rows.  After the call every participating lane holds the same sum.

template <int CTRL> __device__ __forceinline__ float dpp_move(float v) {
  return __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false));
}

// The exchange between the two rows of a 32-lane group is v_permlane16_swap of gfx950:
// handed the same value twice, it returns in every lane the value of the lane's pair in the
// even row and the one in the odd row - one VALU instruction where a shuffle through
// ds_bpermute costs an address computation and a trip through the LDS crossbar (LayerNorm
// fp16 (4096, 768): 3.64 -> 3.50 us).  A full wavefront keeps the shuffles for both of its
// steps: with the swaps the fp32 (4096, 768) launch measured 0.1-0.15 us longer.
struct LanePair {
  float first, second;
};
__device__ __forceinline__ LanePair rows_xor16(float v) {
  const uint32_t u = __builtin_bit_cast(uint32_t, v);
  const auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  return {__builtin_bit_cast(float, (uint32_t)r[0]), __builtin_bit_cast(float, (uint32_t)r[1])};
}

// Sum over groups of LANES consecutive lanes (LANES in {16, 32, 64}).
template <int LANES> __device__ __forceinline__ float group_sum(float v) {
  v += dpp_move<0xB1>(v);  // quad_perm [1,0,3,2]: xor 1
  v += dpp_move<0x4E>(v);  // quad_perm [2,3,0,1]: xor 2
  v += dpp_move<0x141>(v); // row_half_mirror: lane i <-> 7 - i
  v += dpp_move<0x140>(v); // row_mirror:      lane i <-> 15 - i
  if (LANES == 32) {
    const LanePair p = rows_xor16(v);
    v = p.first + p.second;
  }
  if (LANES >= 64) {
    v += __shfl_xor(v, 16);
    v += __shfl_xor(v, 32);
  }
  return v;
}

template <int LANES> __device__ __forceinline__ float group_max(float v) {
  v = fmaxf(v, dpp_move<0xB1>(v));
  v = fmaxf(v, dpp_move<0x4E>(v));
  v = fmaxf(v, dpp_move<0x141>(v));
  v = fmaxf(v, dpp_move<0x140>(v));
  if (LANES == 32) {
    const LanePair p = rows_xor16(v);
    v = fmaxf(p.first, p.second);
  }
  if (LANES >= 64) {
    v = fmaxf(v, __shfl_xor(v, 16));
    v = fmaxf(v, __shfl_xor(v, 32));
  }
  return v;
}

} // namespace mgpu
