// Counterpart of the reference's Kernels/GPU/Utils.h (:6-20).
#ifndef MULTI_DEVICE_MODEL_COMPILER_KERNELS_GPU_UTILS_H_
#define MULTI_DEVICE_MODEL_COMPILER_KERNELS_GPU_UTILS_H_

#include "multi-device-model-compiler/Kernels/GPU/Ops.h"

// invokeCudaCast of the reference (:6-8); specialised for <half, float> and
// <float, half>.
template <typename T_OUT, typename T_IN>
MLIR_GPU_OPS_EXPORT void invokeCast(T_OUT *dst, T_IN const *const src, const size_t size,
                                    hipStream_t stream);

// Counterpart of getSMVersion (:10-20): the gfx target number of the current
// device, e.g. 950 for gfx950.
inline int getGfxVersion() {
  int device = -1;
  checkHipStatus(hipGetDevice(&device));
  hipDeviceProp_t prop;
  checkHipStatus(hipGetDeviceProperties(&prop, device));
  int v = 0;
  for (const char *p = prop.gcnArchName + 3; *p >= '0' && *p <= '9'; ++p) v = v * 10 + (*p - '0');
  return v;
}

#endif
