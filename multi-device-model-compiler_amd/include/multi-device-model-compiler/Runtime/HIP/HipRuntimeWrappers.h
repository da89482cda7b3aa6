// C++ include point for the device runtime C ABI; counterpart of the
// reference's Runtime/CUDA/CudaRuntimeWrappers.h:25-54.
#ifndef MULTI_DEVICE_COMPILER_RUNTIME_HIP_HIPRUNTIMEWRAPPERS_H_
#define MULTI_DEVICE_COMPILER_RUNTIME_HIP_HIPRUNTIMEWRAPPERS_H_

#include "mgpu_runtime.h"

#endif
