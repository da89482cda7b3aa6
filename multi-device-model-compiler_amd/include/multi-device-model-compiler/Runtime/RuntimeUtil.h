// Loading and calling a compiled model library; counterpart of the reference's
// include/multi-device-model-compiler/Runtime/RuntimeUtil.h:10-24 and
// lib/Runtime/RuntimeUtil.cpp:9-179, without the LLVMSupport dependency.
// Behaviour kept: outputs come first in the parameter vector (:100-112), the
// entry point is called with 0..5 descriptor pointers (:133-157), errors are
// reported on stderr with the reference's messages and are not fatal.
#ifndef MULTI_DEVICE_MODEL_COMPILER_RUNTIME_RUNTIMEUTIL_H_
#define MULTI_DEVICE_MODEL_COMPILER_RUNTIME_RUNTIMEUTIL_H_

#include "multi-device-model-compiler/Runtime/ModelInfo.h"
#include "multi-device-model-compiler/Runtime/TensorDescripter.h"

#include <string>
#include <vector>

namespace multi_device {
typedef void (*RunGraphFuncPtr)(...);

// Reads numElements fp32 values; nullptr (plus a message) when the file is
// missing or shorter than that ("Wrong File size", RuntimeUtil.cpp:16-19).
float *LoadFloatData(std::string &file, size_t numElements);
// Generic form: numElements * elementBytes raw bytes into a malloc'd buffer.
void *LoadRawData(const std::string &file, size_t numElements, size_t elementBytes);
template <size_t N> void SaveFloatData(std::string &file, FloatTensor<N> *tensor);
void *GetFloatTensorDescripter(std::vector<size_t> &shapes, std::string file, bool init,
                               bool useFile);
// Descriptor of any element size (the data pointers are typed float* but the
// buffer holds elementBytes per element).
void *GetTensorDescripter(std::vector<size_t> &shapes, std::string file, bool init, bool useFile,
                          size_t elementBytes);
void SaveFloatTensor(ModelInfo *info, std::vector<void *> params, std::string &file);
std::vector<void *> GetParamsVec(ModelInfo *info);
void *LoadLibrary(std::string libName);
RunGraphFuncPtr LoadFunc(void *handle, std::string funcName);
void RunGraphFunc(RunGraphFuncPtr func, std::vector<void *> &params);
void ClearOutputTensor(ModelInfo *info, std::vector<void *> &params);
} // namespace multi_device

#endif
