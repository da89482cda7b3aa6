// Shapes and input files of the model a runner drives; counterpart of the
// reference's include/multi-device-model-compiler/Runtime/ModelInfo.h:10-36 and
// lib/Runtime/ModelInfo.cpp:10-114 with the same flags:
//   --input  3_640_640,3_640_640   (shapes: dims joined by '_', tensors by ',')
//   --output 3_640_640
//   --data   a.dat,b.dat           (one raw little-endian file per input)
// Added: --dtype f32|f16 (element type of every tensor; the reference is fp32
// only, lib/Runtime/RuntimeUtil.cpp:77-98) and ranks up to 5.
#ifndef MULTI_DEVICE_MODEL_COMPILER_RUNTIME_MODELINFO_H_
#define MULTI_DEVICE_MODEL_COMPILER_RUNTIME_MODELINFO_H_

#include "multi-device-model-compiler/Runtime/CommandLine.h"

#include <string>
#include <vector>

namespace multi_device {

extern cl::Option InputShapes;
extern cl::Option OutputShapes;
extern cl::Option InputData;
extern cl::Option DataType;

std::vector<size_t> parseOneShape(const std::string &input);
std::vector<std::vector<size_t>> parseShapes(const std::string &str);

struct ModelInfo {
  static ModelInfo *ParseModelInfo();
  size_t InputNums();
  size_t OutputNums();
  size_t GetInputNumElements(int idx);
  size_t GetOutputNumElements(int idx);
  std::vector<size_t> &GetInputSize(int idx);
  std::vector<size_t> &GetOutputSize(int idx);
  std::string GetFile(int idx);
  bool ExistFile();
  size_t ElementBytes() const { return elementBytes; }

private:
  std::vector<std::vector<size_t>> inputSizes, outputSizes;
  std::vector<std::string> inputData;
  size_t elementBytes = 4;
};

} // namespace multi_device

#endif
