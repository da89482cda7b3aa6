#include "multi-device-model-compiler/Runtime/ModelInfo.h"

#include <cstdio>
#include <string>
#include <vector>

namespace multi_device {

cl::Option InputShapes(cl::Option::String, "input", "Input shape,Use like 3_640_640,3_640_640",
                       "3_640_640,3_640_640");
cl::Option OutputShapes(cl::Option::String, "output", "Output shape,Use like 3_640_640",
                        "3_640_640");
cl::Option InputData(cl::Option::List, "data", "Input data file path");
cl::Option DataType(cl::Option::String, "dtype", "Element type of every tensor: f32 or f16", "f32");

std::vector<size_t> parseOneShape(const std::string &input) {
  std::vector<size_t> shape;
  size_t start = 0;
  while (true) {
    const size_t pos = input.find('_', start);
    shape.push_back(std::stoul(input.substr(start, pos == std::string::npos ? pos : pos - start)));
    if (pos == std::string::npos)
      break;
    start = pos + 1;
  }
  return shape;
}

std::vector<std::vector<size_t>> parseShapes(const std::string &str) {
  std::vector<std::vector<size_t>> shapes;
  size_t start = 0;
  while (true) {
    const size_t pos = str.find(',', start);
    shapes.emplace_back(
        parseOneShape(str.substr(start, pos == std::string::npos ? pos : pos - start)));
    if (pos == std::string::npos)
      break;
    start = pos + 1;
  }
  return shapes;
}

ModelInfo *ModelInfo::ParseModelInfo() {
  ModelInfo *info = new ModelInfo();
  info->inputSizes = parseShapes(InputShapes.str());
  info->outputSizes = parseShapes(OutputShapes.str());
  for (auto &data : InputData.values)
    info->inputData.emplace_back(data);
  if (DataType.str() == "f16") {
    info->elementBytes = 2;
  } else if (DataType.str() != "f32") {
    std::fprintf(stderr, "Not Implemented type!\n");
    delete info;
    return nullptr;
  }
  if (!info->inputData.empty() && info->inputData.size() != info->InputNums()) {
    std::fprintf(stderr, "Data num not equal input num!");
    delete info;
    return nullptr;
  }
  return info;
}

size_t ModelInfo::InputNums() { return inputSizes.size(); }
size_t ModelInfo::OutputNums() { return outputSizes.size(); }

static size_t product(const std::vector<size_t> &shape) {
  size_t nums = 1;
  for (auto sz : shape)
    nums *= sz;
  return nums;
}

size_t ModelInfo::GetInputNumElements(int idx) { return product(inputSizes[idx]); }
size_t ModelInfo::GetOutputNumElements(int idx) { return product(outputSizes[idx]); }
std::vector<size_t> &ModelInfo::GetInputSize(int idx) { return inputSizes[idx]; }
std::vector<size_t> &ModelInfo::GetOutputSize(int idx) { return outputSizes[idx]; }
std::string ModelInfo::GetFile(int idx) { return inputData[idx]; }
bool ModelInfo::ExistFile() { return !inputData.empty(); }

} // namespace multi_device
