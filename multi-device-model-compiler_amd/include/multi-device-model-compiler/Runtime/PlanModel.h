// A model given as a device plan instead of a compiled library: the runners
// accept `<name>.plan` where the reference takes the `.so` that
// multi-device-lib-generate produced from the lowered module.  Loading parses,
// verifies and lowers the plan once (Conversion/ConvertDeviceToRuntimeCalls.h);
// every run executes the lowered call list, i.e. does what the compiled
// _mlir_ciface_main_graph of that model would do.
#ifndef MULTI_DEVICE_MODEL_COMPILER_RUNTIME_PLANMODEL_H_
#define MULTI_DEVICE_MODEL_COMPILER_RUNTIME_PLANMODEL_H_

#include "multi-device-model-compiler/Conversion/ConvertDeviceToRuntimeCalls.h"

#include <string>
#include <vector>

namespace multi_device {

bool IsPlanFile(const std::string &path); // ends in ".plan"

class PlanModel {
public:
  // nullptr (message on stderr) when the plan cannot be read, parsed, verified
  // or lowered for `device`, or a constant's file is missing or of the wrong size.
  static PlanModel *Load(const std::string &path, conversion::DeviceType device);
  ~PlanModel();

  // Host buffers of the function arguments: read from `files` (one raw file
  // per input, in signature order; sizes are checked: "Wrong File size") or,
  // with no files, zero-filled.  Outputs are allocated here as well.
  bool PrepareIO(const std::vector<std::string> &files);
  // One execution of the lowered program.  `library` as in executeRuntimeProgram.
  bool Run(void *library = nullptr);
  // Raw bytes of output `idx` in its own element type.
  bool SaveOutput(size_t idx, const std::string &file) const;

  const conversion::DevicePlan &Plan() const { return plan; }
  const conversion::RuntimeProgram &Program() const { return program; }
  void *InputData(size_t idx) { return buffers[plan.inputs[idx]]; }
  void *OutputData(size_t idx) { return buffers[plan.outputs[idx]]; }

private:
  conversion::DevicePlan plan;
  conversion::RuntimeProgram program;
  conversion::HostBuffers buffers;
};

} // namespace multi_device

#endif
