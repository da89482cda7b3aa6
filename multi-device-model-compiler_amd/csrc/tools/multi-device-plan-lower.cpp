// multi-device-plan-lower: the textual end of the device -> runtime-call
// lowering.  Reads a device plan, verifies it and prints either the plan
// (round trip) or the runtime calls a run would make, in order; the role
// `multi-device-opt --convert-device-to-llvm` plays for the reference's MLIR
// pipeline (tools/multi-device-opt).  Needs no GPU.
//
//   multi-device-plan-lower <file.plan> [--device gpu|cpu] [--emit calls|plan]
//
// Exit status 0 when the plan verifies, lowers and its call sequence passes
// the ordering check; 1 otherwise, with the reason on stderr.
#include "multi-device-model-compiler/Conversion/ConvertDeviceToRuntimeCalls.h"
#include "multi-device-model-compiler/Runtime/CommandLine.h"

#include <cstdio>
#include <fstream>
#include <sstream>

using namespace multi_device;
using namespace multi_device::conversion;

static cl::Option PlanPath(cl::Option::Positional, "plan", "<plan> Device plan file");
static cl::Option Device(cl::Option::String, "device", "Target device: gpu or cpu", "gpu");
static cl::Option Emit(cl::Option::String, "emit", "What to print: calls or plan", "calls");

int main(int argc, char **argv) {
  if (!cl::ParseCommandLineOptions(argc, argv, "Multi device plan lowering\n")) {
    std::fprintf(stderr, "Failed to parse options\n");
    return 1;
  }
  std::ifstream in(PlanPath.str());
  if (!in) {
    std::fprintf(stderr, "Failed to open plan:%s\n", PlanPath.str().c_str());
    return 1;
  }
  std::stringstream text;
  text << in.rdbuf();
  DevicePlan plan;
  std::string error;
  if (!parseDevicePlan(text.str(), plan, error) || !verifyDevicePlan(plan, error)) {
    std::fprintf(stderr, "%s: %s\n", PlanPath.str().c_str(), error.c_str());
    return 1;
  }
  if (Emit.str() == "plan") {
    std::fputs(printDevicePlan(plan).c_str(), stdout);
    return 0;
  }
  if (Emit.str() != "calls" || (Device.str() != "gpu" && Device.str() != "cpu")) {
    std::fprintf(stderr, "--emit is calls or plan, --device is gpu or cpu\n");
    return 1;
  }
  RuntimeProgram program;
  if (!lowerToRuntimeCalls(plan, Device.str() == "gpu" ? DeviceType::GPU : DeviceType::CPU, program, error)) {
    std::fprintf(stderr, "%s: %s\n", PlanPath.str().c_str(), error.c_str());
    return 1;
  }
  std::fputs(printRuntimeProgram(plan, program).c_str(), stdout);
  if (!checkRuntimeProgram(program, error)) {
    std::fprintf(stderr, "%s: ordering check failed: %s\n", PlanPath.str().c_str(), error.c_str());
    return 1;
  }
  return 0;
}
