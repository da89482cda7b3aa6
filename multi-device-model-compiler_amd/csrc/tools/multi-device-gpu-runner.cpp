// multi-device-gpu-runner: loads the code object of generated kernels and a
// compiled model library, runs the model once (optionally dumping output 0),
// then `--rerun N` more times between two timing events.
//
// Same flags, call order and output lines as the reference's
// tools/multi-device-gpu-runner/multi-device-gpu-runner.cpp:19-93; the
// differences are the argument parser (no LLVM), `--ops` defaulting to
// ./ops.hsaco (a gfx950 code object instead of ops.cubin) and `--dtype`.  A
// `<name>.plan` in place of the library runs that device plan through its GPU
// lowering; shapes and element types then come from the plan and --input /
// --output / --dtype are ignored.
#include "mgpu_ops.h"
#include "multi-device-model-compiler/Kernels/GPU/Ops.h"
#include "multi-device-model-compiler/Runtime/HIP/HipRuntimeWrappers.h"
#include "multi-device-model-compiler/Runtime/ModelInfo.h"
#include "multi-device-model-compiler/Runtime/PlanModel.h"
#include "multi-device-model-compiler/Runtime/RuntimeUtil.h"
#include "multi-device-model-compiler/Runtime/TensorDescripter.h"

#include <cstdio>
#include <dlfcn.h>
#include <string>

using namespace multi_device;

static cl::Option LibPath(cl::Option::Positional, "lib", "<lib> Model Library Path");
static cl::Option RunFuncName(cl::Option::String, "func", "Model Run Func Name",
                              "_mlir_ciface_main_graph");
static cl::Option OutputName(cl::Option::String, "out-data", "Output file name", "");
static cl::Option RerunTimes(cl::Option::Int, "rerun", "Rerun time", "0");
static cl::Option OpsLibPath(cl::Option::String, "ops", "Ops library path", "./ops.hsaco");

int main(int argc, char **argv) {
  if (!cl::ParseCommandLineOptions(argc, argv, "Multi device gpu runner\n")) {
    std::fprintf(stderr, "Failed to parse options\n");
    return 1;
  }

  mgpuModuleFileLoad(OpsLibPath.str().c_str());
  gpuOpsInit();

  if (IsPlanFile(LibPath.str())) {
    PlanModel *model = PlanModel::Load(LibPath.str(), conversion::DeviceType::GPU);
    // A rejected op or a failed runtime call leaves the output undefined: every
    // run is followed by a look at both error slots, before anything is saved.
    auto runChecked = [&]() -> bool {
      if (!model->Run())
        return false;
      bool ok = true;
      if (const char *err = mgpuOpsTakeLastError()) {
        std::fprintf(stderr, "%s\n", err);
        ok = false;
      }
      if (int code = mgpuRuntimeTakeLastError()) {
        std::fprintf(stderr, "device runtime call failed with status %d\n", code);
        ok = false;
      }
      return ok;
    };
    if (!model || !model->PrepareIO(InputData.values) || !runChecked())
      return 1;
    if (!OutputName.str().empty())
      model->SaveOutput(0, OutputName.str());
    const int reruns = RerunTimes.asInt();
    if (reruns != 0) {
      auto stream = mgpuStreamCreate();
      auto eventBegin = mgpuEventEnableTimeCreate(), eventEnd = mgpuEventEnableTimeCreate();
      float elapsed = 0;
      for (int i = 0; i < reruns; ++i) {
        mgpuEventRecord(eventBegin, stream);
        if (!runChecked())
          return 1;
        mgpuEventRecord(eventEnd, stream);
        mgpuEventSynchronize(eventEnd);
        elapsed += mgpuEventElapsedTime(eventBegin, eventEnd);
      }
      mgpuEventDestroy(eventBegin);
      mgpuEventDestroy(eventEnd);
      mgpuStreamDestroy(stream);
      std::printf("Run \t%d\ttimes\n", reruns);
      std::printf("Average time:\t%g\tseconds\n", elapsed / (reruns * 1000.0f));
    }
    delete model;
    gpuOpsDeinit();
    mgpuModuleUnload();
    return 0;
  }

  ModelInfo *info = ModelInfo::ParseModelInfo();
  if (!info)
    return 1;
  auto params = GetParamsVec(info);

  void *handle = LoadLibrary(LibPath.str());
  auto func = LoadFunc(handle, RunFuncName.str());
  if (!func)
    return 1;

  RunGraphFunc(func, params);
  if (!OutputName.str().empty()) {
    std::string name = OutputName.str();
    SaveFloatTensor(info, params, name);
  }
  auto stream = mgpuStreamCreate();
  const int reruns = RerunTimes.asInt();
  if (reruns != 0) {
    auto eventBegin = mgpuEventEnableTimeCreate(), eventEnd = mgpuEventEnableTimeCreate();
    float elapsed = 0;
    for (int i = 0; i < reruns; ++i) {
      ClearOutputTensor(info, params);
      mgpuEventRecord(eventBegin, stream);
      RunGraphFunc(func, params);
      mgpuEventRecord(eventEnd, stream);
      mgpuEventSynchronize(eventEnd);
      elapsed += mgpuEventElapsedTime(eventBegin, eventEnd);
    }
    mgpuEventDestroy(eventBegin);
    mgpuEventDestroy(eventEnd);
    std::printf("Run \t%d\ttimes\n", reruns);
    std::printf("Average time:\t%g\tseconds\n", elapsed / (reruns * 1000.0f));
  }
  mgpuStreamDestroy(stream);

  gpuOpsDeinit();
  mgpuModuleUnload();
  dlclose(handle);
  return 0;
}
