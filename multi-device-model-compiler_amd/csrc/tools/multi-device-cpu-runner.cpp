// multi-device-cpu-runner: the CPU twin of the GPU runner, timing each rerun
// with std::chrono; flags, order and output lines follow the reference's
// tools/multi-device-cpu-runner/multi-device-cpu-runner.cpp:19-86.  A
// `<name>.plan` in place of the library runs that device plan through its CPU
// lowering; shapes then come from the plan and --input / --output are ignored.
#include "multi-device-model-compiler/Kernels/CPU/Ops.h"
#include "multi-device-model-compiler/Runtime/ModelInfo.h"
#include "multi-device-model-compiler/Runtime/PlanModel.h"
#include "multi-device-model-compiler/Runtime/RuntimeUtil.h"
#include "multi-device-model-compiler/Runtime/TensorDescripter.h"

#include <chrono>
#include <cstdio>
#include <dlfcn.h>
#include <string>

using namespace multi_device;

static cl::Option LibPath(cl::Option::Positional, "lib", "<lib> Model Library Path");
static cl::Option RunFuncName(cl::Option::String, "func", "Model Run Func Name",
                              "_mlir_ciface_main_graph");
static cl::Option OutputName(cl::Option::String, "out-data", "Output file name", "");
static cl::Option RerunTimes(cl::Option::Int, "rerun", "Rerun time", "0");
static cl::Option FastMode(cl::Option::Bool, "fast", "Fast mode,with precision loss", "false");

int main(int argc, char **argv) {
  if (!cl::ParseCommandLineOptions(argc, argv, "Multi device cpu runner\n")) {
    std::fprintf(stderr, "Failed to parse options\n");
    return 1;
  }

  cpuOpsInit(FastMode.asBool());

  if (IsPlanFile(LibPath.str())) {
    PlanModel *model = PlanModel::Load(LibPath.str(), conversion::DeviceType::CPU);
    if (!model || !model->PrepareIO(InputData.values) || !model->Run())
      return 1;
    if (!OutputName.str().empty())
      model->SaveOutput(0, OutputName.str());
    const int reruns = RerunTimes.asInt();
    if (reruns != 0) {
      std::chrono::duration<double> elapsed(0);
      for (int i = 0; i < reruns; ++i) {
        auto start = std::chrono::high_resolution_clock::now();
        if (!model->Run())
          return 1;
        auto end = std::chrono::high_resolution_clock::now();
        elapsed += (end - start);
      }
      std::printf("Run \t%d\ttimes\n", reruns);
      std::printf("Average time:\t%g\tseconds\n", elapsed.count() / reruns);
      std::printf("Threads:\t%d\n", cpuOpsNumThreads());
    }
    delete model;
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

  const int reruns = RerunTimes.asInt();
  if (reruns != 0) {
    std::chrono::duration<double> elapsed(0);
    for (int i = 0; i < reruns; ++i) {
      ClearOutputTensor(info, params);
      auto start = std::chrono::high_resolution_clock::now();
      RunGraphFunc(func, params);
      auto end = std::chrono::high_resolution_clock::now();
      elapsed += (end - start);
    }
    std::printf("Run \t%d\ttimes\n", reruns);
    std::printf("Average time:\t%g\tseconds\n", elapsed.count() / reruns);
    std::printf("Threads:\t%d\n", cpuOpsNumThreads());
  }

  dlclose(handle);
  return 0;
}
