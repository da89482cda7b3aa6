// Drives the ordering check of the lowered call list: the lowering of a plan
// passes; the same call list with a cross-stream record removed, a buffer
// freed early or a stream left alive must be rejected.
#include "multi-device-model-compiler/Conversion/ConvertDeviceToRuntimeCalls.h"

#include <cstdio>
#include <string>

using namespace multi_device::conversion;

static const char *kPlan = R"(func @main_graph(%a: 4x8xf32, %b: 4x8xf32, %g: 8xf32, %be: 8xf32) -> (%y: 4x8xf32) {
  %c = device.add %a, %b : 4x8xf32
  %y = device.layernorm %c, %g, %be : 4x8xf32
  return
}
)";

static int failures = 0;
static void expect(bool cond, const char *what) {
  std::printf("%s %s\n", cond ? "ok  " : "FAIL", what);
  if (!cond) failures++;
}

static RuntimeProgram without(const RuntimeProgram &p, const std::string &callee, int nth) {
  RuntimeProgram q = p;
  int seen = 0;
  for (size_t i = 0; i < q.calls.size(); i++)
    if (q.calls[i].callee == callee && seen++ == nth) {
      q.calls.erase(q.calls.begin() + i);
      break;
    }
  return q;
}

int main() {
  DevicePlan plan;
  RuntimeProgram prog;
  std::string err;
  expect(parseDevicePlan(kPlan, plan, err) && lowerToRuntimeCalls(plan, DeviceType::GPU, prog, err), "plan lowers");
  expect(checkRuntimeProgram(prog, err), "lowered call list passes the check");

  // kernel stream no longer waits for the uploads in front of the first op
  RuntimeProgram q = without(prog, "mgpuStreamWaitEvent", 0);
  expect(!checkRuntimeProgram(q, err) && err.find("without waiting") != std::string::npos, "missing data->kernel wait is caught");
  // data stream frees / copies back without waiting for the kernel stream
  int waits = 0;
  for (const RuntimeCall &c : prog.calls) waits += c.callee == "mgpuStreamWaitEvent";
  q = without(prog, "mgpuStreamWaitEvent", waits - 1);
  expect(!checkRuntimeProgram(q, err) && err.find("without waiting") != std::string::npos, "missing kernel->data wait is caught");
  // use after free: move the first free to the front of the first op
  q = prog;
  for (size_t i = 0; i < q.calls.size(); i++)
    if (q.calls[i].callee == "mgpuMemFree") {
      RuntimeCall f = q.calls[i];
      q.calls.erase(q.calls.begin() + i);
      for (size_t j = 0; j < q.calls.size(); j++)
        if (q.calls[j].callee == "mgpuAddF32") {
          q.calls.insert(q.calls.begin() + j, f);
          break;
        }
      break;
    }
  expect(!checkRuntimeProgram(q, err), "use after free is caught");
  q = without(prog, "mgpuMemFree", 0);
  expect(!checkRuntimeProgram(q, err) && err.find("never freed") != std::string::npos, "leaked buffer is caught");
  q = without(prog, "mgpuStreamSynchronize", 1);
  expect(!checkRuntimeProgram(q, err) && err.find("synchronize") != std::string::npos, "unsynchronised stream is caught");
  q = without(prog, "mgpuStreamDestroy", 0);
  expect(!checkRuntimeProgram(q, err) && err.find("still live") != std::string::npos, "leaked stream is caught");
  q = without(prog, "mgpuEventRecord", 0);
  expect(!checkRuntimeProgram(q, err), "wait on an unrecorded event is caught");
  // CPU lowering of the same plan: two library calls, one temporary
  RuntimeProgram cpu;
  expect(lowerToRuntimeCalls(plan, DeviceType::CPU, cpu, err), "plan lowers for the CPU");
  std::string text = printRuntimeProgram(plan, cpu);
  expect(text.find("mcpuAddF32(%a, %b, %d0, 32)") != std::string::npos &&
             text.find("mcpuLayerNormF32(%d0, %g, %be, %y,") != std::string::npos &&
             text.find("%d0 = malloc(128)") != std::string::npos && text.find("free(%d0)") != std::string::npos,
         "CPU lowering calls the CPU library on host buffers");
  return failures ? 1 : 0;
}
