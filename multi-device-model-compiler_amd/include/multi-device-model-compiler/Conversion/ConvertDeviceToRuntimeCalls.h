// Device-level plan -> runtime-call lowering, without MLIR.
//
// The reference lowers a bufferized function of Device-dialect ops
// (include/multi-device-model-compiler/Dialect/Device/IR/DeviceOps.td:17-183)
// to LLVM calls into the mgpu* runtime and kernel library in three passes:
//   * DeviceDataCopyGeneration (lib/Dialect/Device/Transform/
//     DeviceDataCopyGeneration.cpp:26-43,54-75): device buffers, host-to-device
//     copies in front of an op, the copy back and the deallocations behind it;
//   * AsyncDependencyConvert (AsyncDependencyConvert.cpp:45-140): two streams,
//     "DataStream" for alloc / dealloc / memcpy and "KernelStream" for launches
//     and library ops, a device.record for every cross-stream dependency, one
//     closing device.wait on both;
//   * ConvertDeviceToLLVM (lib/Conversion/ConvertDeviceToLLVM/
//     ConvertDeviceToLLVM.cpp:337-396,410-779): stream create + one event per
//     stream, record = mgpuEventRecord + mgpuStreamWaitEvent, the closing wait =
//     event destroy / stream synchronize / stream destroy, each op = one call
//     with the stream as last argument.
// This library does the same on a small textual plan: parse, verify, lower to
// a list of runtime calls (printable, so the call sequence can be checked
// without a GPU), and execute that list against the C ABI of
// include/mgpu_runtime.h / include/mgpu_ops.h (GPU) or the CPU op library
// (lowering for DeviceType::CPU, which like the reference's drops streams,
// device buffers and copies and calls mcpu* on the host buffers directly).
#ifndef MULTI_DEVICE_MODEL_COMPILER_CONVERSION_CONVERTDEVICETORUNTIMECALLS_H_
#define MULTI_DEVICE_MODEL_COMPILER_CONVERSION_CONVERTDEVICETORUNTIMECALLS_H_

#include <cstdint>
#include <map>
#include <string>
#include <vector>

namespace multi_device {
namespace conversion {

enum class ElemType { F32, F16, BF16, I32, I64 };
size_t elemBytes(ElemType t);
const char *elemName(ElemType t);

struct TensorType {
  std::vector<int64_t> shape;
  ElemType elem = ElemType::F32;
  int64_t numel() const;
  size_t bytes() const { return (size_t)numel() * elemBytes(elem); }
  std::string str() const; // "3x640x640xf32"
  bool operator==(const TensorType &o) const { return elem == o.elem && shape == o.shape; }
  bool operator!=(const TensorType &o) const { return !(*this == o); }
};

// A value of the plan: function argument (host memref), function result (host
// memref the caller receives), constant (host data read from a raw file next
// to the plan) or the result of an op (device buffer on the GPU path).
struct PlanValue {
  enum Kind { Input, Output, Constant, Temp };
  std::string name; // without the leading '%'
  TensorType type;
  Kind kind = Temp;
  std::string file; // Constant: raw little-endian file, relative to the plan
  int definedBy = -1; // index of the defining op, -1 for arguments and constants
};

struct AttrValue {
  enum Kind { Number, Bool, String, IntList } kind = Number;
  double number = 0;
  bool flag = false;
  std::string text;
  std::vector<int64_t> ints;
};

struct DeviceOp {
  std::string name;          // "device.matmul", "gpu.launch_func", ...
  std::vector<int> operands; // value indices, -1 for `none`
  std::vector<int> results;
  std::map<std::string, AttrValue> attrs;
  int line = 0;
};

struct DevicePlan {
  std::string func = "main_graph";
  std::vector<PlanValue> values;
  std::vector<int> inputs, outputs; // in signature order
  std::vector<DeviceOp> ops;
  int find(const std::string &name) const;
};

// Text -> plan.  Returns false and a "line N: ..." message on error.
bool parseDevicePlan(const std::string &text, DevicePlan &plan, std::string &error);
// Operand counts, element types and shapes of every op (the dialect's
// verifiers, DeviceDialect.cpp:61-125), every value defined before use, every
// function result produced exactly once.
bool verifyDevicePlan(const DevicePlan &plan, std::string &error);
std::string printDevicePlan(const DevicePlan &plan);

enum class DeviceType { CPU, GPU };

// One argument of a runtime call.
struct CallArg {
  enum Kind { Stream, Event, Device, Host, I64, I32, F32, Bool, Null, Symbol, Params } kind = Null;
  int index = 0;           // Stream / Event / Device slot, Host: plan value index
  int64_t i = 0;           // I64 / I32 / Bool
  float f = 0;             // F32
  std::string text;        // Symbol
  std::vector<CallArg> pack; // Params: pointer-to-argument array of a kernel launch
};

struct RuntimeCall {
  std::string callee; // "mgpuMemAlloc", "mgpuLayerNormF32", ...
  std::vector<CallArg> args;
  CallArg result;     // kind Null when the call returns nothing
  int op = -1;        // plan op this call belongs to (-1: prologue / epilogue / data movement)
};

struct RuntimeProgram {
  DeviceType device = DeviceType::GPU;
  std::vector<RuntimeCall> calls;
  int numStreams = 0, numEvents = 0, numDeviceBuffers = 0;
};

bool lowerToRuntimeCalls(const DevicePlan &plan, DeviceType device, RuntimeProgram &program,
                         std::string &error);
// One call per line: `%d0 = mgpuMemAlloc(4915200, %DataStream)`.
std::string printRuntimeProgram(const DevicePlan &plan, const RuntimeProgram &program);
// Replays the program on handle states only (no device): every handle created
// before use and released once, no buffer touched after its free, every kernel
// stream call ordered after the data-stream work it reads (a record in
// between), every copy back ordered after the kernel work, both streams
// synchronised at the end.  Returns false and the first violation.
bool checkRuntimeProgram(const RuntimeProgram &program, std::string &error);

// Host buffers of the plan's values for one run: inputs and constants are
// read, outputs written.  Indexed like DevicePlan::values; entries of Temp
// values are ignored.
typedef std::vector<void *> HostBuffers;

// Executes the program.  Callees are resolved by name with dlsym in
// `libraryHandle` (nullptr: the global namespace of the process), so the
// executor itself links against no device library.  Returns false with a
// message when a callee is missing; errors of the callees themselves are
// reported the way the libraries report them.
bool executeRuntimeProgram(const DevicePlan &plan, const RuntimeProgram &program,
                           const HostBuffers &buffers, void *libraryHandle, std::string &error);

// Reads the raw files of the plan's constants (relative to `baseDir`) into
// malloc'd buffers placed in `buffers`; the caller frees them.
bool loadPlanConstants(const DevicePlan &plan, const std::string &baseDir, HostBuffers &buffers,
                       std::string &error);

} // namespace conversion
} // namespace multi_device

#endif
