// Executes a lowered runtime program: what the reference gets by compiling the
// LLVM dialect output of ConvertDeviceToLLVM into the model library, done here
// by walking the call list.  Every callee is looked up by name (dlsym), as the
// generated code binds them (ConvertDeviceToLLVM.cpp:111-258 declares each
// callee by symbol name and signature), and called through its C prototype
// from include/mgpu_runtime.h, include/mgpu_ops.h or the CPU op library.
#include "multi-device-model-compiler/Conversion/ConvertDeviceToRuntimeCalls.h"

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <dlfcn.h>
#include <functional>
#include <unordered_map>

namespace multi_device {
namespace conversion {

namespace {

struct Machine {
  const RuntimeProgram &prog;
  const HostBuffers &host;
  void *library;
  std::vector<void *> streams, events, buffers;
  std::unordered_map<std::string, void *> symbols;
  std::string error;

  void *resolve(const std::string &name) {
    auto it = symbols.find(name);
    if (it != symbols.end()) return it->second;
    void *p = dlsym(library ? library : RTLD_DEFAULT, name.c_str());
    if (!p) error = "runtime symbol " + name + " is not loaded";
    symbols[name] = p;
    return p;
  }
  void *pointer(const CallArg &a) const {
    switch (a.kind) {
    case CallArg::Stream: return streams[a.index];
    case CallArg::Event: return events[a.index];
    case CallArg::Device: return buffers[a.index];
    case CallArg::Host: return host[a.index];
    default: return nullptr;
    }
  }
  void store(const CallArg &r, void *value) {
    if (r.kind == CallArg::Stream) streams[r.index] = value;
    else if (r.kind == CallArg::Event) events[r.index] = value;
    else if (r.kind == CallArg::Device) buffers[r.index] = value;
  }
};

typedef void *P;
typedef int64_t L;
typedef int32_t I;
typedef float F;

// Calls `callee` with the arguments of `c`.  One case per prototype.
bool dispatch(Machine &m, const RuntimeCall &c) {
  const std::string &n = c.callee;
  const auto &a = c.args;
  if (n == "malloc") { // CPU temporaries
    m.store(c.result, std::malloc((size_t)a[0].i));
    return true;
  }
  if (n == "free") {
    std::free(m.pointer(a[0]));
    return true;
  }
  void *fn = m.resolve(n);
  if (!fn) return false;
  auto p = [&](size_t i) { return m.pointer(a[i]); };
  auto l = [&](size_t i) { return (L)a[i].i; };
  auto i = [&](size_t k) { return (I)a[k].i; };
  auto f = [&](size_t k) { return a[k].f; };
  auto b = [&](size_t k) { return a[k].i != 0; };

  // ---- runtime (include/mgpu_runtime.h) ------------------------------------
  if (n == "mgpuStreamCreate") { m.store(c.result, ((P(*)())fn)()); return true; }
  if (n == "mgpuEventCreateWithStream") { m.store(c.result, ((P(*)(P))fn)(p(0))); return true; }
  if (n == "mgpuEventRecord" || n == "mgpuStreamWaitEvent") { ((void (*)(P, P))fn)(p(0), p(1)); return true; }
  if (n == "mgpuEventDestroy" || n == "mgpuStreamSynchronize" || n == "mgpuStreamDestroy") { ((void (*)(P))fn)(p(0)); return true; }
  if (n == "mgpuMemAlloc") { m.store(c.result, ((P(*)(uint64_t, P))fn)((uint64_t)l(0), p(1))); return true; }
  if (n == "mgpuMemFree") { ((void (*)(P, P))fn)(p(0), p(1)); return true; }
  if (n == "mgpuMemcpy") { ((void (*)(P, P, size_t, P))fn)(p(0), p(1), (size_t)l(2), p(3)); return true; }
  if (n == "mgpuModuleGetFunction") { m.store(c.result, ((P(*)(const char *))fn)(a[0].text.c_str())); return true; }
  if (n == "mgpuLaunchKernel") {
    // params: array of pointers to the argument values
    const auto &pack = a[9].pack;
    std::vector<uint64_t> values(pack.size());
    std::vector<void *> params(pack.size());
    for (size_t k = 0; k < pack.size(); k++) {
      const CallArg &x = pack[k];
      values[k] = (x.kind == CallArg::I64 || x.kind == CallArg::I32) ? (uint64_t)x.i : (uint64_t)(uintptr_t)m.pointer(x);
      params[k] = &values[k];
    }
    ((void (*)(P, intptr_t, intptr_t, intptr_t, intptr_t, intptr_t, intptr_t, int32_t, P, void **, void **))fn)(
        p(0), (intptr_t)l(1), (intptr_t)l(2), (intptr_t)l(3), (intptr_t)l(4), (intptr_t)l(5), (intptr_t)l(6), i(7), p(8),
        params.data(), nullptr);
    return true;
  }
  // ---- kernel library (include/mgpu_ops.h) ----------------------------------
  if (n == "mgpuAddF32") { ((void (*)(P, P, P, L, P))fn)(p(0), p(1), p(2), l(3), p(4)); return true; }
  if (n == "mgpuLayerNormF32" || n == "mgpuLayerNormF16" || n == "mgpuLayerNormBF16") {
    ((void (*)(P, P, P, P, F, I, I, P))fn)(p(0), p(1), p(2), p(3), f(4), i(5), i(6), p(7));
    return true;
  }
  if (n == "mgpuAddResidualPreLayerNormF32" || n == "mgpuAddResidualPreLayerNormF16" || n == "mgpuAddResidualPreLayerNormBF16") {
    ((void (*)(P, P, P, P, P, P, F, I, I, P))fn)(p(0), p(1), p(2), p(3), p(4), p(5), f(6), i(7), i(8), p(9));
    return true;
  }
  if (n == "mgpuFusedMHAF16" || n == "mgpuFusedMHABF16") {
    ((void (*)(P, P, P, I, I, I, I, F, I, P))fn)(p(0), p(1), p(2), i(3), i(4), i(5), i(6), f(7), i(8), p(9));
    return true;
  }
  if (n == "mgpuCastF32ToF16" || n == "mgpuCastF16ToF32" || n == "mgpuCastF32ToBF16" || n == "mgpuCastBF16ToF32") { ((void (*)(P, P, size_t, P))fn)(p(0), p(1), (size_t)l(2), p(3)); return true; }
  if (n == "mgpuConv2d" || n == "mcpuConv2d") {
    typedef void (*Gpu)(P, P, P, P, P, L, L, L, L, L, L, L, L, L, L, L, L, L, L, L, L, L, bool, bool, P);
    typedef void (*Cpu)(P, P, P, P, P, L, L, L, L, L, L, L, L, L, L, L, L, L, L, L, L, L, bool, bool);
    if (n[1] == 'g')
      ((Gpu)fn)(p(0), p(1), p(2), p(3), p(4), l(5), l(6), l(7), l(8), l(9), l(10), l(11), l(12), l(13), l(14), l(15), l(16),
                l(17), l(18), l(19), l(20), l(21), b(22), b(23), p(24));
    else
      ((Cpu)fn)(p(0), p(1), p(2), p(3), p(4), l(5), l(6), l(7), l(8), l(9), l(10), l(11), l(12), l(13), l(14), l(15), l(16),
                l(17), l(18), l(19), l(20), l(21), b(22), b(23));
    return true;
  }
  if (n == "mgpuPool2d" || n == "mcpuPool2d") {
    typedef void (*Gpu)(P, P, L, L, L, L, L, L, L, L, L, L, L, L, L, L, L, P);
    typedef void (*Cpu)(P, P, L, L, L, L, L, L, L, L, L, L, L, L, L, L, L);
    if (n[1] == 'g')
      ((Gpu)fn)(p(0), p(1), l(2), l(3), l(4), l(5), l(6), l(7), l(8), l(9), l(10), l(11), l(12), l(13), l(14), l(15), l(16), p(17));
    else
      ((Cpu)fn)(p(0), p(1), l(2), l(3), l(4), l(5), l(6), l(7), l(8), l(9), l(10), l(11), l(12), l(13), l(14), l(15), l(16));
    return true;
  }
  if (n == "mgpuMatmul") { ((void (*)(P, P, P, P, L, L, L, P))fn)(p(0), p(1), p(2), p(3), l(4), l(5), l(6), p(7)); return true; }
  if (n == "mgpuMatmulExF16" || n == "mgpuMatmulExF32" || n == "mgpuMatmulExBF16") {
    ((void (*)(P, P, P, P, P, L, L, L, I, I, I, P))fn)(p(0), p(1), p(2), p(3), p(4), l(5), l(6), l(7), i(8), i(9), i(10), p(11));
    return true;
  }
  if (n == "mgpuLLMDecodingContextLayer") {
    ((void (*)(P, P, P, P, P, P, P, P, P, L, L, L, L, L, bool, bool, bool, P))fn)(
        p(0), p(1), p(2), p(3), p(4), p(5), p(6), p(7), p(8), l(9), l(10), l(11), l(12), l(13), b(14), b(15), b(16), p(17));
    return true;
  }
  if (n == "mgpuBertEncoderLayerF16") {
    ((void (*)(P, P, P, P, P, P, P, P, P, P, P, P, P, P, P, L, L, L, L, L, F, P))fn)(
        p(0), p(1), p(2), p(3), p(4), p(5), p(6), p(7), p(8), p(9), p(10), p(11), p(12), p(13), p(14), l(15), l(16), l(17),
        l(18), l(19), f(20), p(21));
    return true;
  }
  // ---- CPU op library (Kernels/CPU/Ops.h) ------------------------------------
  if (n == "mcpuAddF32") { ((void (*)(P, P, P, L))fn)(p(0), p(1), p(2), l(3)); return true; }
  if (n == "mcpuLayerNormF32") { ((void (*)(P, P, P, P, F, I, I))fn)(p(0), p(1), p(2), p(3), f(4), i(5), i(6)); return true; }
  if (n == "mcpuMatmul") { ((void (*)(P, P, P, P, L, L, L))fn)(p(0), p(1), p(2), p(3), l(4), l(5), l(6)); return true; }
  if (n == "mcpuFusedMHAF16") {
    ((void (*)(P, P, P, I, I, I, I, F, I))fn)(p(0), p(1), p(2), i(3), i(4), i(5), i(6), f(7), i(8));
    return true;
  }
  if (n == "mcpuLayerNormF16") { ((void (*)(P, P, P, P, F, I, I))fn)(p(0), p(1), p(2), p(3), f(4), i(5), i(6)); return true; }
  if (n == "mcpuAddResidualPreLayerNormF32" || n == "mcpuAddResidualPreLayerNormF16") {
    ((void (*)(P, P, P, P, P, P, F, I, I))fn)(p(0), p(1), p(2), p(3), p(4), p(5), f(6), i(7), i(8));
    return true;
  }
  if (n == "mcpuCastF32ToF16" || n == "mcpuCastF16ToF32") { ((void (*)(P, P, size_t))fn)(p(0), p(1), (size_t)l(2)); return true; }
  if (n == "mcpuMatmulExF16" || n == "mcpuMatmulExF32") {
    ((void (*)(P, P, P, P, P, L, L, L, I, I, I))fn)(p(0), p(1), p(2), p(3), p(4), l(5), l(6), l(7), i(8), i(9), i(10));
    return true;
  }
  if (n == "mcpuLLMDecodingContextLayer") {
    ((void (*)(P, P, P, P, P, P, P, P, P, L, L, L, L, L, bool, bool, bool))fn)(
        p(0), p(1), p(2), p(3), p(4), p(5), p(6), p(7), p(8), l(9), l(10), l(11), l(12), l(13), b(14), b(15), b(16));
    return true;
  }
  if (n == "mcpuBertEncoderLayerF16") {
    ((void (*)(P, P, P, P, P, P, P, P, P, P, P, P, P, P, P, L, L, L, L, L, F))fn)(
        p(0), p(1), p(2), p(3), p(4), p(5), p(6), p(7), p(8), p(9), p(10), p(11), p(12), p(13), p(14), l(15), l(16), l(17),
        l(18), l(19), f(20));
    return true;
  }
  m.error = "no prototype for callee " + n;
  return false;
}

} // namespace

bool executeRuntimeProgram(const DevicePlan &plan, const RuntimeProgram &prog, const HostBuffers &buffers,
                           void *libraryHandle, std::string &error) {
  if (buffers.size() != plan.values.size()) {
    error = "one host buffer slot per plan value is required";
    return false;
  }
  for (size_t v = 0; v < plan.values.size(); v++)
    if (plan.values[v].kind != PlanValue::Temp && !buffers[v] && plan.values[v].type.numel() > 0) {
      error = "no host buffer for %" + plan.values[v].name;
      return false;
    }
  Machine m{prog, buffers, libraryHandle};
  m.streams.assign(prog.numStreams, nullptr);
  m.events.assign(prog.numEvents, nullptr);
  m.buffers.assign(prog.numDeviceBuffers, nullptr);
  for (const RuntimeCall &c : prog.calls)
    if (!dispatch(m, c)) {
      error = m.error;
      return false;
    }
  return true;
}

bool loadPlanConstants(const DevicePlan &plan, const std::string &baseDir, HostBuffers &buffers, std::string &error) {
  buffers.resize(plan.values.size(), nullptr);
  for (size_t v = 0; v < plan.values.size(); v++) {
    const PlanValue &val = plan.values[v];
    if (val.kind != PlanValue::Constant) continue;
    const std::string path = (!val.file.empty() && val.file[0] == '/') || baseDir.empty() ? val.file : baseDir + "/" + val.file;
    FILE *f = std::fopen(path.c_str(), "rb");
    if (!f) {
      error = "cannot open " + path + " for %" + val.name;
      return false;
    }
    const size_t bytes = val.type.bytes();
    void *data = std::malloc(bytes ? bytes : 1);
    const size_t got = std::fread(data, 1, bytes, f);
    std::fseek(f, 0, SEEK_END);
    const long size = std::ftell(f);
    std::fclose(f);
    if (got != bytes || (size_t)size != bytes) {
      std::free(data);
      error = "Wrong File size: " + path + " holds " + std::to_string(size) + " bytes, %" + val.name + " needs " + std::to_string(bytes);
      return false;
    }
    buffers[v] = data;
  }
  return true;
}

} // namespace conversion
} // namespace multi_device
