// Plan -> runtime calls: data-copy generation, the two-stream discipline and
// the call emission of the reference's lowering in one walk over the ops.
//
// GPU (DeviceType::GPU).  Stream slot 0 is "DataStream", slot 1 "KernelStream",
// event slot i belongs to stream slot i (AsyncDependencyConvert.cpp:49-56,
// ConvertDeviceToLLVM.cpp:358-372).  A host value (argument or constant) gets a
// device buffer and a host-to-device copy on the data stream the first time an
// op reads it; op results get a device buffer; values stay on the device
// between ops (what FoldGPUMemcpy leaves of the per-op copies of
// DeviceDataCopyGeneration.cpp:26-43).  In front of every op the kernel stream
// is made to wait for the data stream (AsyncDependencyConvert.cpp:89-96: the
// record DataStream -> KernelStream the pass puts before each launch / matmul /
// layer op), and a buffer is released or copied back on the data stream only
// behind a record KernelStream -> DataStream (changeAsyncDependencies, :29-43).
// The closing device.wait destroys each event, synchronises and destroys each
// stream (ConvertDeviceToLLVM.cpp:345-354).
//
// CPU (DeviceType::CPU).  No streams, buffers or copies: ops call the CPU op
// library on host memory (ConvertDeviceToLLVM.cpp:433-436: cpuMatmulCallBuilder
// without a stream); temporaries are malloc'd.
#include "multi-device-model-compiler/Conversion/ConvertDeviceToRuntimeCalls.h"

#include <cmath>
#include <sstream>

namespace multi_device {
namespace conversion {

namespace {

constexpr int kData = 0, kKernel = 1;

CallArg stream(int s) { CallArg a; a.kind = CallArg::Stream; a.index = s; return a; }
CallArg event(int e) { CallArg a; a.kind = CallArg::Event; a.index = e; return a; }
CallArg dev(int d) { CallArg a; a.kind = CallArg::Device; a.index = d; return a; }
CallArg host(int v) { CallArg a; a.kind = CallArg::Host; a.index = v; return a; }
CallArg i64(int64_t v) { CallArg a; a.kind = CallArg::I64; a.i = v; return a; }
CallArg i32(int64_t v) { CallArg a; a.kind = CallArg::I32; a.i = v; return a; }
CallArg f32(double v) { CallArg a; a.kind = CallArg::F32; a.f = (float)v; return a; }
CallArg boolean(bool v) { CallArg a; a.kind = CallArg::Bool; a.i = v; return a; }
CallArg null() { return CallArg(); }
CallArg symbol(const std::string &s) { CallArg a; a.kind = CallArg::Symbol; a.text = s; return a; }

struct Lowering {
  const DevicePlan &plan;
  RuntimeProgram &prog;
  DeviceType device;
  std::vector<int> buffer;   // plan value -> device buffer slot (GPU) / -1
  std::vector<int> lastUse;  // plan value -> index of the last op reading it (or a view of it)
  std::vector<int> root;     // plan value -> the value whose buffer it is a view of (itself otherwise)
  bool kernelAhead = false;  // kernel-stream work the data stream has not been made to wait for
  int curOp = -1;

  void call(const std::string &callee, std::vector<CallArg> args, CallArg result = CallArg()) {
    RuntimeCall c;
    c.callee = callee;
    c.args = std::move(args);
    c.result = result;
    c.op = curOp;
    prog.calls.push_back(c);
  }
  void record(int src, int dst) {
    call("mgpuEventRecord", {event(src), stream(src)});
    call("mgpuStreamWaitEvent", {stream(dst), event(src)});
  }
  // pointer argument for a plan value (or null for `none`)
  CallArg ptr(int v) const {
    if (v < 0) return null();
    v = root[v];
    if (device == DeviceType::CPU) return plan.values[v].kind == PlanValue::Temp ? dev(buffer[v]) : host(v);
    return dev(buffer[v]);
  }
  int allocDevice(int v) {
    const int slot = prog.numDeviceBuffers++;
    call("mgpuMemAlloc", {i64((int64_t)plan.values[v].type.bytes()), stream(kData)}, dev(slot));
    buffer[v] = slot;
    return slot;
  }
  void ensureOnDevice(int v) {
    if (v < 0) return;
    v = root[v];
    if (buffer[v] >= 0) return;
    const int slot = allocDevice(v);
    call("mgpuMemcpy", {dev(slot), host(v), i64((int64_t)plan.values[v].type.bytes()), stream(kData)});
  }
  void dataWaitsForKernel() {
    if (!kernelAhead) return;
    record(kKernel, kData);
    kernelAhead = false;
  }
  void release(int v) {
    if (buffer[v] < 0) return;
    dataWaitsForKernel();
    call("mgpuMemFree", {dev(buffer[v]), stream(kData)});
    buffer[v] = -1;
  }
};

double attrNumber(const DeviceOp &op, const char *key, double fallback) {
  auto a = op.attrs.find(key);
  return a == op.attrs.end() ? fallback : a->second.number;
}
bool attrBool(const DeviceOp &op, const char *key, bool fallback) {
  auto a = op.attrs.find(key);
  return a == op.attrs.end() ? fallback : a->second.flag;
}
std::string attrString(const DeviceOp &op, const char *key, const char *fallback) {
  auto a = op.attrs.find(key);
  return a == op.attrs.end() ? std::string(fallback) : a->second.text;
}

// rows x cols view of a [..., n] tensor
void rowsCols(const TensorType &t, int64_t &m, int64_t &n) {
  n = t.shape.back();
  m = n ? t.numel() / n : 0;
}

const char *suffixOf(ElemType e) { return e == ElemType::F32 ? "F32" : e == ElemType::F16 ? "F16" : "BF16"; }

// Emits the library call(s) of one op.  `S` is the stream argument list tail:
// one stream on the GPU, nothing on the CPU.
bool emitOp(Lowering &L, const DeviceOp &op, std::string &error) {
  const DevicePlan &plan = L.plan;
  const bool gpu = L.device == DeviceType::GPU;
  auto in = [&](int i) { return L.ptr(op.operands[i]); };
  auto out = [&](int i) { return L.ptr(op.results[i]); };
  auto inT = [&](int i) -> const TensorType & { return plan.values[op.operands[i]].type; };
  auto withStream = [&](std::vector<CallArg> args) {
    if (gpu) args.push_back(stream(kKernel));
    return args;
  };
  auto noCpu = [&]() {
    error = "line " + std::to_string(op.line) + ": " + op.name + " has no CPU lowering";
    return false;
  };
  const std::string &n = op.name;
  if (n == "device.add") {
    L.call(gpu ? "mgpuAddF32" : "mcpuAddF32", withStream({in(0), in(1), out(0), i64(inT(0).numel())}));
    return true;
  }
  if (n == "device.layernorm") {
    int64_t m, cols;
    rowsCols(inT(0), m, cols);
    if (!gpu && inT(0).elem == ElemType::BF16) return noCpu();
    L.call(std::string(gpu ? "mgpuLayerNorm" : "mcpuLayerNorm") + suffixOf(inT(0).elem),
           withStream({in(0), in(1), in(2), out(0), f32(attrNumber(op, "eps", 1e-5)), i32(m), i32(cols)}));
    return true;
  }
  if (n == "device.add-residual-layernorm") {
    if (!gpu && inT(0).elem == ElemType::BF16) return noCpu();
    int64_t m, cols;
    rowsCols(inT(0), m, cols);
    L.call(std::string(gpu ? "mgpuAddResidualPreLayerNorm" : "mcpuAddResidualPreLayerNorm") + suffixOf(inT(0).elem),
           withStream({in(0), in(1), in(2), in(3), out(0), out(1), f32(attrNumber(op, "eps", 1e-5)), i32(m), i32(cols)}));
    return true;
  }
  if (n == "device.matmul" || n == "device.matmul-ex") {
    int64_t m, k;
    rowsCols(inT(0), m, k);
    const int64_t nn = inT(1).shape[1];
    if (n == "device.matmul") {
      // argument order (…, M, N, K, stream) of ConvertDeviceToLLVM.cpp:433-441
      L.call(gpu ? "mgpuMatmul" : "mcpuMatmul", withStream({in(0), in(1), in(2), out(0), i64(m), i64(nn), i64(k)}));
      return true;
    }
    if (!gpu && inT(0).elem == ElemType::BF16) return noCpu();
    const std::string act = attrString(op, "act", "none");
    const int actCode = act == "relu" ? 1 : act == "gelu" ? 2 : 0;
    L.call(std::string(gpu ? "mgpuMatmulEx" : "mcpuMatmulEx") + suffixOf(inT(0).elem),
           withStream({in(0), in(1), in(2), out(0), in(3), i64(m), i64(nn), i64(k), i32(op.operands[2] >= 0),
                       i32(actCode), i32(op.operands[3] >= 0)}));
    return true;
  }
  if (n == "device.conv2d" || n == "device.pool2d") {
    auto ints = [&](const char *key, std::vector<int64_t> fallback) {
      auto a = op.attrs.find(key);
      return a == op.attrs.end() ? fallback : a->second.ints;
    };
    const TensorType &x = inT(0), &y = plan.values[op.results[0]].type;
    const std::vector<int64_t> pad = ints("pad", {0, 0, 0, 0}), stride = ints("stride", {1, 1});
    std::vector<CallArg> args;
    if (n == "device.conv2d") {
      // argument order of ConvertDeviceToLLVM.cpp:533-548: pointers, N IC H W OC KH KW OH OW,
      // PHL PWL PHR PWR SH SW DH DW, hasPostAdd, containRelu
      const TensorType &w = inT(1);
      const std::vector<int64_t> dil = ints("dilation", {1, 1});
      args = {in(0), in(1), in(2), out(0), in(3)};
      for (int64_t v : {x.shape[0], x.shape[1], x.shape[2], x.shape[3], w.shape[0], w.shape[2], w.shape[3], y.shape[2],
                        y.shape[3], pad[0], pad[1], pad[2], pad[3], stride[0], stride[1], dil[0], dil[1]})
        args.push_back(i64(v));
      args.push_back(boolean(op.operands[3] >= 0));
      args.push_back(boolean(attrBool(op, "containRelu", false)));
      L.call(gpu ? "mgpuConv2d" : "mcpuConv2d", withStream(args));
    } else {
      const std::vector<int64_t> k = ints("kernel", {1, 1});
      args = {in(0), out(0)};
      for (int64_t v : {x.shape[0], x.shape[1], x.shape[2], x.shape[3], y.shape[2], y.shape[3], k[0], k[1], pad[0], pad[1],
                        pad[2], pad[3], stride[0], stride[1], (int64_t)(attrString(op, "method", "max") == "avg")})
        args.push_back(i64(v));
      L.call(gpu ? "mgpuPool2d" : "mcpuPool2d", withStream(args));
    }
    return true;
  }
  if (n == "device.cast") {
    const ElemType from = inT(0).elem, to = plan.values[op.results[0]].type.elem;
    if (!gpu && (from == ElemType::BF16 || to == ElemType::BF16)) return noCpu();
    std::string callee = from == ElemType::F32 ? (to == ElemType::BF16 ? "mgpuCastF32ToBF16" : "mgpuCastF32ToF16")
                                               : (from == ElemType::BF16 ? "mgpuCastBF16ToF32" : "mgpuCastF16ToF32");
    if (!gpu) callee[1] = 'c'; // mcpuCast...
    L.call(callee, withStream({out(0), in(0), i64(inT(0).numel())}));
    return true;
  }
  if (n == "device.fused-mha") {
    const TensorType &q = inT(0);
    if (!gpu && q.elem != ElemType::F16) return noCpu();
    const double scale = attrNumber(op, "scale", 1.0 / std::sqrt((double)q.shape[4]));
    L.call(std::string(gpu ? "mgpuFusedMHA" : "mcpuFusedMHA") + suffixOf(q.elem),
           withStream({in(0), in(1), out(0), i32(q.shape[0]), i32(q.shape[1]), i32(q.shape[3]), i32(q.shape[4]),
                       f32(scale), i32(attrBool(op, "causal", false))}));
    return true;
  }
  if (n == "device.multi-head-attention-layer") {
    const TensorType &x = inT(0);
    // argument order of ConvertDeviceToLLVM.cpp:741-748 (the CPU twin: the same without the stream)
    L.call(gpu ? "mgpuLLMDecodingContextLayer" : "mcpuLLMDecodingContextLayer",
           withStream({in(0), in(1), in(2), in(3), in(4), in(5), in(6), in(7), out(0), i64(x.shape[0]), i64(x.shape[1]),
                       i64(x.shape[2]), i64(inT(4).shape[1]), i64((int64_t)attrNumber(op, "head_num", 0)),
                       boolean(attrBool(op, "norm_first", true)), boolean(attrBool(op, "is_casual", true)),
                       boolean(attrString(op, "act", "relu") == "relu")}));
    return true;
  }
  if (n == "device.bert-encoder-layer") {
    const TensorType &x = inT(0);
    std::vector<CallArg> args;
    for (int i = 0; i < 14; i++) args.push_back(in(i));
    args.push_back(out(0));
    for (int64_t v : {x.shape[0], x.shape[1], x.shape[2], inT(7).shape[1], (int64_t)attrNumber(op, "head_num", 0)})
      args.push_back(i64(v));
    args.push_back(f32(attrNumber(op, "eps", 1e-5)));
    L.call(gpu ? "mgpuBertEncoderLayerF16" : "mcpuBertEncoderLayerF16", withStream(args));
    return true;
  }
  if (n == "gpu.launch_func") {
    if (!gpu) return noCpu();
    // bare-pointer convention of GPUOffloadingAttr.cpp:283-304: operand
    // pointers, result pointers, then the i64 scalars
    CallArg params;
    params.kind = CallArg::Params;
    for (size_t i = 0; i < op.operands.size(); i++) params.pack.push_back(in((int)i));
    for (size_t i = 0; i < op.results.size(); i++) params.pack.push_back(out((int)i));
    auto sc = op.attrs.find("scalars");
    if (sc != op.attrs.end())
      for (int64_t v : sc->second.ints) params.pack.push_back(i64(v));
    const auto &b = op.attrs.find("blocks")->second.ints;
    const auto &t = op.attrs.find("threads")->second.ints;
    const int fn = L.prog.numDeviceBuffers++; // the function handle takes a slot of its own
    L.call("mgpuModuleGetFunction", {symbol(attrString(op, "kernel", ""))}, dev(fn));
    L.call("mgpuLaunchKernel", {dev(fn), i64(b[0]), i64(b[1]), i64(b[2]), i64(t[0]), i64(t[1]), i64(t[2]),
                                i32((int64_t)attrNumber(op, "smem", 0)), stream(kKernel), params, null()});
    return true;
  }
  error = "line " + std::to_string(op.line) + ": " + op.name + ": unknown op";
  return false;
}

} // namespace

bool lowerToRuntimeCalls(const DevicePlan &plan, DeviceType device, RuntimeProgram &prog, std::string &error) {
  if (!verifyDevicePlan(plan, error)) return false;
  prog = RuntimeProgram();
  prog.device = device;
  Lowering L{plan, prog, device, std::vector<int>(plan.values.size(), -1), std::vector<int>(plan.values.size(), -1),
             std::vector<int>(plan.values.size())};
  for (size_t v = 0; v < plan.values.size(); v++) L.root[v] = (int)v;
  for (size_t o = 0; o < plan.ops.size(); o++) {
    const DeviceOp &op = plan.ops[o];
    if (op.name == "device.reshape") L.root[op.results[0]] = L.root[op.operands[0]];
    for (int v : op.operands)
      if (v >= 0) L.lastUse[L.root[v]] = (int)o;
  }

  if (device == DeviceType::CPU) {
    // temporaries are malloc'd host buffers, released behind their last reader
    std::vector<bool> allocated(plan.values.size(), false);
    for (size_t o = 0; o < plan.ops.size(); o++) {
      L.curOp = (int)o;
      const DeviceOp &op = plan.ops[o];
      const bool view = op.name == "device.reshape";
      for (int r : op.results)
        if (!view && plan.values[r].kind == PlanValue::Temp) {
          L.buffer[r] = prog.numDeviceBuffers++;
          L.call("malloc", {i64((int64_t)plan.values[r].type.bytes())}, dev(L.buffer[r]));
          allocated[r] = true;
        }
      if (!view && !emitOp(L, op, error)) return false;
      for (int operand : op.operands) {
        const int v = operand < 0 ? -1 : L.root[operand];
        if (v >= 0 && allocated[v] && L.lastUse[v] == (int)o) {
          L.call("free", {dev(L.buffer[v])});
          allocated[v] = false;
        }
      }
    }
    L.curOp = -1;
    for (size_t v = 0; v < plan.values.size(); v++)
      if (allocated[v]) L.call("free", {dev(L.buffer[v])});
    return true;
  }

  // ---- GPU ----------------------------------------------------------------
  prog.numStreams = prog.numEvents = 2;
  for (int s : {kData, kKernel}) {
    L.call("mgpuStreamCreate", {}, stream(s));
    L.call("mgpuEventCreateWithStream", {stream(s)}, event(s));
  }
  for (size_t o = 0; o < plan.ops.size(); o++) {
    L.curOp = (int)o;
    const DeviceOp &op = plan.ops[o];
    for (int v : op.operands) L.ensureOnDevice(v);
    if (op.name != "device.reshape") { // a view makes no call of its own
      for (int r : op.results) L.allocDevice(r);
      L.record(kData, kKernel);
      if (!emitOp(L, op, error)) return false;
      L.kernelAhead = true;
    }
    // buffers this op read last: release behind a record KernelStream -> DataStream
    for (size_t i = 0; i < op.operands.size(); i++) {
      const int v = op.operands[i] < 0 ? -1 : L.root[op.operands[i]];
      if (v < 0 || L.lastUse[v] != (int)o || plan.values[v].kind == PlanValue::Output) continue;
      L.release(v);
    }
    // results nobody reads and nobody receives
    for (int r : op.results)
      if (L.root[r] == r && L.lastUse[r] < 0 && plan.values[r].kind != PlanValue::Output) L.release(r);
  }
  L.curOp = -1;
  for (int o : plan.outputs) {
    L.dataWaitsForKernel();
    L.call("mgpuMemcpy", {host(o), dev(L.buffer[o]), i64((int64_t)plan.values[o].type.bytes()), stream(kData)});
    L.call("mgpuMemFree", {dev(L.buffer[o]), stream(kData)});
    L.buffer[o] = -1;
  }
  for (int s : {kData, kKernel}) {
    L.call("mgpuEventDestroy", {event(s)});
    L.call("mgpuStreamSynchronize", {stream(s)});
    L.call("mgpuStreamDestroy", {stream(s)});
  }
  return true;
}

namespace {

const char *streamName(int s) { return s == kData ? "%DataStream" : "%KernelStream"; }
const char *eventName(int e) { return e == kData ? "%DataEvent" : "%KernelEvent"; }

std::string printArg(const DevicePlan &plan, const CallArg &a) {
  std::ostringstream os;
  switch (a.kind) {
  case CallArg::Stream: os << streamName(a.index); break;
  case CallArg::Event: os << eventName(a.index); break;
  case CallArg::Device: os << "%d" << a.index; break;
  case CallArg::Host: os << "%" << plan.values[a.index].name; break;
  case CallArg::I64: os << a.i; break;
  case CallArg::I32: os << a.i << " : i32"; break;
  case CallArg::F32: os << a.f << " : f32"; break;
  case CallArg::Bool: os << (a.i ? "true" : "false"); break;
  case CallArg::Null: os << "null"; break;
  case CallArg::Symbol: os << '"' << a.text << '"'; break;
  case CallArg::Params:
    os << "[";
    for (size_t i = 0; i < a.pack.size(); i++) os << (i ? ", " : "") << "&" << printArg(plan, a.pack[i]);
    os << "]";
    break;
  }
  return os.str();
}

} // namespace

std::string printRuntimeProgram(const DevicePlan &plan, const RuntimeProgram &prog) {
  std::ostringstream os;
  int lastOp = -2;
  for (const RuntimeCall &c : prog.calls) {
    if (c.op != lastOp && c.op >= 0)
      os << "// " << plan.ops[c.op].name << " (line " << plan.ops[c.op].line << ")\n";
    lastOp = c.op;
    if (c.result.kind != CallArg::Null) os << printArg(plan, c.result) << " = ";
    os << c.callee << "(";
    for (size_t i = 0; i < c.args.size(); i++) os << (i ? ", " : "") << printArg(plan, c.args[i]);
    os << ")\n";
  }
  return os.str();
}

bool checkRuntimeProgram(const RuntimeProgram &prog, std::string &error) {
  if (prog.device != DeviceType::GPU) return true;
  enum { Absent, Live, Gone };
  std::vector<int> streams(prog.numStreams, Absent), events(prog.numEvents, Absent),
      buffers(prog.numDeviceBuffers, Absent);
  // Work is numbered per stream; seen[a][b] = how much of stream b's work
  // stream a is ordered behind.  An event carries the count of its stream at
  // record time.
  std::vector<int64_t> issued(prog.numStreams, 0), eventStamp(prog.numEvents, -1);
  std::vector<std::vector<int64_t>> seen(prog.numStreams, std::vector<int64_t>(prog.numStreams, 0));
  // per buffer: the stream and work number of its last write and of its last read
  struct Touch { int stream = -1; int64_t number = 0; };
  std::vector<Touch> lastWrite(prog.numDeviceBuffers), lastRead(prog.numDeviceBuffers);
  std::vector<bool> synced(prog.numStreams, false), owned(prog.numDeviceBuffers, false);
  size_t index = 0;
  auto fail = [&](const RuntimeCall &c, const std::string &msg) {
    error = "call " + std::to_string(index) + " (" + c.callee + "): " + msg;
    return false;
  };
  auto orderedAfter = [&](int s, const Touch &t) { return t.stream < 0 || t.stream == s || seen[s][t.stream] >= t.number; };
  for (; index < prog.calls.size(); index++) {
    const RuntimeCall &c = prog.calls[index];
    // handle states
    for (const CallArg &a : c.args) {
      std::vector<const CallArg *> all{&a};
      if (a.kind == CallArg::Params)
        for (const CallArg &p : a.pack) all.push_back(&p);
      for (const CallArg *x : all) {
        if (x->kind == CallArg::Stream && streams[x->index] != Live) return fail(c, "stream is not live");
        if (x->kind == CallArg::Event && events[x->index] != Live) return fail(c, "event is not live");
        if (x->kind == CallArg::Device && buffers[x->index] != Live) return fail(c, "device buffer is not live");
      }
    }
    const std::string &n = c.callee;
    if (n == "mgpuStreamCreate") { streams[c.result.index] = Live; continue; }
    if (n == "mgpuEventCreateWithStream") { events[c.result.index] = Live; continue; }
    if (n == "mgpuModuleGetFunction") { buffers[c.result.index] = Live; continue; }
    if (n == "mgpuEventRecord") { eventStamp[c.args[0].index] = issued[c.args[1].index]; continue; }
    if (n == "mgpuStreamWaitEvent") {
      const int s = c.args[0].index, e = c.args[1].index;
      if (eventStamp[e] < 0) return fail(c, "waits for an event that was never recorded");
      // events belong to the stream of the same slot
      if (seen[s][e] < eventStamp[e]) seen[s][e] = eventStamp[e];
      continue;
    }
    if (n == "mgpuEventDestroy") { events[c.args[0].index] = Gone; continue; }
    if (n == "mgpuStreamSynchronize") { synced[c.args[0].index] = true; continue; }
    if (n == "mgpuStreamDestroy") {
      if (!synced[c.args[0].index]) return fail(c, "stream destroyed without a synchronize");
      streams[c.args[0].index] = Gone;
      continue;
    }
    // everything else is work on the stream named by its (single) stream argument
    int s = -1;
    for (const CallArg &a : c.args)
      if (a.kind == CallArg::Stream) s = a.index;
    if (s < 0) return fail(c, "no stream argument");
    const int64_t number = ++issued[s];
    synced[s] = false;
    if (n == "mgpuMemAlloc") {
      if (s != kData) return fail(c, "allocation outside the data stream");
      buffers[c.result.index] = Live;
      owned[c.result.index] = true;
      lastWrite[c.result.index] = Touch{s, number}; // stream-ordered allocation
      continue;
    }
    std::vector<int> reads, writes;
    if (n == "mgpuMemcpy") {
      if (s != kData) return fail(c, "copy outside the data stream");
      if (c.args[0].kind == CallArg::Device) writes.push_back(c.args[0].index);
      if (c.args[1].kind == CallArg::Device) reads.push_back(c.args[1].index);
    } else if (n == "mgpuMemFree") {
      if (s != kData) return fail(c, "free outside the data stream");
      writes.push_back(c.args[0].index); // a free conflicts with reads and writes alike
    } else {
      if (s != kKernel) return fail(c, "op outside the kernel stream");
      // library ops and launches: conservatively read and write every buffer they name
      for (const CallArg &a : c.args) {
        if (a.kind == CallArg::Device && n != "mgpuLaunchKernel") { reads.push_back(a.index); writes.push_back(a.index); }
        if (a.kind == CallArg::Params)
          for (const CallArg &p : a.pack)
            if (p.kind == CallArg::Device) { reads.push_back(p.index); writes.push_back(p.index); }
      }
    }
    for (int b : reads)
      if (!orderedAfter(s, lastWrite[b])) return fail(c, "reads %d" + std::to_string(b) + " without waiting for its writer");
    for (int b : writes)
      if (!orderedAfter(s, lastWrite[b]) || !orderedAfter(s, lastRead[b]))
        return fail(c, "touches %d" + std::to_string(b) + " without waiting for its last user");
    for (int b : reads) lastRead[b] = Touch{s, number};
    for (int b : writes) lastWrite[b] = Touch{s, number};
    if (n == "mgpuMemFree") buffers[c.args[0].index] = Gone;
  }
  for (size_t s = 0; s < streams.size(); s++)
    if (streams[s] != Gone) { error = "a stream is still live at the end"; return false; }
  for (size_t e = 0; e < events.size(); e++)
    if (events[e] != Gone) { error = "an event is still live at the end"; return false; }
  for (size_t b = 0; b < buffers.size(); b++)
    if (owned[b] && buffers[b] != Gone) { error = "device buffer %d" + std::to_string(b) + " is never freed"; return false; }
  return true;
}

} // namespace conversion
} // namespace multi_device
