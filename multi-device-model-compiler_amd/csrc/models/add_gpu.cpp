// GPU model library for examples/add.onnx: C = A + B on (3,640,640) fp32 (any
// rank-3 shape works).  The add runs as the generated-style kernel
// `main_graph_kernel` from the loaded code object, looked up by name and
// launched through mgpuLaunchKernel with bare-pointer arguments
// (lib/Dialect/Device/IR/GPUOffloadingAttr.cpp:283-304).
#include "model_common.h"

extern "C" void _mlir_ciface_main_graph(MemRef<3> *out, MemRef<3> *a, MemRef<3> *b) {
  const int64_t n = a->numel();
  const size_t bytes = (size_t)n * sizeof(float);
  allocResult(out, a->sizes, sizeof(float));

  TwoStreams s;
  void *da = mgpuMemAlloc(bytes, s.data);
  void *db = mgpuMemAlloc(bytes, s.data);
  void *dc = mgpuMemAlloc(bytes, s.data);
  mgpuMemcpy(da, a->data(), bytes, s.data);
  mgpuMemcpy(db, b->data(), bytes, s.data);
  s.dataToKernel();

  mgpuFunction_t fn = mgpuModuleGetFunction("main_graph_kernel");
  int64_t count = n;
  void *params[] = {&da, &db, &dc, &count};
  const int64_t n4 = n / 4 > 0 ? n / 4 : 1;
  int64_t blocks = (n4 + 255) / 256;
  if (blocks > 256 * 16) blocks = 256 * 16;
  mgpuLaunchKernel(fn, blocks, 1, 1, 256, 1, 1, 0, s.kernel, params, nullptr);
  s.kernelToData();

  mgpuMemcpy(out->data(), dc, bytes, s.data);
  mgpuStreamSynchronize(s.data);
  mgpuMemFree(da, s.data);
  mgpuMemFree(db, s.data);
  mgpuMemFree(dc, s.data);
}
