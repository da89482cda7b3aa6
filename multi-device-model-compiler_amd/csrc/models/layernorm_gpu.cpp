// GPU model library: LayerNorm over the last dim of a rank-3 fp32 tensor,
// main_graph(out, x[B,S,N], gamma[N], beta[N]), eps = 1e-5, as a library-op
// call on the kernel stream (the form ConvertDeviceToLLVM.cpp:410-442 gives
// device ops: pointers, dims, stream last).
#include "model_common.h"
#include "mgpu_ops.h"

extern "C" void _mlir_ciface_main_graph(MemRef<3> *out, MemRef<3> *x, MemRef<1> *gamma,
                                        MemRef<1> *beta) {
  const int64_t n = x->sizes[2], m = x->sizes[0] * x->sizes[1];
  const size_t bytes = (size_t)m * n * sizeof(float), vbytes = (size_t)n * sizeof(float);
  allocResult(out, x->sizes, sizeof(float));

  TwoStreams s;
  float *dx = static_cast<float *>(mgpuMemAlloc(bytes, s.data));
  float *dy = static_cast<float *>(mgpuMemAlloc(bytes, s.data));
  float *dg = static_cast<float *>(mgpuMemAlloc(vbytes, s.data));
  float *db = static_cast<float *>(mgpuMemAlloc(vbytes, s.data));
  mgpuMemcpy(dx, x->data(), bytes, s.data);
  mgpuMemcpy(dg, gamma->data(), vbytes, s.data);
  mgpuMemcpy(db, beta->data(), vbytes, s.data);
  s.dataToKernel();
  mgpuLayerNormF32(dx, dg, db, dy, 1e-5f, (int32_t)m, (int32_t)n, s.kernel);
  s.kernelToData();
  mgpuMemcpy(out->data(), dy, bytes, s.data);
  mgpuStreamSynchronize(s.data);
  mgpuMemFree(dx, s.data);
  mgpuMemFree(dy, s.data);
  mgpuMemFree(dg, s.data);
  mgpuMemFree(db, s.data);
}
