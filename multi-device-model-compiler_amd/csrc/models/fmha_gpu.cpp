// GPU model library: fused multi-head attention on packed fp16 QKV,
// main_graph(out[B,S,H*D], qkv[B,S,3,H,D]); run the runner with --dtype f16.
// No mask, softmax scale 1/sqrt(D).
#include "model_common.h"
#include "mgpu_ops.h"

#include <cmath>

extern "C" void _mlir_ciface_main_graph(MemRef<3> *out, MemRef<5> *qkv) {
  const int64_t B = qkv->sizes[0], S = qkv->sizes[1], H = qkv->sizes[3], D = qkv->sizes[4];
  const intptr_t osz[3] = {(intptr_t)B, (intptr_t)S, (intptr_t)(H * D)};
  allocResult(out, osz, 2);
  const size_t inBytes = (size_t)qkv->numel() * 2, outBytes = (size_t)(B * S * H * D) * 2;

  TwoStreams s;
  void *dq = mgpuMemAlloc(inBytes, s.data);
  void *dout = mgpuMemAlloc(outBytes, s.data);
  mgpuMemcpy(dq, qkv->data(), inBytes, s.data);
  s.dataToKernel();
  mgpuFusedMHAF16(dq, nullptr, dout, (int32_t)B, (int32_t)S, (int32_t)H, (int32_t)D,
                  1.0f / std::sqrt((float)D), 0, s.kernel);
  s.kernelToData();
  mgpuMemcpy(out->data(), dout, outBytes, s.data);
  mgpuStreamSynchronize(s.data);
  mgpuMemFree(dq, s.data);
  mgpuMemFree(dout, s.data);
}
