// CPU model library: the same LayerNorm graph through the CPU op library.
#include "model_common.h"
#include "multi-device-model-compiler/Kernels/CPU/Ops.h"

extern "C" void _mlir_ciface_main_graph(MemRef<3> *out, MemRef<3> *x, MemRef<1> *gamma,
                                        MemRef<1> *beta) {
  allocResult(out, x->sizes, sizeof(float));
  mcpuLayerNormF32(static_cast<const float *>(x->data()), static_cast<const float *>(gamma->data()),
                   static_cast<const float *>(beta->data()), static_cast<float *>(out->data()), 1e-5f,
                   (int32_t)(x->sizes[0] * x->sizes[1]), (int32_t)x->sizes[2]);
}
