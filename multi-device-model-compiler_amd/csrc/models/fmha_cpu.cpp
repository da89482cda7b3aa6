// CPU model library: the same attention graph through the CPU op library.
#include "model_common.h"
#include "multi-device-model-compiler/Kernels/CPU/Ops.h"

#include <cmath>

extern "C" void _mlir_ciface_main_graph(MemRef<3> *out, MemRef<5> *qkv) {
  const int64_t B = qkv->sizes[0], S = qkv->sizes[1], H = qkv->sizes[3], D = qkv->sizes[4];
  const intptr_t osz[3] = {(intptr_t)B, (intptr_t)S, (intptr_t)(H * D)};
  allocResult(out, osz, 2);
  mcpuFusedMHAF16(qkv->data(), nullptr, out->data(), (int32_t)B, (int32_t)S, (int32_t)H, (int32_t)D,
                  1.0f / std::sqrt((float)D), 0);
}
