// CPU model library for examples/add.onnx, the hand-written twin of the
// reference's pre-lowered examples/add.ll:8-104: malloc a 64-byte aligned
// result, one single-threaded elementwise fadd loop nest, descriptor returned
// through the first argument.
#include "model_common.h"

extern "C" void _mlir_ciface_main_graph(MemRef<3> *out, MemRef<3> *a, MemRef<3> *b) {
  allocResult(out, a->sizes, sizeof(float));
  const float *pa = static_cast<const float *>(a->data()) + a->offset;
  const float *pb = static_cast<const float *>(b->data()) + b->offset;
  float *pc = static_cast<float *>(out->data());
  for (intptr_t i = 0; i < a->sizes[0]; i++)
    for (intptr_t j = 0; j < a->sizes[1]; j++)
      for (intptr_t k = 0; k < a->sizes[2]; k++) {
        const intptr_t ia = i * a->strides[0] + j * a->strides[1] + k * a->strides[2];
        const intptr_t ib = i * b->strides[0] + j * b->strides[1] + k * b->strides[2];
        const intptr_t ic = i * out->strides[0] + j * out->strides[1] + k * out->strides[2];
        pc[ic] = pa[ia] + pb[ib];
      }
}
