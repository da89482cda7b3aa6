// Host tensors in MLIR's ranked-memref descriptor ABI.
//
// Same layout and member names as the reference's
// include/multi-device-model-compiler/Runtime/TensorDescripter.h:9-81
// ({allocated, aligned, offset, sizes[N], strides[N]}), which is what a
// compiled model's `_mlir_ciface_*` entry point unpacks (examples/add.ll:80-104).
// Differences: any trivially copyable element type (the runners also carry
// fp16 tensors as uint16_t), ranks 1..5, and clear() releases with free():
// both the model (malloc, add.ll:9) and InitData (aligned_alloc) allocate with
// the C allocator, where the reference's clear() used `delete` (:67-71).
#ifndef MULTI_DEVICE_MODEL_COMPILER_RUNTIME_TENSORDESCRIPTER_H_
#define MULTI_DEVICE_MODEL_COMPILER_RUNTIME_TENSORDESCRIPTER_H_

#include <cstddef>
#include <cstdint>
#include <cstdlib>
#include <vector>

template <typename T, size_t N> struct TensorDescriptor {
  T *allocated = nullptr;
  T *aligned = nullptr;
  intptr_t offset;
  intptr_t sizes[N];
  intptr_t strides[N];

  static TensorDescriptor *CreateTensor(std::vector<size_t> &sizes);
  void InitData();
  void InitData(T *data);
  size_t GetNumElements();
  void clear();
};

template <typename T, size_t N>
TensorDescriptor<T, N> *TensorDescriptor<T, N>::CreateTensor(std::vector<size_t> &sizes) {
  auto *tensor = static_cast<TensorDescriptor<T, N> *>(std::malloc(sizeof(TensorDescriptor<T, N>)));
  tensor->allocated = nullptr;
  tensor->aligned = nullptr;
  tensor->offset = 0;
  intptr_t running = 1;
  for (int64_t i = (int64_t)N - 1; i >= 0; --i) {
    tensor->sizes[i] = (intptr_t)sizes[i];
    tensor->strides[i] = running;
    running *= tensor->sizes[i];
  }
  return tensor;
}

template <typename T, size_t N> void TensorDescriptor<T, N>::InitData() {
  // aligned_alloc wants a size that is a multiple of the alignment.
  const size_t bytes = (GetNumElements() * sizeof(T) + 63) / 64 * 64;
  T *data = static_cast<T *>(std::aligned_alloc(64, bytes ? bytes : 64));
  allocated = data;
  aligned = data;
}

template <typename T, size_t N> void TensorDescriptor<T, N>::InitData(T *data) {
  allocated = data;
  aligned = data;
}

template <typename T, size_t N> size_t TensorDescriptor<T, N>::GetNumElements() {
  size_t num = 1;
  for (auto &siz : sizes)
    num *= (size_t)siz;
  return num;
}

template <typename T, size_t N> void TensorDescriptor<T, N>::clear() {
  if (allocated)
    std::free(allocated);
  allocated = nullptr;
  aligned = nullptr;
}

template <size_t N> using FloatTensor = TensorDescriptor<float, N>;
using Float1DTensor = FloatTensor<1>;
using Float2DTensor = FloatTensor<2>;
using Float3DTensor = FloatTensor<3>;
using FLoat4DTensor = FloatTensor<4>; // spelling kept from the reference (:79)
using Float5DTensor = FloatTensor<5>;

#endif
