// Shared pieces of the hand-lowered model libraries: what the reference's
// `multi-device-opt --mlir-to-gpu` + `multi-device-lib-generate` pipeline emits
// as host code, written by hand.  The call sequence follows the lowering:
// two streams (data / kernel) with one event each
// (lib/Dialect/Device/Transform/AsyncDependencyConvert.cpp:49-56), device
// buffers + host-to-device copies on the data stream
// (DeviceDataCopyGeneration.cpp:26-43), record / wait for cross-stream edges
// (lib/Conversion/ConvertDeviceToLLVM/ConvertDeviceToLLVM.cpp:376-396), the op,
// the copy back, and the final device.wait = destroy event, synchronise and
// destroy each stream (:345-354).  The result buffer is malloc'd here and handed
// back through the output descriptor (examples/add.ll:9-33,80-104).
#pragma once

#include "mgpu_runtime.h"

#include <cstdint>
#include <cstdlib>

template <int N> struct MemRef {
  void *allocated;
  void *aligned;
  intptr_t offset;
  intptr_t sizes[N];
  intptr_t strides[N];
  int64_t numel() const {
    int64_t n = 1;
    for (int i = 0; i < N; i++) n *= sizes[i];
    return n;
  }
  void *data() const { return aligned; }
};

// 64-byte aligned result buffer in the style of add.ll:9-14: `allocated` is
// what free() takes, `aligned` what the data starts at.
template <int N> inline void allocResult(MemRef<N> *out, const intptr_t (&sizes)[N], size_t elemBytes) {
  int64_t n = 1;
  for (int i = 0; i < N; i++) n *= sizes[i];
  void *raw = std::malloc((size_t)n * elemBytes + 64);
  out->allocated = raw;
  out->aligned = reinterpret_cast<void *>((reinterpret_cast<uintptr_t>(raw) + 63) / 64 * 64);
  out->offset = 0;
  intptr_t running = 1;
  for (int i = N - 1; i >= 0; i--) {
    out->sizes[i] = sizes[i];
    out->strides[i] = running;
    running *= sizes[i];
  }
}

struct TwoStreams {
  mgpuStream_t data, kernel;
  mgpuEvent_t dataEvent, kernelEvent;
  TwoStreams() {
    data = mgpuStreamCreate();
    kernel = mgpuStreamCreate();
    dataEvent = mgpuEventCreateWithStream(data);
    kernelEvent = mgpuEventCreateWithStream(kernel);
  }
  // kernel stream waits for everything queued on the data stream so far
  void dataToKernel() {
    mgpuEventRecord(dataEvent, data);
    mgpuStreamWaitEvent(kernel, dataEvent);
  }
  void kernelToData() {
    mgpuEventRecord(kernelEvent, kernel);
    mgpuStreamWaitEvent(data, kernelEvent);
  }
  ~TwoStreams() {
    mgpuEventDestroy(dataEvent);
    mgpuStreamSynchronize(data);
    mgpuStreamDestroy(data);
    mgpuEventDestroy(kernelEvent);
    mgpuStreamSynchronize(kernel);
    mgpuStreamDestroy(kernel);
  }
};
