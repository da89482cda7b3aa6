// Device runtime for one MI355X: the `mgpu*` C ABI (include/mgpu_runtime.h)
// written directly on the HIP runtime and module API.
//
// Counterpart of lib/Runtime/CUDA/CudaRuntimeWrappers.cpp:23-299 of the
// reference (CUDA driver API).  Differences that matter on this hardware:
//  * no context push/pop: HIP has one primary context per device, selected
//    with hipSetDevice from the thread-local default ordinal;
//  * the per-launch device-attribute query and function-attribute write of
//    the reference (:118-131) are replaced by one cached LDS limit per device,
//    so a launch is a single hipModuleLaunchKernel;
//  * the code object is a gfx950 .hsaco instead of a cubin.
#include "mgpu_runtime.h"

#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>

namespace {

thread_local int32_t defaultDevice = 0;
thread_local int32_t lastError = 0;
thread_local bool deviceBound = false;

constexpr const char *kDebugEnvironmentVariable = "MULTI_DEVICE_HIP_DEBUG";

bool isDebugEnabled() {
  static const bool enabled = std::getenv(kDebugEnvironmentVariable) != nullptr;
  return enabled;
}

void report(hipError_t result, const char *expr) {
  if (result == hipSuccess)
    return;
  const char *name = hipGetErrorName(result);
  if (!name)
    name = "<unknown>";
  std::fprintf(stderr, "'%s' failed with '%s'\n", expr, name);
  lastError = static_cast<int32_t>(result);
  // Leave no sticky "last error" behind for unrelated later calls.
  (void)hipGetLastError();
}

#define HIP_REPORT_IF_ERROR(expr) report((expr), #expr)

#define debug_print(fmt, ...)                                                  \
  do {                                                                         \
    if (isDebugEnabled())                                                      \
      std::fprintf(stderr, "%s:%d:%s(): " fmt, "HipRuntimeWrappers.cpp",       \
                   __LINE__, __func__, __VA_ARGS__);                           \
  } while (0)

// Binds the calling thread to the default device once (and again after
// mgpuSetDefaultDevice changed it).
void bindDevice() {
  if (deviceBound)
    return;
  HIP_REPORT_IF_ERROR(hipSetDevice(defaultDevice));
  deviceBound = true;
}

int32_t maxLdsBytes() {
  static thread_local int32_t cachedFor = -1;
  static thread_local int32_t cached = 0;
  if (cachedFor != defaultDevice) {
    int value = 0;
    HIP_REPORT_IF_ERROR(hipDeviceGetAttribute(
        &value, hipDeviceAttributeMaxSharedMemoryPerBlock, defaultDevice));
    cached = value;
    cachedFor = defaultDevice;
  }
  return cached;
}

hipModule_t module = nullptr;

inline hipStream_t S(mgpuStream_t s) { return reinterpret_cast<hipStream_t>(s); }
inline hipEvent_t E(mgpuEvent_t e) { return reinterpret_cast<hipEvent_t>(e); }

} // namespace

extern "C" {

void mgpuModuleFileLoad(const char *fname) {
  bindDevice();
  HIP_REPORT_IF_ERROR(hipModuleLoad(&module, fname));
}

void mgpuModuleUnload() {
  if (module)
    HIP_REPORT_IF_ERROR(hipModuleUnload(module));
  module = nullptr;
}

mgpuFunction_t mgpuModuleGetFunction(const char *name) {
  hipFunction_t function = nullptr;
  HIP_REPORT_IF_ERROR(hipModuleGetFunction(&function, module, name));
  return reinterpret_cast<mgpuFunction_t>(function);
}

void mgpuLaunchKernel(mgpuFunction_t function, intptr_t gridX, intptr_t gridY,
                      intptr_t gridZ, intptr_t blockX, intptr_t blockY,
                      intptr_t blockZ, int32_t smem, mgpuStream_t stream,
                      void **params, void **extra) {
  bindDevice();
  const int32_t maxShmem = maxLdsBytes();
  if (maxShmem < smem) {
    std::fprintf(stderr,
                 "Requested shared memory (%dkb) is larger than maximum allowed "
                 "shared memory (%dkb) for this device\n",
                 smem, maxShmem);
  }
  debug_print("Launching kernel, grid=%ld,%ld,%ld, "
              "threads: %ld, %ld, %ld, "
              "smem: %dkb\n",
              (long)gridX, (long)gridY, (long)gridZ, (long)blockX, (long)blockY,
              (long)blockZ, smem);
  if (!function) {
    report(hipErrorInvalidDeviceFunction, "mgpuLaunchKernel(function == nullptr)");
    return;
  }
  HIP_REPORT_IF_ERROR(hipModuleLaunchKernel(
      reinterpret_cast<hipFunction_t>(function), (unsigned)gridX,
      (unsigned)gridY, (unsigned)gridZ, (unsigned)blockX, (unsigned)blockY,
      (unsigned)blockZ, (unsigned)smem, S(stream), params, extra));
}

mgpuStream_t mgpuStreamCreate() {
  bindDevice();
  hipStream_t stream = nullptr;
  HIP_REPORT_IF_ERROR(hipStreamCreateWithFlags(&stream, hipStreamNonBlocking));
  return stream;
}

void mgpuStreamDestroy(mgpuStream_t stream) {
  HIP_REPORT_IF_ERROR(hipStreamDestroy(S(stream)));
}

void mgpuStreamSynchronize(mgpuStream_t stream) {
  HIP_REPORT_IF_ERROR(hipStreamSynchronize(S(stream)));
}

void mgpuStreamWaitEvent(mgpuStream_t stream, mgpuEvent_t event) {
  HIP_REPORT_IF_ERROR(hipStreamWaitEvent(S(stream), E(event), /*flags=*/0));
}

mgpuEvent_t mgpuEventCreate() {
  bindDevice();
  hipEvent_t event = nullptr;
  HIP_REPORT_IF_ERROR(hipEventCreateWithFlags(&event, hipEventDisableTiming));
  return event;
}

mgpuEvent_t mgpuEventCreateWithStream(mgpuStream_t /*stream*/) {
  return mgpuEventCreate();
}

mgpuEvent_t mgpuEventEnableTimeCreate() {
  bindDevice();
  hipEvent_t event = nullptr;
  HIP_REPORT_IF_ERROR(hipEventCreateWithFlags(&event, hipEventDefault));
  return event;
}

void mgpuEventDestroy(mgpuEvent_t event) {
  HIP_REPORT_IF_ERROR(hipEventDestroy(E(event)));
}

void mgpuEventSynchronize(mgpuEvent_t event) {
  HIP_REPORT_IF_ERROR(hipEventSynchronize(E(event)));
}

void mgpuEventRecord(mgpuEvent_t event, mgpuStream_t stream) {
  HIP_REPORT_IF_ERROR(hipEventRecord(E(event), S(stream)));
}

float mgpuEventElapsedTime(mgpuEvent_t begin, mgpuEvent_t end) {
  float elapsed = 0;
  HIP_REPORT_IF_ERROR(hipEventElapsedTime(&elapsed, E(begin), E(end)));
  return elapsed;
}

void *mgpuMemAlloc(uint64_t sizeBytes, mgpuStream_t /*stream*/) {
  bindDevice();
  void *ptr = nullptr;
  HIP_REPORT_IF_ERROR(hipMalloc(&ptr, sizeBytes));
  return ptr;
}

void mgpuMemFree(void *ptr, mgpuStream_t /*stream*/) {
  HIP_REPORT_IF_ERROR(hipFree(ptr));
}

void *mgpuMemAllocAsync(uint64_t sizeBytes, mgpuStream_t stream) {
  bindDevice();
  void *ptr = nullptr;
  HIP_REPORT_IF_ERROR(hipMallocAsync(&ptr, sizeBytes, S(stream)));
  return ptr;
}

void mgpuMemFreeAsync(void *ptr, mgpuStream_t stream) {
  HIP_REPORT_IF_ERROR(hipFreeAsync(ptr, S(stream)));
}

void mgpuMemcpy(void *dst, void *src, size_t sizeBytes, mgpuStream_t stream) {
  HIP_REPORT_IF_ERROR(
      hipMemcpyAsync(dst, src, sizeBytes, hipMemcpyDefault, S(stream)));
}

void mgpuMemset32(void *dst, unsigned int value, size_t count,
                  mgpuStream_t stream) {
  HIP_REPORT_IF_ERROR(hipMemsetD32Async(reinterpret_cast<hipDeviceptr_t>(dst),
                                        (int)value, count, S(stream)));
}

void mgpuMemset16(void *dst, unsigned short value, size_t count,
                  mgpuStream_t stream) {
  HIP_REPORT_IF_ERROR(hipMemsetD16Async(reinterpret_cast<hipDeviceptr_t>(dst),
                                        value, count, S(stream)));
}

void mgpuMemHostRegister(void *ptr, uint64_t sizeBytes) {
  bindDevice();
  HIP_REPORT_IF_ERROR(hipHostRegister(ptr, sizeBytes, /*flags=*/0));
}

void mgpuMemHostUnregister(void *ptr) {
  HIP_REPORT_IF_ERROR(hipHostUnregister(ptr));
}

namespace {
// Ranked memref descriptor viewed as bytes: two pointers, an offset, then
// `rank` sizes followed by `rank` strides.
struct MemRefHeader {
  char *allocated;
  char *aligned;
  int64_t offset;
  int64_t sizesAndStrides[1];
};
} // namespace

void mgpuMemHostRegisterMemRef(int64_t rank, void *descriptor,
                               int64_t elementSizeBytes) {
  auto *desc = static_cast<MemRefHeader *>(descriptor);
  const int64_t *sizes = desc->sizesAndStrides;
  const int64_t *strides = sizes + rank;
  // Only densely packed tensors are supported, as in the reference.
  int64_t running = 1;
  for (int64_t i = rank - 1; i >= 0; --i) {
    if (strides[i] != running) {
      std::fprintf(stderr, "mgpuMemHostRegisterMemRef: Mismatch in computed dense strides\n");
      lastError = static_cast<int32_t>(hipErrorInvalidValue);
      return;
    }
    running *= sizes[i];
  }
  const uint64_t sizeBytes = static_cast<uint64_t>(running * elementSizeBytes);
  mgpuMemHostRegister(desc->aligned + desc->offset * elementSizeBytes, sizeBytes);
}

void mgpuMemHostUnregisterMemRef(int64_t /*rank*/, void *descriptor,
                                 int64_t elementSizeBytes) {
  auto *desc = static_cast<MemRefHeader *>(descriptor);
  mgpuMemHostUnregister(desc->aligned + desc->offset * elementSizeBytes);
}

void mgpuSetDefaultDevice(int32_t device) {
  defaultDevice = device;
  deviceBound = false;
}

int32_t mgpuRuntimeTakeLastError() {
  const int32_t e = lastError;
  lastError = 0;
  return e;
}

} // extern "C"
