/*
 * mgpu_runtime.h - C ABI of the device runtime (streams, events, buffers,
 * code-object loading and kernel launch) for one MI355X.
 *
 * Drop-in for the `mgpu*` wrappers the reference exports from
 * lib/Runtime/CUDA/CudaRuntimeWrappers.cpp (declared in
 * include/multi-device-model-compiler/Runtime/CUDA/CudaRuntimeWrappers.h:25-54)
 * and that compiled model libraries call by symbol name
 * (lib/Conversion/ConvertDeviceToLLVM/ConvertDeviceToLLVM.cpp:337-396,
 * lib/Dialect/Device/IR/GPUOffloadingAttr.cpp:162-193,283-304).
 * Implemented directly on the HIP runtime/module API in libmgpu_hip_runtime.so.
 *
 * Conventions kept from the reference: every entry point returns void or a
 * handle; a failing HIP call prints `'<expr>' failed with '<name>'` to stderr
 * and execution continues (CudaRuntimeWrappers.cpp:3-12).  Handles are opaque
 * pointers (hipStream_t / hipEvent_t / hipFunction_t underneath).
 */
#ifndef MGPU_RUNTIME_H_
#define MGPU_RUNTIME_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void *mgpuStream_t;   /* hipStream_t   (reference: CUstream)   */
typedef void *mgpuEvent_t;    /* hipEvent_t    (reference: CUevent)    */
typedef void *mgpuFunction_t; /* hipFunction_t (reference: CUfunction) */

/* One process-global code object, like the reference's `static CUmodule module`
 * (CudaRuntimeWrappers.cpp:89-107).  `fname` is a gfx950 .hsaco file. */
void mgpuModuleFileLoad(const char *fname);         /* CudaRuntimeWrappers.cpp:91-95  */
void mgpuModuleUnload(void);                        /* :97-100 */
mgpuFunction_t mgpuModuleGetFunction(const char *name); /* :102-107 */

/* Grid/block extents are intptr_t to match MLIR's index type (:109-139).
 * `params` is an array of pointers to the individual kernel arguments. */
void mgpuLaunchKernel(mgpuFunction_t function, intptr_t gridX, intptr_t gridY, intptr_t gridZ,
                      intptr_t blockX, intptr_t blockY, intptr_t blockZ, int32_t smem,
                      mgpuStream_t stream, void **params, void **extra);

mgpuStream_t mgpuStreamCreate(void);                /* :141-146 non-blocking stream */
void mgpuStreamDestroy(mgpuStream_t stream);        /* :148-150 */
void mgpuStreamSynchronize(mgpuStream_t stream);    /* :152-155 */
void mgpuStreamWaitEvent(mgpuStream_t stream, mgpuEvent_t event); /* :157-160 */

mgpuEvent_t mgpuEventCreate(void);                  /* :162-167 timing disabled */
mgpuEvent_t mgpuEventCreateWithStream(mgpuStream_t stream); /* :169-175 */
mgpuEvent_t mgpuEventEnableTimeCreate(void);        /* :177-182 timing enabled */
void mgpuEventDestroy(mgpuEvent_t event);           /* :184-186 */
void mgpuEventSynchronize(mgpuEvent_t event);       /* :188-190 */
void mgpuEventRecord(mgpuEvent_t event, mgpuStream_t stream); /* :192-195 */
float mgpuEventElapsedTime(mgpuEvent_t begin, mgpuEvent_t end); /* :197-202, milliseconds */

void *mgpuMemAlloc(uint64_t sizeBytes, mgpuStream_t stream);      /* :204-209 */
void mgpuMemFree(void *ptr, mgpuStream_t stream);                 /* :211-213 */
void *mgpuMemAllocAsync(uint64_t sizeBytes, mgpuStream_t stream); /* :215-219 stream ordered */
void mgpuMemFreeAsync(void *ptr, mgpuStream_t stream);            /* :221-224 */
/* Asynchronous copy on `stream`; direction is inferred from the pointers (:226-231). */
void mgpuMemcpy(void *dst, void *src, size_t sizeBytes, mgpuStream_t stream);
void mgpuMemset32(void *dst, unsigned int value, size_t count, mgpuStream_t stream);   /* :233-237 */
void mgpuMemset16(void *dst, unsigned short value, size_t count, mgpuStream_t stream); /* :239-243 */

/* Page-lock an existing host range (:251-255, :282-285). */
void mgpuMemHostRegister(void *ptr, uint64_t sizeBytes);
void mgpuMemHostUnregister(void *ptr);
/* `descriptor` is a ranked MLIR memref descriptor {allocated, aligned, offset,
 * sizes[rank], strides[rank]} (:260-279, :289-295). */
void mgpuMemHostRegisterMemRef(int64_t rank, void *descriptor, int64_t elementSizeBytes);
void mgpuMemHostUnregisterMemRef(int64_t rank, void *descriptor, int64_t elementSizeBytes);

void mgpuSetDefaultDevice(int32_t device);          /* :297-299 thread-local ordinal */

/* Not in the reference: the code of the most recent failing HIP call made by
 * this library on the calling thread (0 = none), cleared by the query.  Lets a
 * host test assert on the print-and-continue convention. */
int32_t mgpuRuntimeTakeLastError(void);

#ifdef __cplusplus
}
#endif
#endif /* MGPU_RUNTIME_H_ */
