// Code object of the kernels that the reference's compiler would have
// generated and combined into the device module `ops`
// (lib/Dialect/Device/Transform/CombineGPUKernel.cpp:28-47), loaded at run time
// with mgpuModuleFileLoad and launched by name through mgpuLaunchKernel
// (lib/Dialect/Device/IR/GPUOffloadingAttr.cpp:283-304).  Kernels take bare
// pointers (lib/Pipelines/MLIRToGPU.cpp:162-165,181-182).
//
// main_graph_kernel is the elementwise add of examples/add.onnx, hand written
// for gfx950: the reference emits 1200 blocks x 1024 threads with one scalar
// element per thread; here every lane moves 128-bit vectors in a grid-stride
// loop and the host picks the grid.
#include <hip/hip_runtime.h>

#include <cstdint>

typedef float float4v __attribute__((ext_vector_type(4)));

extern "C" __global__ __launch_bounds__(256) void main_graph_kernel(const float *__restrict__ a,
                                                                    const float *__restrict__ b,
                                                                    float *__restrict__ c,
                                                                    int64_t n) {
  const int64_t n4 = n / 4;
  const float4v *a4 = reinterpret_cast<const float4v *>(a);
  const float4v *b4 = reinterpret_cast<const float4v *>(b);
  float4v *c4 = reinterpret_cast<float4v *>(c);
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  const int64_t tid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  for (int64_t i = tid; i < n4; i += stride)
    __builtin_nontemporal_store(a4[i] + b4[i], c4 + i);
  for (int64_t i = n4 * 4 + tid; i < n; i += stride) c[i] = a[i] + b[i];
}
