// Table of the real HIP runtime entry points.
//
// Neither libinttemp.so nor scheduler_eval.so links against libamdhip64: a
// PyTorch-ROCm process carries its own copy of the runtime, and binding to any
// other copy would split streams and kernels between two runtimes.  The table
// is filled on first use from the runtime that is already loaded in the process
// (found by walking the loaded objects), else from `libamdhip64.so.7`; the
// environment variable ORION_HIP_LIBRARY names a different library (tests use a
// recording stand-in to run the whole path on a host without a GPU).
//
// Reference counterpart: the dlsym(RTLD_NEXT / RTLD_DEFAULT, "cuda...") lookups
// of src/cuda_capture/intercept_temp.cpp:153-156 and
// src/scheduler/utils_sched.cpp:159-237 (register_functions).
#pragma once

#ifndef __HIP_PLATFORM_AMD__
#define __HIP_PLATFORM_AMD__ 1
#endif
#include <hip/hip_runtime_api.h>
// The three extension entry points are declared here rather than through
// <hip/hip_ext.h>, whose templates need the HIP compiler.
extern "C" {
hipError_t hipExtModuleLaunchKernel(hipFunction_t f, uint32_t globalWorkSizeX,
                                    uint32_t globalWorkSizeY, uint32_t globalWorkSizeZ,
                                    uint32_t localWorkSizeX, uint32_t localWorkSizeY,
                                    uint32_t localWorkSizeZ, size_t sharedMemBytes,
                                    hipStream_t hStream, void** kernelParams, void** extra,
                                    hipEvent_t startEvent, hipEvent_t stopEvent, uint32_t flags);
hipError_t hipHccModuleLaunchKernel(hipFunction_t f, uint32_t globalWorkSizeX,
                                    uint32_t globalWorkSizeY, uint32_t globalWorkSizeZ,
                                    uint32_t localWorkSizeX, uint32_t localWorkSizeY,
                                    uint32_t localWorkSizeZ, size_t sharedMemBytes,
                                    hipStream_t hStream, void** kernelParams, void** extra,
                                    hipEvent_t startEvent, hipEvent_t stopEvent);
hipError_t hipExtLaunchKernel(const void* function_address, dim3 numBlocks, dim3 dimBlocks,
                              void** args, size_t sharedMemBytes, hipStream_t stream,
                              hipEvent_t startEvent, hipEvent_t stopEvent, int flags);
}

namespace orion {

// name, return type, parameter list
#define ORION_HIP_FUNCTIONS(X)                                                              \
  X(hipLaunchKernel, hipError_t, (const void*, dim3, dim3, void**, size_t, hipStream_t))    \
  X(hipExtLaunchKernel, hipError_t,                                                         \
    (const void*, dim3, dim3, void**, size_t, hipStream_t, hipEvent_t, hipEvent_t, int))    \
  X(hipLaunchCooperativeKernel, hipError_t,                                                 \
    (const void*, dim3, dim3, void**, unsigned int, hipStream_t))                           \
  X(hipModuleLaunchKernel, hipError_t,                                                      \
    (hipFunction_t, unsigned, unsigned, unsigned, unsigned, unsigned, unsigned, unsigned,   \
     hipStream_t, void**, void**))                                                          \
  X(hipExtModuleLaunchKernel, hipError_t,                                                   \
    (hipFunction_t, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, size_t,     \
     hipStream_t, void**, void**, hipEvent_t, hipEvent_t, uint32_t))                        \
  X(hipModuleLaunchCooperativeKernel, hipError_t,                                           \
    (hipFunction_t, unsigned, unsigned, unsigned, unsigned, unsigned, unsigned, unsigned,   \
     hipStream_t, void**))                                                                  \
  X(hipMalloc, hipError_t, (void**, size_t))                                                \
  X(hipFree, hipError_t, (void*))                                                           \
  X(hipMallocAsync, hipError_t, (void**, size_t, hipStream_t))                              \
  X(hipFreeAsync, hipError_t, (void*, hipStream_t))                                         \
  X(hipMemcpy2D, hipError_t,                                                                \
    (void*, size_t, const void*, size_t, size_t, size_t, hipMemcpyKind))                    \
  X(hipMemcpy, hipError_t, (void*, const void*, size_t, hipMemcpyKind))                     \
  X(hipMemcpyAsync, hipError_t, (void*, const void*, size_t, hipMemcpyKind, hipStream_t))   \
  X(hipMemcpyWithStream, hipError_t,                                                        \
    (void*, const void*, size_t, hipMemcpyKind, hipStream_t))                               \
  X(hipMemcpy2DAsync, hipError_t,                                                           \
    (void*, size_t, const void*, size_t, size_t, size_t, hipMemcpyKind, hipStream_t))       \
  X(hipMemset, hipError_t, (void*, int, size_t))                                            \
  X(hipMemsetAsync, hipError_t, (void*, int, size_t, hipStream_t))                          \
  X(hipMemsetD32Async, hipError_t, (hipDeviceptr_t, int, size_t, hipStream_t))              \
  X(hipMemsetD16Async, hipError_t, (hipDeviceptr_t, unsigned short, size_t, hipStream_t))   \
  X(hipMemsetD8Async, hipError_t, (hipDeviceptr_t, unsigned char, size_t, hipStream_t))     \
  X(hipGraphLaunch, hipError_t, (hipGraphExec_t, hipStream_t))                              \
  X(hipGraphCreate, hipError_t, (hipGraph_t*, unsigned int))                                \
  X(hipGraphAddKernelNode, hipError_t,                                                      \
    (hipGraphNode_t*, hipGraph_t, const hipGraphNode_t*, size_t,                            \
     const hipKernelNodeParams*))                                                           \
  X(hipGraphKernelNodeSetParams, hipError_t, (hipGraphNode_t, const hipKernelNodeParams*))  \
  X(hipGraphKernelNodeGetParams, hipError_t, (hipGraphNode_t, hipKernelNodeParams*))        \
  X(hipGraphDestroyNode, hipError_t, (hipGraphNode_t))                                      \
  X(hipLaunchHostFunc, hipError_t, (hipStream_t, hipHostFn_t, void*))                       \
  X(hipStreamWriteValue32, hipError_t, (hipStream_t, void*, uint32_t, unsigned int))        \
  X(hipStreamWriteValue64, hipError_t, (hipStream_t, void*, uint64_t, unsigned int))        \
  X(hipStreamWaitValue32, hipError_t,                                                       \
    (hipStream_t, void*, uint32_t, unsigned int, uint32_t))                                 \
  X(hipStreamWaitValue64, hipError_t,                                                       \
    (hipStream_t, void*, uint64_t, unsigned int, uint64_t))                                 \
  X(hipMemcpyToSymbol, hipError_t,                                                          \
    (const void*, const void*, size_t, size_t, hipMemcpyKind))                              \
  X(hipMemcpyToSymbolAsync, hipError_t,                                                     \
    (const void*, const void*, size_t, size_t, hipMemcpyKind, hipStream_t))                 \
  X(hipMemcpyFromSymbol, hipError_t,                                                        \
    (void*, const void*, size_t, size_t, hipMemcpyKind))                                    \
  X(hipMemcpyFromSymbolAsync, hipError_t,                                                   \
    (void*, const void*, size_t, size_t, hipMemcpyKind, hipStream_t))                       \
  X(hipStreamSynchronize, hipError_t, (hipStream_t))                                        \
  X(hipStreamQuery, hipError_t, (hipStream_t))                                              \
  X(hipStreamWaitEvent, hipError_t, (hipStream_t, hipEvent_t, unsigned int))                \
  X(hipStreamCreateWithFlags, hipError_t, (hipStream_t*, unsigned int))                     \
  X(hipExtStreamCreateWithCUMask, hipError_t, (hipStream_t*, uint32_t, const uint32_t*))    \
  X(hipStreamDestroy, hipError_t, (hipStream_t))                                            \
  X(hipEventCreateWithFlags, hipError_t, (hipEvent_t*, unsigned))                           \
  X(hipEventDestroy, hipError_t, (hipEvent_t))                                              \
  X(hipEventRecord, hipError_t, (hipEvent_t, hipStream_t))                                  \
  X(hipEventQuery, hipError_t, (hipEvent_t))                                                \
  X(hipEventSynchronize, hipError_t, (hipEvent_t))                                          \
  X(hipEventElapsedTime, hipError_t, (float*, hipEvent_t, hipEvent_t))                      \
  X(hipDeviceSynchronize, hipError_t, (void))                                               \
  X(hipModuleUnload, hipError_t, (hipModule_t))                                             \
  X(hipHostFree, hipError_t, (void*))                                                       \
  X(hipFreeHost, hipError_t, (void*))                                                       \
  X(hipDeviceGetAttribute, hipError_t, (int*, hipDeviceAttribute_t, int))                   \
  X(hipSetDevice, hipError_t, (int))                                                        \
  X(hipGetDevice, hipError_t, (int*))                                                       \
  X(hipGetLastError, hipError_t, (void))                                                    \
  X(hipPeekAtLastError, hipError_t, (void))                                                 \
  X(hipGetErrorString, const char*, (hipError_t))                                           \
  X(hipFuncGetAttributes, hipError_t, (struct hipFuncAttributes*, const void*))             \
  X(hipFuncGetAttribute, hipError_t, (int*, hipFunction_attribute, hipFunction_t))          \
  X(hipKernelNameRef, const char*, (const hipFunction_t))                                   \
  X(hipKernelNameRefByPtr, const char*, (const void*, hipStream_t))

struct HipApi {
#define X(name, ret, params) ret(*name) params;
  ORION_HIP_FUNCTIONS(X)
#undef X
  const char* library_path;  // where the table came from
  // True when the table came from the host-only stand-in runtime of the tests
  // (recognised by its control entry point), which launches nothing on a GPU.
  bool stand_in;
};

}  // namespace orion

// Exported by libinttemp.so.  Never returns null; aborts with a message when no
// HIP runtime can be found (the product has no CPU path to fall back to).
// Symbols the runtime lacks are left null and checked where they are used.
extern "C" const orion::HipApi* orion_hip_api(void);
