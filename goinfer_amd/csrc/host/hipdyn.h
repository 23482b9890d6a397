// hipdyn.h — libamdhip64 bound at run time with dlopen, the cgo-free way goinfer's backend/cuda binds its driver
// (backend/cuda/internal/gpudev/cuda.go:65-83). Only the HIP types come from the headers; no HIP symbol is linked.
#pragma once
#ifndef __HIP_PLATFORM_AMD__
#define __HIP_PLATFORM_AMD__ 1
#endif
#include <hip/hip_runtime_api.h>

struct HipApi {
    hipError_t (*Init)(unsigned int);
    hipError_t (*GetDeviceCount)(int *);
    hipError_t (*SetDevice)(int);
    hipError_t (*DeviceSynchronize)();
    hipError_t (*MemGetInfo)(size_t *, size_t *);
    hipError_t (*Malloc)(void **, size_t);
    hipError_t (*Free)(void *);
    hipError_t (*HostMalloc)(void **, size_t, unsigned int);
    hipError_t (*HostFree)(void *);
    hipError_t (*Memcpy)(void *, const void *, size_t, hipMemcpyKind);
    hipError_t (*MemcpyAsync)(void *, const void *, size_t, hipMemcpyKind, hipStream_t);
    hipError_t (*Memset)(void *, int, size_t);
    hipError_t (*MemsetAsync)(void *, int, size_t, hipStream_t);
    hipError_t (*StreamCreate)(hipStream_t *);
    hipError_t (*StreamDestroy)(hipStream_t);
    hipError_t (*StreamSynchronize)(hipStream_t);
    hipError_t (*EventCreate)(hipEvent_t *);
    hipError_t (*EventDestroy)(hipEvent_t);
    hipError_t (*EventRecord)(hipEvent_t, hipStream_t);
    hipError_t (*EventSynchronize)(hipEvent_t);
    hipError_t (*EventElapsedTime)(float *, hipEvent_t, hipEvent_t);
    hipError_t (*ModuleLoadData)(hipModule_t *, const void *);
    hipError_t (*ModuleUnload)(hipModule_t);
    hipError_t (*ModuleGetFunction)(hipFunction_t *, hipModule_t, const char *);
    hipError_t (*ModuleLaunchKernel)(hipFunction_t, unsigned, unsigned, unsigned, unsigned, unsigned, unsigned, unsigned, hipStream_t,
                                     void **, void **);
    hipError_t (*StreamBeginCapture)(hipStream_t, hipStreamCaptureMode);
    hipError_t (*StreamEndCapture)(hipStream_t, hipGraph_t *);
    hipError_t (*GraphInstantiate)(hipGraphExec_t *, hipGraph_t, hipGraphNode_t *, char *, size_t);
    hipError_t (*GraphLaunch)(hipGraphExec_t, hipStream_t);
    hipError_t (*GraphDestroy)(hipGraph_t);
    hipError_t (*GraphExecDestroy)(hipGraphExec_t);
    const char *(*GetErrorString)(hipError_t);
    hipError_t (*GetLastError)();
};

// Loads libamdhip64 (ROCMDECODE_HIP_LIB, then the usual sonames) once; returns nullptr and sets *why on failure.
const HipApi *hip_api(const char **why);
