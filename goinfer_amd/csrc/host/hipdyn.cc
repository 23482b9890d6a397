// hipdyn.cc — resolves the HIP runtime entry points from libamdhip64 with dlopen/dlsym.
#include "hipdyn.h"
#include <dlfcn.h>
#include <mutex>
#include <stdio.h>
#include <stdlib.h>

static HipApi g_api;
static bool g_ok = false;
static char g_why[256];

template <typename F> static bool sym(void *h, const char *name, F &out) {
    void *p = dlsym(h, name);
    if (!p) {
        snprintf(g_why, sizeof g_why, "libamdhip64: missing symbol %s", name);
        return false;
    }
    out = reinterpret_cast<F>(p);
    return true;
}

static void load_once() {
    const char *names[] = {getenv("ROCMDECODE_HIP_LIB"), "libamdhip64.so.7", "libamdhip64.so", "/opt/rocm/lib/libamdhip64.so"};
    void *h = nullptr;
    for (const char *n : names) {
        if (!n || !*n) continue;
        h = dlopen(n, RTLD_NOW | RTLD_GLOBAL);
        if (h) break;
    }
    if (!h) {
        snprintf(g_why, sizeof g_why, "cannot load libamdhip64: %s", dlerror());
        return;
    }
    HipApi &a = g_api;
    g_ok = sym(h, "hipInit", a.Init) && sym(h, "hipGetDeviceCount", a.GetDeviceCount) && sym(h, "hipSetDevice", a.SetDevice) &&
           sym(h, "hipDeviceSynchronize", a.DeviceSynchronize) && sym(h, "hipMemGetInfo", a.MemGetInfo) && sym(h, "hipMalloc", a.Malloc) &&
           sym(h, "hipFree", a.Free) && sym(h, "hipHostMalloc", a.HostMalloc) && sym(h, "hipHostFree", a.HostFree) &&
           sym(h, "hipMemcpy", a.Memcpy) && sym(h, "hipMemcpyAsync", a.MemcpyAsync) && sym(h, "hipMemset", a.Memset) &&
           sym(h, "hipMemsetAsync", a.MemsetAsync) && sym(h, "hipStreamCreate", a.StreamCreate) &&
           sym(h, "hipStreamDestroy", a.StreamDestroy) && sym(h, "hipStreamSynchronize", a.StreamSynchronize) &&
           sym(h, "hipEventCreate", a.EventCreate) && sym(h, "hipEventDestroy", a.EventDestroy) && sym(h, "hipEventRecord", a.EventRecord) &&
           sym(h, "hipEventSynchronize", a.EventSynchronize) && sym(h, "hipEventElapsedTime", a.EventElapsedTime) &&
           sym(h, "hipModuleLoadData", a.ModuleLoadData) && sym(h, "hipModuleUnload", a.ModuleUnload) &&
           sym(h, "hipModuleGetFunction", a.ModuleGetFunction) && sym(h, "hipModuleLaunchKernel", a.ModuleLaunchKernel) &&
           sym(h, "hipStreamBeginCapture", a.StreamBeginCapture) && sym(h, "hipStreamEndCapture", a.StreamEndCapture) &&
           sym(h, "hipGraphInstantiate", a.GraphInstantiate) && sym(h, "hipGraphLaunch", a.GraphLaunch) &&
           sym(h, "hipGraphDestroy", a.GraphDestroy) && sym(h, "hipGraphExecDestroy", a.GraphExecDestroy) &&
           sym(h, "hipGetErrorString", a.GetErrorString) && sym(h, "hipGetLastError", a.GetLastError);
}

const HipApi *hip_api(const char **why) {
    static std::once_flag once;
    std::call_once(once, load_once);
    if (!g_ok) {
        if (why) *why = g_why;
        return nullptr;
    }
    return &g_api;
}
