#include "hip_runtime_loader.h"

#include <dlfcn.h>

#include <mutex>

// The runtime this library is linked against (for the hipcc-built unit that holds the fixed device scratch).
extern "C" int hipGetDevice(int* device);

namespace singe_hip {

namespace {

HipRuntime g_runtime;
bool g_ready = false;
std::once_flag g_once;

void* open_runtime() {
    // A runtime the process already holds wins, so streams and pointers created through it are ours too.
    const char* names[] = {"libamdhip64.so.7", "libamdhip64.so", "libamdhip64.so.6"};
    for (const char* name : names)
        if (void* handle = dlopen(name, RTLD_NOW | RTLD_NOLOAD | RTLD_GLOBAL)) return handle;
    for (const char* name : names)
        if (void* handle = dlopen(name, RTLD_NOW | RTLD_GLOBAL)) return handle;
    const char* fallbacks[] = {"/opt/rocm/lib/libamdhip64.so.7", "/opt/rocm/lib/libamdhip64.so"};
    for (const char* name : fallbacks)
        if (void* handle = dlopen(name, RTLD_NOW | RTLD_GLOBAL)) return handle;
    return nullptr;
}

template <class F>
bool resolve(void* handle, const char* name, F& slot) {
    slot = reinterpret_cast<F>(dlsym(handle, name));
    return slot != nullptr;
}

void load() {
    void* handle = open_runtime();
    if (handle == nullptr) return;
    bool ok = true;
    ok &= resolve(handle, "hipGetDevice", g_runtime.hipGetDevice);
    ok &= resolve(handle, "hipDeviceGetAttribute", g_runtime.hipDeviceGetAttribute);
    ok &= resolve(handle, "hipModuleLoadData", g_runtime.hipModuleLoadData);
    ok &= resolve(handle, "hipModuleUnload", g_runtime.hipModuleUnload);
    ok &= resolve(handle, "hipModuleGetFunction", g_runtime.hipModuleGetFunction);
    ok &= resolve(handle, "hipModuleLaunchKernel", g_runtime.hipModuleLaunchKernel);
    ok &= resolve(handle, "hipGetErrorString", g_runtime.hipGetErrorString);
    ok &= resolve(handle, "hipEventCreate", g_runtime.hipEventCreate);
    ok &= resolve(handle, "hipEventDestroy", g_runtime.hipEventDestroy);
    ok &= resolve(handle, "hipEventRecord", g_runtime.hipEventRecord);
    ok &= resolve(handle, "hipEventSynchronize", g_runtime.hipEventSynchronize);
    ok &= resolve(handle, "hipEventElapsedTime", g_runtime.hipEventElapsedTime);
    ok &= resolve(handle, "hipStreamIsCapturing", g_runtime.hipStreamIsCapturing);
    // Kernel launches go through the table above, the fixed scratch's address comes from the linked runtime: both must
    // be the one copy, or the address would belong to another runtime's context.
    ok &= reinterpret_cast<void*>(g_runtime.hipGetDevice) == reinterpret_cast<void*>(&::hipGetDevice);
    g_ready = ok;
}

}  // namespace

const HipRuntime* hip_runtime() {
    std::call_once(g_once, load);
    return g_ready ? &g_runtime : nullptr;
}

}  // namespace singe_hip
