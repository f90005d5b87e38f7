// The handful of HIP runtime entry points the launcher needs, resolved with dlopen on first use
// (the pattern of the reference's sys crates: singe-loader/src/lib.rs:298-322).  Declaring them here
// keeps the library free of a link-time dependency on ROCm, and lets it share the runtime instance
// the host process already loaded (for example the one PyTorch ships) instead of loading a second one.
#pragma once

#include <stddef.h>
#include <stdint.h>

namespace singe_hip {

using hipError_t = int;
using hipModule_t = void*;
using hipFunction_t = void*;
using hipStream_t = void*;

constexpr hipError_t hipSuccess = 0;

struct HipRuntime {
    hipError_t (*hipGetDevice)(int*);
    hipError_t (*hipDeviceGetAttribute)(int*, int, int);
    hipError_t (*hipModuleLoadData)(hipModule_t*, const void*);
    hipError_t (*hipModuleUnload)(hipModule_t);
    hipError_t (*hipModuleGetFunction)(hipFunction_t*, hipModule_t, const char*);
    hipError_t (*hipModuleLaunchKernel)(hipFunction_t, unsigned, unsigned, unsigned, unsigned, unsigned, unsigned,
                                        unsigned, hipStream_t, void**, void**);
    const char* (*hipGetErrorString)(hipError_t);
    // Timing and capture queries, for the one entry point that tunes itself.
    hipError_t (*hipEventCreate)(void**);
    hipError_t (*hipEventDestroy)(void*);
    hipError_t (*hipEventRecord)(void*, hipStream_t);
    hipError_t (*hipEventSynchronize)(void*);
    hipError_t (*hipEventElapsedTime)(float*, void*, void*);
    hipError_t (*hipStreamIsCapturing)(hipStream_t, int*);
};

// Returns the resolved table, or nullptr when no HIP runtime can be opened.
const HipRuntime* hip_runtime();

}  // namespace singe_hip
