// The scratch of the entry points that allocate nothing: one fixed array in device memory per GPU,
// part of this library's device image, for callers that cannot allocate (code under HIP graph
// capture, tight serving loops, harnesses that forbid hipMalloc).
//
// The array's name is a host-side stand-in, not a device address, so the host resolves its address
// once per device with hipGetSymbolAddress (with that device current) and only ever hands that
// address to kernels.  Each GPU holds its own copy at its own address until the process ends.  Every
// call on a GPU shares that GPU's array and the array keeps the last call's contents: calls that
// overlap on one GPU race.
#include <hip/hip_runtime.h>

#include <atomic>

#include "static_scratch.h"

static __device__ __align__(256) unsigned char scratch[SINGE_HIP_STATIC_SCRATCH_BYTES];
static_assert(sizeof(scratch) == SINGE_HIP_STATIC_SCRATCH_BYTES, "the size callers are refused by is the array's");

namespace {

// Touches the array from device code so the device image always carries it.
__global__ void singe_static_scratch_probe(unsigned int* seen) {
    if (seen != nullptr) *seen = scratch[0];
}

constexpr int kMaxDevices = 64;
std::atomic<void*> g_address[kMaxDevices] = {};

}  // namespace

namespace singe_hip {

int static_scratch(void** pointer, size_t* bytes) {
    int device = 0;
    if (hipError_t error = hipGetDevice(&device)) return -static_cast<int>(error);
    if (device < 0 || device >= kMaxDevices) return -static_cast<int>(hipErrorInvalidDevice);
    void* address = g_address[device].load(std::memory_order_acquire);
    if (address == nullptr) {
        // Two threads that get here together resolve the same address.
        if (hipError_t error = hipGetSymbolAddress(&address, HIP_SYMBOL(scratch))) return -static_cast<int>(error);
        if (address == nullptr) return -static_cast<int>(hipErrorInvalidSymbol);
        g_address[device].store(address, std::memory_order_release);
    }
    *pointer = address;
    *bytes = SINGE_HIP_STATIC_SCRATCH_BYTES;
    return 0;
}

}  // namespace singe_hip
