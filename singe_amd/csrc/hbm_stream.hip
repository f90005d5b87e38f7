// What the memory system delivers to a kernel that does nothing but read: every workgroup streams its share of a
// buffer with 16-byte non-temporal loads (the loads the decode kernels use for their value rows), several in flight per
// lane, and folds them into one word per lane so the reads cannot be dropped.  The decode kernels are priced against
// the published HBM peak and against this measured ceiling.  A measurement aid: the reference has no counterpart.
#include "common.hip.h"
#include "kernel_args.h"

extern "C" __global__ __launch_bounds__(512) void singe_hbm_stream_read(HbmStreamArgs a) {
    const unsigned long long lanes = static_cast<unsigned long long>(gridDim.x) * blockDim.x;
    const unsigned long long lane = static_cast<unsigned long long>(blockIdx.x) * blockDim.x + threadIdx.x;
    const uint4* chunks = static_cast<const uint4*>(a.data);
    unsigned int folded = 0;
    // A workgroup reads contiguous runs of 8 KiB (512 lanes x 16 bytes), eight runs in flight.
    unsigned long long at = lane;
    for (; at + 7 * lanes < a.chunks; at += 8 * lanes) {
        uint4 held[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) held[i] = stream_load_16(chunks + at + i * lanes);
#pragma unroll
        for (int i = 0; i < 8; ++i) folded ^= held[i].x ^ held[i].y ^ held[i].z ^ held[i].w;
    }
    for (; at < a.chunks; at += lanes) {
        const uint4 held = stream_load_16(chunks + at);
        folded ^= held.x ^ held.y ^ held.z ^ held.w;
    }
    a.out[lane] = folded;
}
