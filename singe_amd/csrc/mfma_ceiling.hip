// What the matrix cores sustain on given operands with nothing else in the way: a register-only loop of the
// prefill kernels' product, v_mfma_f32_32x32x16_bf16 (or _f16), no LDS, no softmax, no memory traffic inside the
// loop.  The clock under such a loop is set by power, and power by how many operand bits toggle, so the rate on
// N(0, 1) data is well below the rate on zeros; the prefill kernels are priced against both the published peak
// and this measured ceiling.  A measurement aid: the reference has no counterpart.
//
// Each lane loads sixteen 16-byte operands (eight A, eight B) from `operands` (4096 bytes per wave, taken modulo
// the buffer) and then issues `iterations` rounds of 32 products into four independent accumulators, the same
// dependency distance the prefill kernels' score and value products have.  Flop per workgroup of four waves:
// 4 * iterations * 32 * 32768.
#include "common.hip.h"
#include "kernel_args.h"

namespace {

typedef _Float16 f16x8_ceiling_t __attribute__((ext_vector_type(8)));

template <bool F16>
SINGE_DEVICE void mfma_ceiling_body(const MfmaCeilingArgs& a) {
    const unsigned int lane = threadIdx.x & 63;
    const unsigned long long wave = static_cast<unsigned long long>(blockIdx.x) * (blockDim.x >> 6) + (threadIdx.x >> 6);
    uint4 left[8], right[8];
#pragma unroll
    for (int s = 0; s < 16; ++s) {
        const unsigned long long chunk = (wave * 16 + s) * 64 + lane;  // 16-byte chunks
        const uint4 bits = static_cast<const uint4*>(a.operands)[chunk % a.operand_chunks];
        if (s < 8) left[s] = bits; else right[s - 8] = bits;
    }
    f32x16_t acc[4];
#pragma unroll
    for (int c = 0; c < 4; ++c)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[c][r] = 0.0f;
    for (unsigned int round = 0; round < a.iterations; ++round) {
#pragma unroll
        for (int n = 0; n < 32; ++n) {
            if constexpr (F16)
                acc[n & 3] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_ceiling_t, left[n & 7]),
                                                                    __builtin_bit_cast(f16x8_ceiling_t, right[(n >> 2) & 7]), acc[n & 3], 0, 0, 0);
            else
                acc[n & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, left[n & 7]),
                                                                     __builtin_bit_cast(bf16x8_t, right[(n >> 2) & 7]), acc[n & 3], 0, 0, 0);
        }
    }
    float sum = 0.0f;
#pragma unroll
    for (int c = 0; c < 4; ++c)
#pragma unroll
        for (int r = 0; r < 16; ++r) sum += acc[c][r];
    a.out[wave * 64 + lane] = sum;
}

}  // namespace

extern "C" __global__ __launch_bounds__(256, 2) void singe_mfma_ceiling_bf16(MfmaCeilingArgs a) { mfma_ceiling_body<false>(a); }
extern "C" __global__ __launch_bounds__(256, 2) void singe_mfma_ceiling_f16(MfmaCeilingArgs a) { mfma_ceiling_body<true>(a); }
