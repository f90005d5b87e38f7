// Shared definitions of the bf16 flash-attention prefill kernels (dense and paged): one wave folds keys
// into the running softmax state of its 32 query rows.  Everything is kept transposed so the softmax
// weights never leave registers:
//
//   S^T[key, query] = K . Q^T      v_mfma_f32_32x32x16_bf16, A = K rows read from LDS (16-byte reads), B = the
//                                  wave's Q^T, resident in 32 VGPRs (head_dim 128) for the whole kernel;
//   online softmax                 base two; a lane holds the scores of ONE query (its MFMA column), so
//                                  the row maximum is in-lane max ops plus one v_permlane32_swap, and
//                                  rescaling O^T needs no broadcast;
//   O^T[dim, query] += V^T . P^T   A = V^T read from LDS with ds_read_b64_tr_b16 (the hardware transposes
//                                  four keys x four dims per 16 lanes: lane 16G + s of a 16-lane group points
//                                  at key (s >> 2), dims 4 (s & 3) .. +4 of the group's 16 dims, and lane i
//                                  receives the four keys of dim i), B = P^T packed to bf16 straight from
//                                  the S^T accumulator registers, whose (lane, register) -> key map is what
//                                  fixes the V^T read pattern.
//
// Probabilities are rounded to bf16 for the second product and summed unrounded, like the reference's
// tensor-core kernel (singe/src/backend/cuda/kernel_plan/source/tensor_core.rs:112-194).  The loop that
// uses these is in prefill_blocks.hip.h.
#pragma once

#include "common.hip.h"

namespace prefill {

// The head dimension a build of these kernels is for: the sources are compiled once per value (128, and the other
// multiples of 16 with -DSINGE_HEAD_DIM=...), each into its own part of the code object.
#ifndef SINGE_HEAD_DIM
#define SINGE_HEAD_DIM 128
#endif
constexpr int kHeadDim = SINGE_HEAD_DIM;
static_assert(kHeadDim % 16 == 0 && kHeadDim >= 16 && kHeadDim <= 128, "head dimensions the matrix-core kernels are built for");
constexpr int kSteps = kHeadDim / 16;      // products per 32-key block of scores: sixteen dims each
constexpr int kDimBlocks = (kHeadDim + 31) / 32;  // 32-dim blocks of O^T; at an odd multiple of 16 the last one is half
                                                 // real: its other sixteen dims multiply whatever the LDS rows hold past
                                                 // a key's last chunk, stay in registers of their own and are never stored
constexpr int kQueryTile = 128;       // query rows per workgroup
constexpr int kKeyTile = 64;          // keys per LDS stage

typedef short v4i16_t __attribute__((ext_vector_type(4)));
typedef short v8i16_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2v_t __attribute__((ext_vector_type(2)));
typedef float f32x2v_t __attribute__((ext_vector_type(2)));

// max(a, b) in one instruction, without the canonicalising copies the compiler puts in front of fmaxf when
// it cannot see where the operands come from (here: out of inline assembly); for values that are never
// signalling NaNs.
SINGE_DEVICE float max2(float a, float b) {
    float result;
    asm("v_max_f32 %0, %1, %2" : "=v"(result) : "v"(a), "v"(b));
    return result;
}

SINGE_DEVICE float swap32_max(float value) {
    float kept = value, taken = value;
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(kept), "+v"(taken));
    return max2(kept, taken);
}

SINGE_DEVICE float swap32_sum(float value) {
    float kept = value, taken = value;
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(kept), "+v"(taken));
    return kept + taken;
}

// max(a, b, c) in one instruction.  The scores come straight out of the matrix core and are never
// signalling NaNs, so the canonicalising copies the compiler puts in front of fmaxf are not needed.
SINGE_DEVICE float max3(float a, float b, float c) {
    float result;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(result) : "v"(a), "v"(b), "v"(c));
    return result;
}

// The 16-bit storage type of Q, K, V, P and the output: a tag the functions below are overloaded on.  The
// operands travel as bit patterns (uint4 = eight halves); only the product and the rounding differ.
struct Bf16 {};
struct F16 {};

typedef _Float16 f16x2v_t __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8v_t __attribute__((ext_vector_type(8)));

// Two f32 values rounded to nearest even and packed, low half first.
SINGE_DEVICE unsigned int pack_pair(Bf16, float lo, float hi) {
    f32x2v_t both = {lo, hi};
    return __builtin_bit_cast(unsigned int, __builtin_convertvector(both, bf16x2v_t));
}
SINGE_DEVICE unsigned int pack_pair(F16, float lo, float hi) {
    f32x2v_t both = {lo, hi};
    return __builtin_bit_cast(unsigned int, __builtin_convertvector(both, f16x2v_t));
}
SINGE_DEVICE unsigned int pack_pair(float lo, float hi) { return pack_pair(Bf16{}, lo, hi); }

// D = A . B + C on the matrix core: 32 x 32 outputs, sixteen values of the contracted index per lane pair.
SINGE_DEVICE f32x16_t mma(Bf16, uint4 a, uint4 b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
}
SINGE_DEVICE f32x16_t mma(F16, uint4 a, uint4 b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8v_t, a), __builtin_bit_cast(f16x8v_t, b), c, 0, 0, 0);
}

// How far (log2 units) a row's maximum may run ahead of the reference point its weights are scaled
// by before the accumulators are rescaled.  Any reference point gives the same quotient; letting it lag
// by up to 2^6 keeps weights far inside bf16/f32 range and makes the rescale of O^T rare after the
// first tiles.
constexpr float kMaxLag = 6.0f;

// Running state of a wave's 32 query rows: lane (query = lane % 32, hi = lane / 32) holds dims
// 32db + 8(r / 4) + 4hi + (r % 4) of its query in out[db][r].
struct RowState {
    f32x16_t out[kDimBlocks];
    float reference;    // point the weights are scaled by (scaled log2 units); trails the row maximum
    float running_sum;  // of this lane's keys only
};

SINGE_DEVICE void reset(RowState& state) {
#pragma unroll
    for (int db = 0; db < kDimBlocks; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) state.out[db][r] = 0.0f;
    state.reference = -INFINITY;
    state.running_sum = 0.0f;
}

}  // namespace prefill
