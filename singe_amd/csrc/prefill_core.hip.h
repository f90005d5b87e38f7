// Shared core of the bf16 flash-attention prefill kernels (dense and paged): one wave folds a staged
// tile of 64 keys into the running softmax state of its 32 query rows.  Everything is kept transposed
// so the softmax weights never leave registers:
//
//   S^T[key, query] = K . Q^T      v_mfma_f32_32x32x16_bf16, A = K rows read from LDS (16-byte reads,
//                                  rows padded to 272 B so 16 lanes hit 64 distinct banks), B = the
//                                  wave's Q^T, resident in 32 VGPRs for the whole kernel;
//   online softmax                 base two; a lane holds the scores of ONE query (its MFMA column), so
//                                  the row maximum is in-lane max ops plus one v_permlane32_swap, and
//                                  rescaling O^T needs no broadcast;
//   O^T[dim, query] += V^T . P^T   A = V^T read from LDS with ds_read_b64_tr_b16 (the hardware transposes
//                                  four keys x four dims per 16 lanes; rows padded to 320 B), B = P^T
//                                  packed to bf16 straight from the S^T accumulator registers, whose
//                                  (lane, register) -> key map is what fixes the V^T read pattern.
//
// Probabilities are rounded to bf16 for the second product and summed unrounded, like the reference's
// tensor-core kernel (singe/src/backend/cuda/kernel_plan/source/tensor_core.rs:112-194).
#pragma once

#include "common.hip.h"

namespace prefill {

constexpr int kHeadDim = 128;
constexpr int kQueryTile = 128;       // query rows per workgroup
constexpr int kKeyTile = 64;          // keys per LDS stage
constexpr int kKeyRowBytes = 272;     // 256 B of K + 16 B pad
constexpr int kValueRowBytes = 320;   // 256 B of V + 64 B pad
constexpr int kKeyStageBytes = kKeyTile * kKeyRowBytes;
constexpr int kValueStageBytes = kKeyTile * kValueRowBytes;
constexpr int kStageBytes = kKeyStageBytes + kValueStageBytes;

typedef short v4i16_t __attribute__((ext_vector_type(4)));
typedef short v8i16_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2v_t __attribute__((ext_vector_type(2)));
typedef float f32x2v_t __attribute__((ext_vector_type(2)));

SINGE_DEVICE float swap32_max(float value) {
    float kept = value, taken = value;
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(kept), "+v"(taken));
    return fmaxf(kept, taken);
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

SINGE_DEVICE unsigned int pack_pair(float lo, float hi) {
    f32x2v_t both = {lo, hi};
    return __builtin_bit_cast(unsigned int, __builtin_convertvector(both, bf16x2v_t));
}

// How far (log2 units) a row's maximum may run ahead of the reference point its weights are scaled
// by before the accumulators are rescaled.  Any reference point gives the same quotient; letting it lag
// by up to 2^6 keeps weights far inside bf16/f32 range and makes the rescale of O^T rare after the
// first tiles.
constexpr float kMaxLag = 6.0f;

// Running state of a wave's 32 query rows: lane (query = lane % 32, hi = lane / 32) holds dims
// 32db + 8(r / 4) + 4hi + (r % 4) of its query in out[db][r].
struct RowState {
    f32x16_t out[4];
    float reference;    // point the weights are scaled by (scaled log2 units); trails the row maximum
    float running_sum;  // of this lane's keys only
};

SINGE_DEVICE void reset(RowState& state) {
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) state.out[db][r] = 0.0f;
    state.reference = -INFINITY;
    state.running_sum = 0.0f;
}

// Per-lane LDS read offsets.  K: row = key (lane % 32), 16 B at dims 16s + 8hi.  V^T through the
// transposing read: lane 16G + s of a 16-lane group points at key (s >> 2), dims 4 (s & 3) .. +4 of
// the group's 16 dims; the hardware hands lane i the four keys of dim i.
SINGE_DEVICE unsigned int key_read_offset(unsigned int lane) { return (lane & 31u) * kKeyRowBytes + 16 * (lane >> 5); }
SINGE_DEVICE unsigned int value_read_offset(unsigned int lane) {
    const unsigned int group = lane >> 4, sub = lane & 15u, hi = lane >> 5;
    return (4 * hi + (sub >> 2)) * kValueRowBytes + (16 * (group & 1u) + 4 * (sub & 3u)) * 2;
}

// Scores of a wave's 32 queries against the 64 keys staged at `keys`: S^T blocks s0 (keys 0..31) and s1
// (keys 32..63; left at zero when live1 is false).  All eight K operands of a block are read before its
// MFMA chain starts and the two blocks' chains alternate, so no MFMA waits on an LDS round trip or on the
// MFMA issued just before it.  The products run on while the caller does other work.
struct Scores {
    f32x16_t s0, s1;
};

SINGE_DEVICE void score_staged_keys(Scores& scores, const bf16x8_t (&q)[8], const unsigned char* keys, unsigned int key_read,
                                    bool live1) {
    f32x16_t s0, s1;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        s0[r] = 0.0f;
        s1[r] = 0.0f;
    }
    uint4 ka[8], kb[8];
#pragma unroll
    for (int step = 0; step < 8; ++step) ka[step] = *reinterpret_cast<const uint4*>(keys + key_read + step * 32);
    if (live1) {
#pragma unroll
        for (int step = 0; step < 8; ++step) kb[step] = *reinterpret_cast<const uint4*>(keys + 32 * kKeyRowBytes + key_read + step * 32);
#pragma unroll
        for (int step = 0; step < 8; ++step) {
            s0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, ka[step]), q[step], s0, 0, 0, 0);
            s1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, kb[step]), q[step], s1, 0, 0, 0);
        }
    } else {
#pragma unroll
        for (int step = 0; step < 8; ++step)
            s0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, ka[step]), q[step], s0, 0, 0, 0);
    }
    scores.s0 = s0;
    scores.s1 = s1;
}

// Folds the scores of a staged tile, whose values sit at `values`, into `state`.
//   factor     scale * log2(e) (positive; a negative scale is moved into Q by the caller)
//   live1      false when the second 32-key block is wholly hidden from this wave
//   edge       true when some score of this tile must be hidden; then hidden(block, key_in_block)
//              says which (key_in_block = 8(r / 4) + 4hi + (r % 4) for accumulator register r)
//   SOFTCAP    scores become cap * tanh(score * scale / cap) before the softmax
//              (singe/src/backend/cuda/kernel_plan/source/tensor_core.rs:49-54)
template <bool SOFTCAP, class Hidden>
SINGE_DEVICE void fold_scores(RowState& state, Scores& scores, const unsigned char* values, unsigned int value_read,
                              unsigned int hi, float factor, bool live1, bool edge, Hidden&& hidden, float cap_scale = 0.0f,
                              float cap_log2e = 0.0f) {
    f32x16_t& s0 = scores.s0;
    f32x16_t& s1 = scores.s1;
    if constexpr (SOFTCAP) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            s0[r] = tanhf(s0[r] * cap_scale) * cap_log2e;
            s1[r] = tanhf(s1[r] * cap_scale) * cap_log2e;
        }
    }
    // Hide what the query may not see.  Only tiles on an edge pay for this.
    if (edge) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const unsigned int key = 8 * (r >> 2) + 4 * hi + (r & 3);
            if (hidden(0, key)) s0[r] = -INFINITY;
            if (!live1 || hidden(1, key)) s1[r] = -INFINITY;
        }
    }

    float largest = max3(s0[0], s1[0], s0[1]), other = max3(s1[1], s0[2], s1[2]);
#pragma unroll
    for (int r = 3; r < 15; r += 2) {
        largest = max3(largest, s0[r], s1[r]);
        other = max3(other, s0[r + 1], s1[r + 1]);
    }
    largest = max3(largest, s0[15], s1[15]);
    largest = swap32_max(fmaxf(largest, other)) * factor;  // both lanes of a query agree from here on
    if (__any(largest > state.reference + kMaxLag || (state.reference == -INFINITY && largest != -INFINITY))) {
        const float moved = fmaxf(state.reference, largest);
        const float base = moved == -INFINITY ? 0.0f : moved;
        const float rescale = fast_exp2(state.reference - base);
        state.running_sum *= rescale;
#pragma unroll
        for (int db = 0; db < 4; ++db)
#pragma unroll
            for (int r = 0; r < 16; ++r) state.out[db][r] *= rescale;
        state.reference = moved;
    }
    const float shift = state.reference == -INFINITY ? 0.0f : -state.reference;
    float total = 0.0f;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        s0[r] = fast_exp2(fmaf(s0[r], factor, shift));
        s1[r] = fast_exp2(fmaf(s1[r], factor, shift));
        total += s0[r] + s1[r];
    }
    state.running_sum += total;

    // O^T += V^T . P^T, 16 keys per MFMA: registers 8j .. 8j+7 of a block are keys
    // 16j + {0..3, 8..11} + 4hi of it, which is what the two transposing reads fetch.  The V^T operands
    // of the next 16 keys are read while the matrix core works on the current ones.
    typedef v4i16_t __attribute__((address_space(3))) * lds_v4_t;
    auto read_group = [&](int group, v8i16_t (&operand)[4]) __attribute__((always_inline)) {
        const unsigned char* rows = values + (16 * group) * kValueRowBytes + value_read;
#pragma unroll
        for (int db = 0; db < 4; ++db) {
            const v4i16_t low = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4_t)(rows + db * 64));
            const v4i16_t high = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4_t)(rows + 8 * kValueRowBytes + db * 64));
            operand[db] = __builtin_shufflevector(low, high, 0, 1, 2, 3, 4, 5, 6, 7);
        }
    };
    auto weights_of = [&](const f32x16_t& s, int j) __attribute__((always_inline)) {
        return make_uint4(pack_pair(s[8 * j + 0], s[8 * j + 1]), pack_pair(s[8 * j + 2], s[8 * j + 3]),
                          pack_pair(s[8 * j + 4], s[8 * j + 5]), pack_pair(s[8 * j + 6], s[8 * j + 7]));
    };
    auto multiply = [&](const v8i16_t (&operand)[4], const uint4& weights) __attribute__((always_inline)) {
#pragma unroll
        for (int db = 0; db < 4; ++db)
            state.out[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, operand[db]),
                                                              __builtin_bit_cast(bf16x8_t, weights), state.out[db], 0, 0, 0);
    };
    v8i16_t even[4], odd[4];
    read_group(0, even);
    read_group(1, odd);
    multiply(even, weights_of(s0, 0));
    if (live1) read_group(2, even);
    multiply(odd, weights_of(s0, 1));
    if (live1) {
        read_group(3, odd);
        multiply(even, weights_of(s1, 0));
        multiply(odd, weights_of(s1, 1));
    }
}

// Scores and fold in one go.
template <bool SOFTCAP, class Hidden>
SINGE_DEVICE void fold_staged_keys(RowState& state, const bf16x8_t (&q)[8], const unsigned char* keys,
                                   const unsigned char* values, unsigned int key_read, unsigned int value_read,
                                   unsigned int hi, float factor, bool live1, bool edge, Hidden&& hidden,
                                   float cap_scale = 0.0f, float cap_log2e = 0.0f) {
    Scores scores;
    score_staged_keys(scores, q, keys, key_read, live1);
    fold_scores<SOFTCAP>(state, scores, values, value_read, hi, factor, live1, edge, hidden, cap_scale, cap_log2e);
}

}  // namespace prefill
