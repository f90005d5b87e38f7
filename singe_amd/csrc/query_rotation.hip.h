// The query rotation the paged attention kernels fuse (paged_attention.hip, paged_attention_pair.hip): a lane's
// share of one query row, as the eight 16-byte chunks of Q^T it holds, is normalised, turned by the token's angles and
// rounded on its way into the registers.
#pragma once

#include "kernel_args.h"
#include "prefill_blocks.hip.h"

namespace prefill {

// One value of an angle table of f32, bf16 or f16 (SingeElement).
SINGE_DEVICE float table_value(const void* table, uint32_t table_type, size_t at) {
    if (table_type == kElementF32) return static_cast<const float*>(table)[at];
    if (table_type == kElementBf16) return __builtin_bit_cast(float, static_cast<unsigned int>(static_cast<const unsigned short*>(table)[at]) << 16);
    return static_cast<float>(static_cast<const _Float16*>(table)[at]);
}

// Eight consecutive values of such a table, the index a multiple of eight: as one or two 16-byte loads when the table
// starts on a 16-byte boundary, one by one otherwise.
SINGE_DEVICE void table_values8(float (&out)[8], const void* table, uint32_t table_type, size_t at) {
    if (reinterpret_cast<uintptr_t>(table) % 16 != 0) {
#pragma unroll
        for (int i = 0; i < 8; ++i) out[i] = table_value(table, table_type, at + i);
        return;
    }
    if (table_type == kElementF32) {
        const float4* from = reinterpret_cast<const float4*>(static_cast<const float*>(table) + at);
        const float4 low = from[0], high = from[1];
        out[0] = low.x; out[1] = low.y; out[2] = low.z; out[3] = low.w;
        out[4] = high.x; out[5] = high.y; out[6] = high.z; out[7] = high.w;
        return;
    }
    const uint4 raw = *reinterpret_cast<const uint4*>(static_cast<const unsigned short*>(table) + at);
    const unsigned int words[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const unsigned short bits = static_cast<unsigned short>(words[i / 2] >> (16 * (i % 2)));
        out[i] = table_type == kElementBf16 ? __builtin_bit_cast(float, static_cast<unsigned int>(bits) << 16)
                                            : static_cast<float>(__builtin_bit_cast(_Float16, bits));
    }
}

// bits[s]: dims 16 s + 8 hi .. + 7 of the lane's query row (lanes l and l ^ 32 hold one row, hi = l / 32), as loaded.
// `token`: the row's token in the packed queries (its row of the angle tables).
template <class Half>
SINGE_DEVICE void rotate_query(Half half, uint4 (&bits)[kSteps], const PagedAttentionArgs& a, size_t token, bool row_valid, unsigned int hi) {
    // The query arrives before its rotation (paged_attention.rs:881-977): an optional RMS norm over
    // the head dimension with an optional weight, then half-split pairs (p, p + head_dim / 2) turned by the
    // token's angles, first = a cos - b sin, second = b cos + a sin, rounded to the query's type as the
    // reference rounds what it stores in its tile.  The other half of the row's squares is one swap away.
    constexpr bool kF16 = std::is_same<Half, F16>::value;
    constexpr uint32_t kOwnElement = kF16 ? kElementF16 : kElementBf16;
    auto wide = [](unsigned int pair, int upper) __attribute__((always_inline)) {
        if constexpr (kF16) return static_cast<float>(__builtin_bit_cast(_Float16, static_cast<unsigned short>(upper ? pair >> 16 : pair & 0xffffu)));
        else return __builtin_bit_cast(float, upper ? pair & 0xffff0000u : pair << 16);
    };
    float scale = 1.0f;
    if (a.has_query_norm != 0) {
        float squares = 0.0f;
#pragma unroll
        for (int s = 0; s < kSteps; ++s) {
            const unsigned int words[4] = {bits[s].x, bits[s].y, bits[s].z, bits[s].w};
#pragma unroll
            for (int w = 0; w < 4; ++w) squares += wide(words[w], 0) * wide(words[w], 0) + wide(words[w], 1) * wide(words[w], 1);
        }
        squares = swap32_sum(squares);
        scale = rsqrtf(squares / static_cast<float>(kHeadDim) + a.query_eps);
    }
    constexpr int kPairs = kHeadDim / 2;
    const bool normed = a.has_query_norm != 0, weighted = normed && a.query_weight != nullptr;
    // One chunk of eight dims turned against its partner chunk: `mine` holds dims dim0 .. dim0 + 7.
    auto turn = [&](uint4 mine, uint4 partner, unsigned int dim0, bool mine_is_first) __attribute__((always_inline)) {
        const unsigned int pair0 = mine_is_first ? dim0 : dim0 - kPairs, partner_dim0 = mine_is_first ? dim0 + kPairs : dim0 - kPairs;
        float cosines[8], sines[8], own_weights[8], partner_weights[8];
        table_values8(cosines, a.cos, a.table_type, token * kPairs + pair0);
        table_values8(sines, a.sin, a.table_type, token * kPairs + pair0);
        if (weighted) {
            table_values8(own_weights, a.query_weight, kOwnElement, dim0);
            table_values8(partner_weights, a.query_weight, kOwnElement, partner_dim0);
        }
        const unsigned int own_words[4] = {mine.x, mine.y, mine.z, mine.w}, partner_words[4] = {partner.x, partner.y, partner.z, partner.w};
        unsigned int turned[4];
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            float rotated[2];
#pragma unroll
            for (int upper = 0; upper < 2; ++upper) {
                float own = wide(own_words[w], upper), other = wide(partner_words[w], upper);
                if (normed) {
                    own *= scale;
                    other *= scale;
                    if (weighted) {
                        own *= own_weights[2 * w + upper];
                        other *= partner_weights[2 * w + upper];
                    }
                }
                const float cosine = cosines[2 * w + upper], sine = sines[2 * w + upper];
                // first = a cos - b sin, second = b cos + a sin
                rotated[upper] = mine_is_first ? own * cosine - other * sine : own * cosine + other * sine;
            }
            turned[w] = row_valid ? pack_pair(half, rotated[0], rotated[1]) : 0u;
        }
        return make_uint4(turned[0], turned[1], turned[2], turned[3]);
    };
    if constexpr (kSteps % 2 == 0) {
        // Multiples of 32: a lane holds both halves of its pairs (dims 16 s + 8 hi + j and the same + head_dim / 2),
        // whole steps apart, so a step's angles and weights are fetched once for both.
        constexpr int kHalfSteps = kSteps / 2;
#pragma unroll
        for (int s = 0; s < kHalfSteps; ++s) {
            unsigned int first_words[4] = {bits[s].x, bits[s].y, bits[s].z, bits[s].w};
            unsigned int second_words[4] = {bits[s + kHalfSteps].x, bits[s + kHalfSteps].y, bits[s + kHalfSteps].z, bits[s + kHalfSteps].w};
            const unsigned int first_pair = 16u * s + 8u * hi;
            float cosines[8], sines[8], low_weights[8], high_weights[8];
            table_values8(cosines, a.cos, a.table_type, token * kPairs + first_pair);
            table_values8(sines, a.sin, a.table_type, token * kPairs + first_pair);
            if (weighted) {
                table_values8(low_weights, a.query_weight, kOwnElement, first_pair);
                table_values8(high_weights, a.query_weight, kOwnElement, first_pair + kPairs);
            }
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                float rotated_first[2], rotated_second[2];
#pragma unroll
                for (int upper = 0; upper < 2; ++upper) {
                    float first = wide(first_words[w], upper), second = wide(second_words[w], upper);
                    if (normed) {
                        first *= scale;
                        second *= scale;
                        if (weighted) {
                            first *= low_weights[2 * w + upper];
                            second *= high_weights[2 * w + upper];
                        }
                    }
                    const float cosine = cosines[2 * w + upper], sine = sines[2 * w + upper];
                    rotated_first[upper] = first * cosine - second * sine;
                    rotated_second[upper] = second * cosine + first * sine;
                }
                first_words[w] = row_valid ? pack_pair(half, rotated_first[0], rotated_first[1]) : 0u;
                second_words[w] = row_valid ? pack_pair(half, rotated_second[0], rotated_second[1]) : 0u;
            }
            bits[s] = make_uint4(first_words[0], first_words[1], first_words[2], first_words[3]);
            bits[s + kHalfSteps] = make_uint4(second_words[0], second_words[1], second_words[2], second_words[3]);
        }
    } else {
        // Odd multiples of 16: half a head is a whole number of steps and a half, so the partner of a lane's
        // chunk sits in the row's other lane (lane ^ 32), at another step: chunk (s, hi = 0) pairs with
        // (s + (kSteps - 1) / 2, hi = 1) and chunk (s, hi = 1) with (s + (kSteps + 1) / 2, hi = 0).  Each lane
        // hands the other what it asks for at step s, one lane swap per word.
        constexpr int kLow = (kSteps - 1) / 2, kHigh = (kSteps + 1) / 2;
        uint4 turned[kSteps];
#pragma unroll
        for (int s = 0; s < kSteps; ++s) {
            // what the other lane of the row needs from this one at its step s
            const int wanted_from_low = s <= kLow - 1 ? s + kHigh : s - kLow;  // asked by hi = 1 of the hi = 0 lane
            const int wanted_from_high = s <= kLow ? s + kLow : s - kHigh;     // asked by hi = 0 of the hi = 1 lane
            const uint4 give = hi == 0 ? bits[wanted_from_low] : bits[wanted_from_high];
            uint4 partner;
            partner.x = __shfl_xor(give.x, 32, 64);
            partner.y = __shfl_xor(give.y, 32, 64);
            partner.z = __shfl_xor(give.z, 32, 64);
            partner.w = __shfl_xor(give.w, 32, 64);
            const unsigned int dim0 = 16u * s + 8u * hi;
            turned[s] = turn(bits[s], partner, dim0, dim0 < static_cast<unsigned int>(kPairs));
        }
#pragma unroll
        for (int s = 0; s < kSteps; ++s) bits[s] = turned[s];
    }
}

}  // namespace prefill
