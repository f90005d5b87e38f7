// Block-pipelined core of the dense bf16 flash-attention prefill kernel: one wave folds blocks of 32 keys
// into the running softmax state of its 32 query rows, with the score products of the next block issued
// before the softmax of the current one so the matrix core and the vector unit work at the same time.
// Everything is kept transposed so the softmax weights never leave registers (see prefill_core.hip.h for
// the register layouts, which this file shares):
//
//   S^T[key, query] = K . Q^T      v_mfma_f32_32x32x16_bf16 (or _f16), A = K rows from LDS, B = the wave's Q^T;
//   O^T[dim, query] += V^T . P^T   A = V^T through ds_read_b64_tr_b16, B = P^T packed from the S^T registers.
//
// Tiles of 64 keys reach LDS straight from global memory (global_load_lds_dwordx4: lane l of a wave puts
// its 16 bytes at the wave's LDS base + 16 l, whatever global address it read), so rows are stored
// unpadded, 256 bytes each, and bank conflicts are avoided by permuting the sixteen 16-byte chunks of a
// row instead: K keeps chunk c of row r at position c ^ (r & 15), V at position c ^ 4 (r & 3).  The
// permutation is applied on the global side (which chunk a lane fetches) and undone by the read offsets.
#pragma once

#include "prefill_core.hip.h"

namespace prefill {

constexpr int kRowBytes = 256;                       // an LDS row: one key's 128 halves; at head_dim 64 its chunks 0 .. 7,
                                                     // scattered over the sixteen positions by the same permutation
constexpr int kGlobalRowBytes = 2 * kHeadDim;        // one key's halves in global memory
constexpr int kTileBytes = kKeyTile * kRowBytes;     // 64 keys of K or of V
constexpr int kBlockBytes = 32 * kRowBytes;
// LDS of a workgroup: three stages of K and two of V, so K can be loaded two tiles ahead and V one.
constexpr int kKeyStages = 3, kValueStages = 2;
constexpr int kValueBase = kKeyStages * kTileBytes;
constexpr int kStagedLdsBytes = (kKeyStages + kValueStages) * kTileBytes;

typedef unsigned int __attribute__((address_space(3))) * lds_words_t;


// Per-lane LDS read offsets inside a 32-key block, kept as a base and the bits the row's permutation
// flips so that each read's offset costs one xor-add instead of a register.
struct ReadOffsets {
    unsigned int key_base, key_flip;      // K operand of step s: key_base + ((32 s) ^ key_flip)
    unsigned int value_base, value_flip;  // V^T operand of dim block db: value_base + ((64 db) ^ value_flip)
    SINGE_DEVICE unsigned int key(unsigned int step) const { return ((32u * step) ^ key_flip) + key_base; }
    SINGE_DEVICE unsigned int value(unsigned int db) const { return ((64u * db) ^ value_flip) + value_base; }
};

// K: row lane % 32, chunk (2 s + hi) ^ (row & 15), 16 bytes per chunk.  V^T: keys 4 hi + (sub >> 2) of a
// 16-key group (add 8 rows for its high half), chunk (4 db + 2 (group & 1) + ((sub & 3) >> 1)) ^ 4 (row & 3),
// 8 bytes at 8 (sub & 1) inside it.
SINGE_DEVICE ReadOffsets read_offsets(unsigned int lane) {
    ReadOffsets offsets;
    const unsigned int hi = lane >> 5, row = lane & 31u;
    offsets.key_base = row * kRowBytes;
    offsets.key_flip = ((lane & 15u) ^ hi) * 16u;
    const unsigned int group = lane >> 4, sub = lane & 15u, row_in_quad = sub >> 2;
    offsets.value_base = (4u * hi + row_in_quad) * kRowBytes + (2u * (group & 1u) + ((sub & 3u) >> 1)) * 16u + 8u * (sub & 1u);
    offsets.value_flip = 64u * row_in_quad;
    return offsets;
}

// Scores of the wave's 32 queries against the 32 keys of the block at `keys` (LDS byte address of the
// block's first row).  The products run on while the caller does other work.
template <class Half>
SINGE_DEVICE void score_block(Half half, f32x16_t& scores, const uint4 (&q)[kSteps], const unsigned char* keys, const ReadOffsets& offsets) {
    f32x16_t s;
#pragma unroll
    for (int r = 0; r < 16; ++r) s[r] = 0.0f;
    uint4 operand[kSteps];
#pragma unroll
    for (int step = 0; step < kSteps; ++step) operand[step] = *reinterpret_cast<const uint4*>(keys + offsets.key(step));
#pragma unroll
    for (int step = 0; step < kSteps; ++step)
        s = mma(half, operand[step], q[step], s);
    scores = s;
}

// Whether a row's scaled maximum has run too far ahead of the point its weights are scaled by (or the row sees its
// first key).
SINGE_DEVICE bool reference_lags(const RowState& state, float largest) {
    return largest > state.reference + kMaxLag || (state.reference == -INFINITY && largest != -INFINITY);
}

// Moves the reference point up to the row's maximum and rescales what was summed under the old one.
SINGE_DEVICE void move_reference(RowState& state, float largest) {
    const float moved = fmaxf(state.reference, largest);
    const float base = moved == -INFINITY ? 0.0f : moved;
    const float rescale = fast_exp2(state.reference - base);
    state.running_sum *= rescale;
#pragma unroll
    for (int db = 0; db < kDimBlocks; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) state.out[db][r] *= rescale;
    state.reference = moved;
}

// First half of folding a 32-key block: hides what the mask hides, takes the row maxima and moves the
// softmax reference point when a row's maximum has run too far ahead of it.  Returns the shift the
// exponentials take (minus the reference, 0 for rows that have seen nothing).
//   edge     true when some score of the block must be hidden; then hidden(key_in_block) says which
//            (key_in_block = 8(r / 4) + 4hi + (r % 4) for accumulator register r)
template <class Hidden>
SINGE_DEVICE float begin_block(RowState& state, f32x16_t& s, unsigned int hi, float factor, bool edge, Hidden&& hidden) {
    if (edge) {
#pragma unroll
        for (int r = 0; r < 16; ++r)
            if (hidden(8u * (r >> 2) + 4u * hi + (r & 3))) s[r] = -INFINITY;
    }
    float largest = max3(s[0], s[1], s[2]), other = max3(s[3], s[4], s[5]);
    largest = max3(largest, s[6], s[7]);
    other = max3(other, s[8], s[9]);
    largest = max3(largest, s[10], s[11]);
    other = max3(other, s[12], s[13]);
    largest = max3(largest, s[14], s[15]);
    largest = swap32_max(max2(largest, other)) * factor;  // both lanes of a query agree from here on
    if (__any(reference_lags(state, largest))) move_reference(state, largest);
    return state.reference == -INFINITY ? 0.0f : -state.reference;
}

// Second half, free of branches so the compiler can weave its parts together: the scores `s` become
// weights and O^T += V^T . P^T, and, when NEXT is set, the score products of the block at `next_keys` are
// issued in between: one MFMA, then the exponentials of two registers, and so on, so the matrix core
// computes the next block's scores while the vector unit exponentiates this one's.
//   AHEAD       the K operands travel between calls in `operand`: on entry those of the block whose scores
//               are computed here (`next_keys` is not read), on return those of the block at `after_keys`, each
//               read as soon as the product that used its register has been issued, a whole block before
//               its use.  Otherwise the operands are read from `next_keys` at the start of the call.
template <bool NEXT, bool AHEAD = false, class Half>
SINGE_DEVICE void finish_block(Half half, RowState& state, f32x16_t& s, float factor, float shift, const unsigned char* values,
                               const ReadOffsets& offsets, f32x16_t& next, const uint4 (&q)[kSteps], const unsigned char* next_keys,
                               uint4 (&operand)[kSteps], const unsigned char* after_keys) {
    typedef v4i16_t __attribute__((address_space(3))) * lds_v4_t;
    if constexpr (NEXT && !AHEAD) {
#pragma unroll
        for (int step = 0; step < kSteps; ++step) operand[step] = *reinterpret_cast<const uint4*>(next_keys + offsets.key(step));
    }
    v8i16_t first[kDimBlocks], second[kDimBlocks];
#pragma unroll
    for (int db = 0; db < kDimBlocks; ++db) {
        const v4i16_t low = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4_t)(values + offsets.value(db)));
        const v4i16_t high = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4_t)(values + 8 * kRowBytes + offsets.value(db)));
        first[db] = __builtin_shufflevector(low, high, 0, 1, 2, 3, 4, 5, 6, 7);
    }
    f32x16_t upcoming;
#pragma unroll
    for (int r = 0; r < 16; ++r) upcoming[r] = 0.0f;
    float total = 0.0f;
    // The two waves of a SIMD belong to different workgroups and drift apart.  While this one turns scores into weights
    // (a dependent chain on the vector unit, with the next block's score products in between) it goes first; during its
    // value products, which only need the matrix core to be free, the other one does.  Together with the priority
    // around a tile's loads (fold_interior_tile), measured on the dense prefill: 0.580 -> 0.566 ms, on the chunked
    // paged prefill 1.257 -> 1.249 ms; this one alone: 0.567 ms and, on the paged kernel, a loss (1.232 -> 1.249 ms);
    // around the value products instead: 0.592 ms; levels 1 to 3 alike.
    __builtin_amdgcn_s_setprio(1);
#pragma unroll
    for (int step = 0; step < 8; ++step) {
        if (step == 4) {
            // The second half of the values, fetched once half of the K operands have been used up.
#pragma unroll
            for (int db = 0; db < kDimBlocks; ++db) {
                const v4i16_t low = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4_t)(values + 16 * kRowBytes + offsets.value(db)));
                const v4i16_t high = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4_t)(values + 24 * kRowBytes + offsets.value(db)));
                second[db] = __builtin_shufflevector(low, high, 0, 1, 2, 3, 4, 5, 6, 7);
            }
        }
        if constexpr (NEXT) {
            // Eight pairs of exponentials take the block's kSteps products between them.
            if (step < kSteps) {
                upcoming = mma(half, operand[step], q[step], upcoming);
                if constexpr (AHEAD) operand[step] = *reinterpret_cast<const uint4*>(after_keys + offsets.key(step));
            }
        }
        s[2 * step] = fast_exp2(fmaf(s[2 * step], factor, shift));
        s[2 * step + 1] = fast_exp2(fmaf(s[2 * step + 1], factor, shift));
        total += s[2 * step] + s[2 * step + 1];
    }
    __builtin_amdgcn_s_setprio(0);
    state.running_sum += total;
    // O^T += V^T . P^T, 16 keys per MFMA: registers 8j .. 8j+7 are keys 16j + {0..3, 8..11} + 4hi.
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const uint4 weights = make_uint4(pack_pair(half, s[8 * j + 0], s[8 * j + 1]), pack_pair(half, s[8 * j + 2], s[8 * j + 3]),
                                         pack_pair(half, s[8 * j + 4], s[8 * j + 5]), pack_pair(half, s[8 * j + 6], s[8 * j + 7]));
#pragma unroll
        for (int db = 0; db < kDimBlocks; ++db)
            state.out[db] = mma(half, __builtin_bit_cast(uint4, j == 0 ? first[db] : second[db]), weights, state.out[db]);
    }
    if constexpr (NEXT) next = upcoming;
}

template <bool NEXT, class Half>
SINGE_DEVICE void finish_block(Half half, RowState& state, f32x16_t& s, float factor, float shift, const unsigned char* values,
                               const ReadOffsets& offsets, f32x16_t& next, const uint4 (&q)[kSteps], const unsigned char* next_keys) {
    uint4 operand[kSteps];
    finish_block<NEXT, false>(half, state, s, factor, shift, values, offsets, next, q, next_keys, operand, next_keys);
}

// The stages of a tile's iteration, as the tile functions below take them.  The functions' pointer
// parameters are __restrict__ and that is what they are for: once inlined, every LDS read in them is known
// not to touch the stages the iteration's direct-to-LDS loads write, so the compiler does not make the
// first read after those loads wait for them to land (without that knowledge it must, and each tile would
// stall for a round trip to memory).  The caller waits for the loads itself, with loads_landed(), before
// the barrier that hands the stages on.
struct TileStages {
    const unsigned char* keys;       // K of this tile
    const unsigned char* next_keys;  // K of the next tile, landed before the last barrier
    const unsigned char* values;     // V of this tile
    unsigned char* key_dest;         // where K of the tile after next goes
    unsigned char* value_dest;       // where V of the next tile goes
};

// All of this wave's outstanding loads from global memory, those to LDS included, have completed.
SINGE_DEVICE void loads_landed() { __builtin_amdgcn_s_waitcnt(0x0F70); }  // vmcnt(0), other counters left alone

// A tile no mask touches, with another block to come after it: issue(key_dest, value_dest) starts the
// iteration's loads, then both blocks are folded while the scores of the block after each are computed.
// With AHEAD the K operands of those products are read a block early and carried in `operand`: those of the
// tile's second block on entry (read_key_operands before the first tile), of the next tile's on return.
//   shape(scores, which)   turns the raw scores of the tile's first (which = 0) or second block into what the softmax
//                          takes (a score cap, an added mask) before they are folded; the caller then passes the
//                          factor that is left to apply (1 when shape did the scaling).
template <bool AHEAD, class Half, class Issue, class Shape>
SINGE_DEVICE void fold_interior_tile(Half half, RowState& state, f32x16_t& scores, uint4 (&operand)[kSteps], const uint4 (&q)[kSteps],
                                     const ReadOffsets& offsets, unsigned int hi, float factor, const unsigned char* __restrict__ keys,
                                     const unsigned char* __restrict__ next_keys, const unsigned char* __restrict__ values,
                                     unsigned char* __restrict__ key_dest, unsigned char* __restrict__ value_dest, Issue&& issue,
                                     Shape&& shape) {
    // (the tile's loads and their address arithmetic go out ahead of the other wave's work: see finish_block)
    __builtin_amdgcn_s_setprio(2);
    issue(key_dest, value_dest);
    __builtin_amdgcn_s_setprio(0);
    shape(scores, 0u);
    const float shift_even = begin_block(state, scores, hi, factor, false, [](unsigned int) { return false; });
    finish_block<true, AHEAD>(half, state, scores, factor, shift_even, values, offsets, scores, q, keys + kBlockBytes, operand, next_keys);
    __builtin_amdgcn_sched_barrier(0);  // keeps the second block's operand reads out of the first block's registers
    shape(scores, 1u);
    const float shift_odd = begin_block(state, scores, hi, factor, false, [](unsigned int) { return false; });
    finish_block<true, AHEAD>(half, state, scores, factor, shift_odd, values + kBlockBytes, offsets, scores, q, next_keys, operand,
                              next_keys + kBlockBytes);
}

template <bool AHEAD, class Half, class Issue>
SINGE_DEVICE void fold_interior_tile(Half half, RowState& state, f32x16_t& scores, uint4 (&operand)[kSteps], const uint4 (&q)[kSteps],
                                     const ReadOffsets& offsets, unsigned int hi, float factor, const unsigned char* __restrict__ keys,
                                     const unsigned char* __restrict__ next_keys, const unsigned char* __restrict__ values,
                                     unsigned char* __restrict__ key_dest, unsigned char* __restrict__ value_dest, Issue&& issue) {
    fold_interior_tile<AHEAD>(half, state, scores, operand, q, offsets, hi, factor, keys, next_keys, values, key_dest, value_dest, issue,
                              [](f32x16_t&, unsigned int) {});
}

// The K operands of the block at `keys`.
SINGE_DEVICE void read_key_operands(uint4 (&operand)[kSteps], const unsigned char* keys, const ReadOffsets& offsets) {
#pragma unroll
    for (int step = 0; step < kSteps; ++step) operand[step] = *reinterpret_cast<const uint4*>(keys + offsets.key(step));
}

// Any other tile: the same steps one after the other, each only if the wave still has that block;
// fold(block, scores, values) applies the masks and folds one block.
template <class Half, class Issue, class Fold>
SINGE_DEVICE void fold_edge_tile(Half half, f32x16_t& scores, const uint4 (&q)[kSteps], const ReadOffsets& offsets, unsigned int block,
                                 unsigned int wave_blocks, const unsigned char* __restrict__ keys,
                                 const unsigned char* __restrict__ next_keys, const unsigned char* __restrict__ values,
                                 unsigned char* __restrict__ key_dest, unsigned char* __restrict__ value_dest, Issue&& issue, Fold&& fold) {
    issue(key_dest, value_dest);
    if (block < wave_blocks) fold(block, scores, values);
    if (block + 1 < wave_blocks) {
        score_block(half, scores, q, keys + kBlockBytes, offsets);
        fold(block + 1, scores, values + kBlockBytes);
    }
    if (block + 2 < wave_blocks) score_block(half, scores, q, next_keys, offsets);
}

}  // namespace prefill
