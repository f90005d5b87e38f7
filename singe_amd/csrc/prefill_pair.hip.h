// The two-tile block of the flash-attention prefill kernels that give a wave alone on its SIMD two 32-row tiles
// (fmha_prefill_pair.hip says why and how; paged_attention_pair.hip is the same loop over a paged cache): the score
// products as assembly with their register classes spelled out, Q^T loaded straight into accumulation registers, the
// row maxima of two score tiles in alternating chains, and fold_pair_block, one 32-key block of both tiles with its
// vector work dealt out over the slots between its matrix instructions (32 at head_dim 128, 24 at 96, 16 at 64, ...: the text of the
// block is written by prefill_pair_deal.py).
#pragma once

#include "prefill_blocks.hip.h"

namespace prefill {

static_assert(kHeadDim % 16 == 0 && kHeadDim >= 16 && kHeadDim <= 128, "the two-tile kernels are built for the multiples of 16 up to 128");

// The kernels' names carry the head dimension they were built for.
#define SINGE_PAIR_DIM_(N) d##N
#define SINGE_PAIR_DIM_OF(N) SINGE_PAIR_DIM_(N)
#define SINGE_PAIR_DIM SINGE_PAIR_DIM_OF(SINGE_HEAD_DIM)
#define SINGE_PAIR_JOIN_(A, B, C, D, E) A##_##B##_##C##_##D##_##E
#define SINGE_PAIR_JOIN(A, B, C, D, E) SINGE_PAIR_JOIN_(A, B, C, D, E)

constexpr int kPairWaves = 4;
constexpr unsigned int kPairRows = 64u * kPairWaves;  // query rows of a workgroup
constexpr int kPairStages = 4;                        // of K and of V: a tile is loaded three tiles ahead
constexpr int kPairAhead = kPairStages - 1;
constexpr int kPairValueBase = kPairStages * kTileBytes;
constexpr int kPairLdsBytes = 2 * kPairStages * kTileBytes;
// A tile of 32 output rows a wave, behind the stages of the kernels that store through LDS (store_rows below).
constexpr int kPairStoreBytes = kPairWaves * 32 * kRowBytes;

// A tile's direct-to-LDS loads fill whole 256-byte LDS rows, sixteen 16-byte places each, from cache rows of
// kGlobalRowBytes.  Below head_dim 128 some places hold no chunk of the row: their lanes fetch one of the row's chunks
// again, which lands where nobody reads, so the load needs no predicate (and what the half-used last dim block of an odd
// multiple of 16 would read there is finite).
SINGE_DEVICE unsigned int fetched_chunk(unsigned int chunk_of_place) { return chunk_of_place % (kGlobalRowBytes / 16u); }

typedef v4i16_t __attribute__((address_space(3))) * lds_tr_t;

typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
// s (+)= k . q^T with s in vector registers, where the vector unit reads it, and q in accumulation registers: as a
// built-in the compiler would give it an accumulation-register destination, like every matrix instruction of a kernel
// with more than 256 registers.
// SETTLED: the operands were written long ago (the loop: K operands come from LDS reads the compiler waits for, Q^T
// never changes).  Otherwise two idle issue slots come first, what a matrix instruction needs after a vector
// instruction wrote one of its operands.
template <bool FIRST, bool SETTLED, class Half>
SINGE_DEVICE void score_step(f32x16_t& s, const uint4& k_bits, const u32x4_t& q) {
    const u32x4_t k = __builtin_bit_cast(u32x4_t, k_bits);
#define SINGE_SCORE_STEP(OPCODE)                                                                                              \
    if constexpr (FIRST && SETTLED) asm volatile(OPCODE " %0, %1, %2, 0" : "=&v"(s) : "v"(k), "a"(q));                          \
    else if constexpr (FIRST) asm volatile("s_nop 1\n\t" OPCODE " %0, %1, %2, 0" : "=&v"(s) : "v"(k), "a"(q));                 \
    else if constexpr (SETTLED) asm volatile(OPCODE " %0, %1, %2, %0" : "+v"(s) : "v"(k), "a"(q));                             \
    else asm volatile("s_nop 1\n\t" OPCODE " %0, %1, %2, %0" : "+v"(s) : "v"(k), "a"(q));
    if constexpr (std::is_same_v<Half, F16>) {
        SINGE_SCORE_STEP("v_mfma_f32_32x32x16_f16")
    } else {
        SINGE_SCORE_STEP("v_mfma_f32_32x32x16_bf16")
    }
#undef SINGE_SCORE_STEP
}

// Sixteen bytes from global memory straight into accumulation registers: Q^T is born there, as a value whose only
// class is the one the score products read it from, so the register allocator has no vector-register home to copy it
// back from in front of each use.  The compiler does not know this is a load: accumulation_loads_landed() before
// the first use.
SINGE_DEVICE u32x4_t load_to_accumulation(const void* address) {
    u32x4_t loaded;
    asm volatile("global_load_dwordx4 %0, %1, off" : "=a"(loaded) : "v"(address) : "memory");
    return loaded;
}
SINGE_DEVICE unsigned int lds_address(const unsigned char* in_lds) {
    return static_cast<unsigned int>(reinterpret_cast<size_t>((lds_words_t)(in_lds)));
}

// Sixteen bytes from LDS straight into accumulation registers: the same birth for a Q^T that was worked out in vector
// registers (a fused rotation) and parked in LDS on its way.  A wave's LDS operations run in order, so the read sees
// what the same lane wrote just before; accumulation_loads_landed() before the first use.
SINGE_DEVICE u32x4_t lds_to_accumulation(unsigned int lds_byte_address) {
    u32x4_t loaded;
    asm volatile("ds_read_b128 %0, %1" : "=a"(loaded) : "v"(lds_byte_address) : "memory");
    return loaded;
}
// All of this wave's loads but the eight it issued last (a tile's: four of K, four of V) have completed.
SINGE_DEVICE void older_loads_landed() { __builtin_amdgcn_s_waitcnt(0x0F78); }  // vmcnt(8), other counters left alone
SINGE_DEVICE void accumulation_loads_landed() { asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory"); }

// The scores of a whole block outside the scheduled loop (the first block, the diagonal tile): the same products, then
// the wait the compiler would have put in front of the first reader had it known what the statements above it are.
template <class Half>
SINGE_DEVICE void score_block_pair(Half, f32x16_t& s, const u32x4_t (&q)[kSteps], const unsigned char* keys, const ReadOffsets& offsets) {
    uint4 operand[kSteps];
    read_key_operands(operand, keys, offsets);
    static_for<kSteps>([&](auto step) { score_step<step.value == 0, false, Half>(s, operand[step.value], q[step.value]); });
    asm volatile("s_nop 7\n\ts_nop 7" : "+v"(s));
}

// The row maxima of two score tiles, the two chains a statement apart so that no instruction waits for the one before
// it (the compiler puts an idle slot after every statement whose instruction it does not know): three statements of
// eight instructions, dealt to three slots of the schedule.
SINGE_DEVICE void row_maxima_0(const f32x16_t& a, const f32x16_t& b, float& ma, float& na, float& mb, float& nb) {
    asm volatile(
        "v_max3_f32 %0, %4, %5, %6\n\tv_max3_f32 %2, %14, %15, %16\n\tv_max3_f32 %1, %7, %8, %9\n\tv_max3_f32 %3, %17, %18, %19\n\t"
        "v_max3_f32 %0, %0, %10, %11\n\tv_max3_f32 %2, %2, %20, %21\n\tv_max3_f32 %1, %1, %12, %13\n\tv_max3_f32 %3, %3, %22, %23"
        : "=&v"(ma), "=&v"(na), "=&v"(mb), "=&v"(nb)
        : "v"(a[0]), "v"(a[1]), "v"(a[2]), "v"(a[3]), "v"(a[4]), "v"(a[5]), "v"(a[6]), "v"(a[7]), "v"(a[8]), "v"(a[9]), "v"(b[0]), "v"(b[1]),
          "v"(b[2]), "v"(b[3]), "v"(b[4]), "v"(b[5]), "v"(b[6]), "v"(b[7]), "v"(b[8]), "v"(b[9]));
}
SINGE_DEVICE void row_maxima_1(const f32x16_t& a, const f32x16_t& b, float& ma, float& na, float& mb, float& nb) {
    asm volatile(
        "v_max3_f32 %0, %0, %4, %5\n\tv_max3_f32 %2, %2, %10, %11\n\tv_max3_f32 %1, %1, %6, %7\n\tv_max3_f32 %3, %3, %12, %13\n\t"
        "v_max3_f32 %0, %0, %8, %9\n\tv_max3_f32 %2, %2, %14, %15\n\tv_max_f32 %0, %0, %1\n\tv_max_f32 %2, %2, %3"
        : "+v"(ma), "+v"(na), "+v"(mb), "+v"(nb)
        : "v"(a[10]), "v"(a[11]), "v"(a[12]), "v"(a[13]), "v"(a[14]), "v"(a[15]), "v"(b[10]), "v"(b[11]), "v"(b[12]), "v"(b[13]), "v"(b[14]),
          "v"(b[15]));
}
// (the two lanes of a query exchange their maxima: see swap32_max)
SINGE_DEVICE void row_maxima_2(float& ma, float& mb) {
    float ta, tb;
    asm volatile(
        "v_mov_b32 %2, %0\n\tv_mov_b32 %3, %1\n\ts_nop 0\n\tv_permlane32_swap_b32 %0, %2\n\tv_permlane32_swap_b32 %1, %3\n\t"
        "v_max_f32 %0, %0, %2\n\tv_max_f32 %1, %1, %3"
        : "+v"(ma), "+v"(mb), "=&v"(ta), "=&v"(tb));
}

// Normalises the 32 rows of one tile, rounds them and stores them.  Lane (query, hi) holds dims 32 db + 8 (r / 4) +
// 4 hi + (r % 4) of its row: stored from there, an instruction would touch 32 rows with sixteen bytes each.  The rows go
// through the wave's own 8 KiB behind the stages instead (which it may use while other waves still fold their tiles):
// chunk c of row q sits at place c ^ (q % 16), its halves swapped for q >= 16, so that neither the 8-byte writes nor the
// 16-byte reads meet in a bank; lane l then takes place l % 16 of row 4 i + l / 16, and an instruction stores four whole
// rows.  row_address(r): where row r of the tile goes, or null.  A wave's LDS operations run in order, so the next tile's
// writes come after this one's reads.
template <class Half, class RowAddress>
SINGE_DEVICE void store_rows(Half half, const RowState& state, float inverse, unsigned int lane, unsigned char* staging, RowAddress&& row_address) {
    const unsigned int column = lane & 31u, hi = lane >> 5;
    unsigned char* const mine = staging + column * kRowBytes + 8u * (hi ^ (column >> 4));
#pragma unroll
    for (int db = 0; db < kDimBlocks; ++db)
#pragma unroll
        for (int quad = 0; quad < 4; ++quad) {
            if (32 * db + 8 * quad >= kHeadDim) continue;  // (the last dim block of an odd multiple of 16 is half)
            uint2 packed;
            packed.x = pack_pair(half, state.out[db][4 * quad + 0] * inverse, state.out[db][4 * quad + 1] * inverse);
            packed.y = pack_pair(half, state.out[db][4 * quad + 2] * inverse, state.out[db][4 * quad + 3] * inverse);
            *reinterpret_cast<uint2*>(mine + 16u * ((4u * db + quad) ^ (column & 15u))) = packed;
        }
    const unsigned int row = lane >> 4, place = lane & 15u;
#pragma unroll
    for (unsigned int i = 0; i < 8; ++i) {
        const unsigned int r = 4u * i + row, chunk = place ^ (r & 15u);
        uint4 bits = *reinterpret_cast<const uint4*>(staging + r * kRowBytes + 16u * place);
        if (i >= 4) bits = make_uint4(bits.z, bits.w, bits.x, bits.y);
        uint16_t* const to = row_address(r);
        if (to != nullptr && chunk < kGlobalRowBytes / 16u) *reinterpret_cast<uint4*>(to + 8u * chunk) = bits;
    }
}

// One 32-key block b for both row tiles.  On entry a_cur / b_cur hold the raw scores of block b (shift_a / shift_b:
// minus the rows' reference points, which already cover them) and `operand` the K operands of block b + 1; the V^T
// operands of block b are read in the block's first half, from value_origin (the first V stage, kept where the
// compiler cannot fold its address into the offset) + the lane's offsets + `values` (the block's byte offset from
// there, a constant once inlined: together with the stage's own address it would not fit the instruction's 16 bits).
// On return a_nxt / b_nxt hold the raw scores of block b + 1 and largest_a / largest_b their scaled row maxima,
// `operand` the K operands of block b + 2 (read from keys_after); the rows' sums and O^T have taken block b in; the
// return value says whether some row's maximum has run too far ahead of its reference point (the test is part of the
// schedule; moving the references, which is rare, is the caller's).  issue(0 .. 3) is called once each (four of
// the tile's eight direct-to-LDS loads of this wave).
template <class Half, class Issue>
SINGE_DEVICE bool fold_pair_block(Half half, RowState& A, RowState& B, f32x16_t& a_cur, f32x16_t& b_cur, f32x16_t& a_nxt, f32x16_t& b_nxt,
                                  float factor, float shift_a, float shift_b, float& largest_a_out, float& largest_b_out,
                                  const u32x4_t (&qa)[kSteps], const u32x4_t (&qb)[kSteps], uint4 (&operand)[kSteps], const unsigned char* __restrict__ keys_after,
                                  const unsigned char* __restrict__ value_origin, unsigned int values, const ReadOffsets& offsets, Issue&& issue) {
    unsigned int wa[2][4], wb[2][4];
    v8i16_t v[2][kDimBlocks];
    float total_a = 0.0f, total_b = 0.0f;
    float largest_a, other_a, largest_b, other_b;
    bool lagging;
#define QK(S, Q, J) score_step<(J) == 0, true, Half>(S, operand[J], Q[J])
#define PV(X, H, D, WORDS) \
    X.out[D] = mma(half, __builtin_bit_cast(uint4, v[H][D]), make_uint4(WORDS[H][0], WORDS[H][1], WORDS[H][2], WORDS[H][3]), X.out[D])
#define E(S, I, SHIFT) S[I] = fast_exp2(fmaf(S[I], factor, SHIFT))
// (as a statement the compiler must keep in its place: a plain addition, whose result nothing needs before the block's
// end, is collected with all the others behind the last matrix instruction)
#define T(TOTAL, S, I) asm volatile("v_add_f32_e32 %0, %1, %0" : "+v"(TOTAL) : "v"(S[I]))
#define W(WORDS, S, I) WORDS[(I) / 4][(I) % 4] = pack_pair(half, S[2 * (I)], S[2 * (I) + 1])
#define ROW_MAXIMA_0 row_maxima_0(a_nxt, b_nxt, largest_a, other_a, largest_b, other_b)
#define ROW_MAXIMA_1 row_maxima_1(a_nxt, b_nxt, largest_a, other_a, largest_b, other_b)
#define ROW_MAXIMA_2 row_maxima_2(largest_a, largest_b)
#define LAG_TEST                             \
    largest_a *= factor;                     \
    largest_b *= factor;                     \
    lagging = __any(reference_lags(A, largest_a) || reference_lags(B, largest_b))
#define KR(J) operand[J] = *reinterpret_cast<const uint4*>(keys_after + offsets.key(J))
#define VR(H, D)                                                                                                                        \
    {                                                                                                                                   \
        const v4i16_t low = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_tr_t)(value_origin + offsets.value(D) + (values + (16 * (H)) * kRowBytes))); \
        const v4i16_t high = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_tr_t)(value_origin + offsets.value(D) + (values + (16 * (H) + 8) * kRowBytes))); \
        v[H][D] = __builtin_shufflevector(low, high, 0, 1, 2, 3, 4, 5, 6, 7);                                                        \
    }
#if SINGE_HEAD_DIM == 128
#include "prefill_pair_block_d128.inc"
#elif SINGE_HEAD_DIM == 112
#include "prefill_pair_block_d112.inc"
#elif SINGE_HEAD_DIM == 96
#include "prefill_pair_block_d96.inc"
#elif SINGE_HEAD_DIM == 80
#include "prefill_pair_block_d80.inc"
#elif SINGE_HEAD_DIM == 64
#include "prefill_pair_block_d64.inc"
#elif SINGE_HEAD_DIM == 48
#include "prefill_pair_block_d48.inc"
#elif SINGE_HEAD_DIM == 32
#include "prefill_pair_block_d32.inc"
#else
#include "prefill_pair_block_d16.inc"
#endif
#undef QK
#undef PV
#undef E
#undef T
#undef W
#undef KR
#undef ROW_MAXIMA_0
#undef ROW_MAXIMA_1
#undef ROW_MAXIMA_2
#undef LAG_TEST
#undef VR
    A.running_sum += total_a;
    B.running_sum += total_b;
    largest_a_out = largest_a;
    largest_b_out = largest_b;
    return lagging;
}

}  // namespace prefill
