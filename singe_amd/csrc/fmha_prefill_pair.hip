// Dense flash-attention prefill for long rows, bf16 or f16, head_dim 128, no options: the same arithmetic and
// register layouts as fmha_prefill.hip (S^T = K . Q^T, per-lane softmax, O^T += V^T . P^T; prefill_core.hip.h), with
// the work laid out the other way round.  There, two waves share a SIMD and each folds keys into 32 query rows;
// what one wave leaves idle the other uses.  Here ONE wave owns a SIMD (up to 512 registers) and folds every key
// block into TWO tiles of 32 query rows, A and B:
//   * each K and V^T operand read from LDS feeds two matrix instructions instead of one, a workgroup's 64-key
//     tile serves 256 query rows instead of 128, and there is one barrier per 64 matrix instructions;
//   * the order of a wave's instructions is the schedule: a block is 32 matrix instructions (8 score products of
//     the NEXT block for A, 8 for B, 8 value products of this block for A, 8 for B) and the vector work of the block
//     (exponentials, sums, packing, the next block's row maxima, LDS operand reads, the tile's loads) is dealt out
//     over the 32 slots between them, at most seven issue cycles a slot, so that each piece is done before the
//     matrix instruction that needs it is issued and the matrix pipe never waits (fold_pair_block);
//   * the score accumulators must be in ordinary vector registers (the vector unit reads them) while O^T and Q^T
//     live in the accumulation registers; the compiler gives every matrix instruction of such a kernel an
//     accumulation-register destination, so the score products are written as assembly with the register classes
//     spelled out.  The distance between a score product and the first vector instruction that reads its result is
//     part of the schedule (at least four slots, some thirty instructions), since the compiler does not see a
//     matrix instruction there.
// query/out [batch, query_len, heads, 128], key/value [batch, key_len, kv_heads, 128] with element strides from
// FmhaPrefillConfig; lse [batch, heads, query_len], natural log.  The host sends calls here whose key_len is a
// multiple of 64 (every tile whole) and that fill the chip with 256-row tiles; everything else stays on
// fmha_prefill.hip.
//
// Grid: one workgroup of four waves per (batch, head, pair of 256-row query tiles), tile i from the end and tile i
// from the start; ids laid out as in fmha_prefill.hip.  LDS: four stages of K and four of V (128 KiB), each tile
// loaded three tiles ahead, straight from global memory, and waited for a tile after it was asked for (a wave alone
// on its SIMD has nobody to cover a wait for fresh loads); one barrier per tile.
#include "kernel_args.h"
#include "prefill_blocks.hip.h"

namespace {

using namespace prefill;
static_assert(kHeadDim == 128, "the two-tile kernel is built for head_dim 128");

constexpr int kPairWaves = 4;
constexpr unsigned int kPairRows = 64u * kPairWaves;  // query rows of a workgroup
constexpr int kPairStages = 4;                        // of K and of V: a tile is loaded three tiles ahead
constexpr int kPairAhead = kPairStages - 1;
constexpr int kPairValueBase = kPairStages * kTileBytes;
constexpr int kPairLdsBytes = 2 * kPairStages * kTileBytes;

typedef v4i16_t __attribute__((address_space(3))) * lds_tr_t;

// s (+)= k . q^T with s in vector registers and q in accumulation registers (see the header comment).
typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
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
// All of this wave's loads but the eight it issued last (a tile's: four of K, four of V) have completed.
SINGE_DEVICE void older_loads_landed() { __builtin_amdgcn_s_waitcnt(0x0F78); }  // vmcnt(8), other counters left alone
SINGE_DEVICE void accumulation_loads_landed() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

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
                                  const u32x4_t (&qa)[8], const u32x4_t (&qb)[8], uint4 (&operand)[8], const unsigned char* __restrict__ keys_after,
                                  const unsigned char* __restrict__ value_origin, unsigned int values, const ReadOffsets& offsets, Issue&& issue) {
    unsigned int wa[2][4], wb[2][4];
    v8i16_t v[2][4];
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
    // slot 0
    QK(a_nxt, qa, 0);
    __builtin_amdgcn_sched_barrier(0);
    issue(0);
    E(a_cur, 0, shift_a);
    __builtin_amdgcn_sched_barrier(0);
    // slot 1
    QK(b_nxt, qb, 0);
    __builtin_amdgcn_sched_barrier(0);
    E(a_cur, 1, shift_a);
    T(total_a, a_cur, 0);
    E(a_cur, 2, shift_a);
    __builtin_amdgcn_sched_barrier(0);
    // slot 2
    QK(a_nxt, qa, 1);
    __builtin_amdgcn_sched_barrier(0);
    issue(1);
    T(total_a, a_cur, 1);
    E(a_cur, 3, shift_a);
    __builtin_amdgcn_sched_barrier(0);
    // slot 3
    QK(b_nxt, qb, 1);
    __builtin_amdgcn_sched_barrier(0);
    T(total_a, a_cur, 2);
    W(wa, a_cur, 0);
    E(a_cur, 4, shift_a);
    T(total_a, a_cur, 3);
    W(wa, a_cur, 1);
    __builtin_amdgcn_sched_barrier(0);
    // slot 4
    QK(a_nxt, qa, 2);
    __builtin_amdgcn_sched_barrier(0);
    issue(2);
    E(a_cur, 5, shift_a);
    T(total_a, a_cur, 4);
    __builtin_amdgcn_sched_barrier(0);
    // slot 5
    QK(b_nxt, qb, 2);
    __builtin_amdgcn_sched_barrier(0);
    E(a_cur, 6, shift_a);
    T(total_a, a_cur, 5);
    E(a_cur, 7, shift_a);
    __builtin_amdgcn_sched_barrier(0);
    // slot 6
    QK(a_nxt, qa, 3);
    __builtin_amdgcn_sched_barrier(0);
    issue(3);
    T(total_a, a_cur, 6);
    W(wa, a_cur, 2);
    T(total_a, a_cur, 7);
    W(wa, a_cur, 3);
    __builtin_amdgcn_sched_barrier(0);
    // slot 7
    QK(b_nxt, qb, 3);
    __builtin_amdgcn_sched_barrier(0);
    E(a_cur, 8, shift_a);
    E(a_cur, 9, shift_a);
    __builtin_amdgcn_sched_barrier(0);
    // slot 8
    QK(a_nxt, qa, 4);
    __builtin_amdgcn_sched_barrier(0);
    VR(0, 0);
    T(total_a, a_cur, 8);
    E(a_cur, 10, shift_a);
    T(total_a, a_cur, 9);
    __builtin_amdgcn_sched_barrier(0);
    // slot 9
    QK(b_nxt, qb, 4);
    __builtin_amdgcn_sched_barrier(0);
    VR(0, 1);
    E(a_cur, 11, shift_a);
    T(total_a, a_cur, 10);
    W(wa, a_cur, 4);
    __builtin_amdgcn_sched_barrier(0);
    // slot 10
    QK(a_nxt, qa, 5);
    __builtin_amdgcn_sched_barrier(0);
    VR(0, 2);
    E(a_cur, 12, shift_a);
    T(total_a, a_cur, 11);
    W(wa, a_cur, 5);
    __builtin_amdgcn_sched_barrier(0);
    // slot 11
    QK(b_nxt, qb, 5);
    __builtin_amdgcn_sched_barrier(0);
    VR(0, 3);
    E(a_cur, 13, shift_a);
    T(total_a, a_cur, 12);
    __builtin_amdgcn_sched_barrier(0);
    // slot 12
    QK(a_nxt, qa, 6);
    __builtin_amdgcn_sched_barrier(0);
    VR(1, 0);
    E(a_cur, 14, shift_a);
    T(total_a, a_cur, 13);
    W(wa, a_cur, 6);
    __builtin_amdgcn_sched_barrier(0);
    // slot 13
    QK(b_nxt, qb, 6);
    __builtin_amdgcn_sched_barrier(0);
    VR(1, 1);
    E(a_cur, 15, shift_a);
    T(total_a, a_cur, 14);
    __builtin_amdgcn_sched_barrier(0);
    // slot 14
    QK(a_nxt, qa, 7);
    __builtin_amdgcn_sched_barrier(0);
    VR(1, 2);
    T(total_a, a_cur, 15);
    W(wa, a_cur, 7);
    E(b_cur, 0, shift_b);
    __builtin_amdgcn_sched_barrier(0);
    // slot 15
    QK(b_nxt, qb, 7);
    __builtin_amdgcn_sched_barrier(0);
    VR(1, 3);
    E(b_cur, 1, shift_b);
    T(total_b, b_cur, 0);
    __builtin_amdgcn_sched_barrier(0);
    // slot 16
    PV(A, 0, 0, wa);
    __builtin_amdgcn_sched_barrier(0);
    KR(0);
    E(b_cur, 2, shift_b);
    T(total_b, b_cur, 1);
    W(wb, b_cur, 0);
    __builtin_amdgcn_sched_barrier(0);
    // slot 17
    PV(A, 0, 1, wa);
    __builtin_amdgcn_sched_barrier(0);
    KR(1);
    E(b_cur, 3, shift_b);
    T(total_b, b_cur, 2);
    __builtin_amdgcn_sched_barrier(0);
    // slot 18
    PV(A, 0, 2, wa);
    __builtin_amdgcn_sched_barrier(0);
    KR(2);
    E(b_cur, 4, shift_b);
    T(total_b, b_cur, 3);
    W(wb, b_cur, 1);
    __builtin_amdgcn_sched_barrier(0);
    // slot 19
    PV(A, 0, 3, wa);
    __builtin_amdgcn_sched_barrier(0);
    KR(3);
    E(b_cur, 5, shift_b);
    T(total_b, b_cur, 4);
    __builtin_amdgcn_sched_barrier(0);
    // slot 20
    PV(A, 1, 0, wa);
    __builtin_amdgcn_sched_barrier(0);
    KR(4);
    E(b_cur, 6, shift_b);
    T(total_b, b_cur, 5);
    W(wb, b_cur, 2);
    __builtin_amdgcn_sched_barrier(0);
    // slot 21
    PV(A, 1, 1, wa);
    __builtin_amdgcn_sched_barrier(0);
    KR(5);
    E(b_cur, 7, shift_b);
    T(total_b, b_cur, 6);
    __builtin_amdgcn_sched_barrier(0);
    // slot 22
    PV(A, 1, 2, wa);
    __builtin_amdgcn_sched_barrier(0);
    KR(6);
    T(total_b, b_cur, 7);
    W(wb, b_cur, 3);
    E(b_cur, 8, shift_b);
    __builtin_amdgcn_sched_barrier(0);
    // slot 23
    PV(A, 1, 3, wa);
    __builtin_amdgcn_sched_barrier(0);
    KR(7);
    E(b_cur, 9, shift_b);
    T(total_b, b_cur, 8);
    __builtin_amdgcn_sched_barrier(0);
    // slot 24
    PV(B, 0, 0, wb);
    __builtin_amdgcn_sched_barrier(0);
    E(b_cur, 10, shift_b);
    T(total_b, b_cur, 9);
    E(b_cur, 11, shift_b);
    __builtin_amdgcn_sched_barrier(0);
    // slot 25
    PV(B, 0, 1, wb);
    __builtin_amdgcn_sched_barrier(0);
    T(total_b, b_cur, 10);
    W(wb, b_cur, 4);
    E(b_cur, 12, shift_b);
    T(total_b, b_cur, 11);
    W(wb, b_cur, 5);
    __builtin_amdgcn_sched_barrier(0);
    // slot 26
    PV(B, 0, 2, wb);
    __builtin_amdgcn_sched_barrier(0);
    E(b_cur, 13, shift_b);
    T(total_b, b_cur, 12);
    E(b_cur, 14, shift_b);
    __builtin_amdgcn_sched_barrier(0);
    // slot 27
    PV(B, 0, 3, wb);
    __builtin_amdgcn_sched_barrier(0);
    T(total_b, b_cur, 13);
    E(b_cur, 15, shift_b);
    T(total_b, b_cur, 14);
    W(wb, b_cur, 6);
    __builtin_amdgcn_sched_barrier(0);
    // slot 28
    W(wb, b_cur, 7);
    PV(B, 1, 0, wb);
    __builtin_amdgcn_sched_barrier(0);
    ROW_MAXIMA_0;
    __builtin_amdgcn_sched_barrier(0);
    // slot 29
    PV(B, 1, 1, wb);
    __builtin_amdgcn_sched_barrier(0);
    ROW_MAXIMA_1;
    __builtin_amdgcn_sched_barrier(0);
    // slot 30
    PV(B, 1, 2, wb);
    __builtin_amdgcn_sched_barrier(0);
    ROW_MAXIMA_2;
    __builtin_amdgcn_sched_barrier(0);
    // slot 31
    PV(B, 1, 3, wb);
    __builtin_amdgcn_sched_barrier(0);
    LAG_TEST;
    T(total_b, b_cur, 15);
    __builtin_amdgcn_sched_barrier(0);
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

// One 256-row query tile of (batch, head) pair `bh`.
template <bool CAUSAL, class Half>
SINGE_DEVICE void fmha_prefill_pair_tile(const PrefillArgs& a, unsigned char* lds, unsigned int bh, unsigned int query_tile) {
    constexpr unsigned int kLoadRows = 4u * kPairWaves;  // key rows one load instruction of every wave brings in
    const unsigned int tid = threadIdx.x, lane = tid & 63;
    const unsigned int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const unsigned int column = lane & 31, hi = lane >> 5;
    const unsigned int group = a.heads / a.kv_heads;
    const unsigned int batch = bh / a.heads, head = bh % a.heads, kv_head = head / group;
    const unsigned int key_len = a.key_len;  // a multiple of 64 (the host's gate)

    const unsigned int first_row = query_tile * kPairRows + wave * 64u;  // of this wave: tile A, then tile B 32 rows on
    const unsigned int query_a = first_row + column, query_b = query_a + 32u;
    const bool valid_a = query_a < a.query_len, valid_b = query_b < a.query_len;

    const uint16_t* q_base = a.query + batch * a.query_batch_stride + head * a.query_head_stride;
    const unsigned char* const k_bytes = reinterpret_cast<const unsigned char*>(a.key + batch * a.key_batch_stride + kv_head * a.key_head_stride);
    const unsigned char* const v_bytes = reinterpret_cast<const unsigned char*>(a.value + batch * a.value_batch_stride + kv_head * a.value_head_stride);

    // Q^T of both tiles as MFMA B operands: lane (column = query, hi) holds dims 16s + 8hi .. +8 for s = 0..7 (rows
    // past query_len read row 0 and are not stored).  The scale's sign is not folded into Q^T here: the host sends
    // only positive scales.
    const float factor = a.scale_log2e;
    const Half half{};
    u32x4_t qa[kSteps], qb[kSteps];
    {
        const uint16_t* row_a = q_base + static_cast<size_t>(valid_a ? query_a : 0) * a.query_sequence_stride + 8 * hi;
        const uint16_t* row_b = q_base + static_cast<size_t>(valid_b ? query_b : 0) * a.query_sequence_stride + 8 * hi;
#pragma unroll
        for (int s = 0; s < kSteps; ++s) qa[s] = load_to_accumulation(row_a + 16 * s);
#pragma unroll
        for (int s = 0; s < kSteps; ++s) qb[s] = load_to_accumulation(row_b + 16 * s);
    }
    const uint4 no_query[kSteps] = {};  // the masked path's folding functions take a Q^T they do not read

    // Tiles of keys the workgroup visits, and how many of them this wave folds without a mask: under the causal mask
    // the tile that holds the wave's own rows (index first_row / 64) is its last and takes the masked path.
    unsigned int key_end = key_len;
    if (CAUSAL) {
        const unsigned int reach = query_tile * kPairRows + kPairRows;
        key_end = key_end < reach ? key_end : reach;
    }
    const unsigned int tiles = key_end / kKeyTile;
    unsigned int interior_tiles = tiles;
    if (CAUSAL) interior_tiles = first_row / kKeyTile < tiles ? first_row / kKeyTile : tiles;
    const bool has_diagonal = CAUSAL && interior_tiles < tiles;

    // The loads of a tile, as in fmha_prefill.hip: instruction i of wave w fills rows 16 i + 4 w .. + 3 of the stage.
    const unsigned int key_stride_bytes = static_cast<unsigned int>(a.key_sequence_stride) * 2u;
    const unsigned int value_stride_bytes = static_cast<unsigned int>(a.value_sequence_stride) * 2u;
    const unsigned int load_row = 4u * wave + (lane >> 4), position = lane & 15u;
    const unsigned int key_lane = load_row * key_stride_bytes + (position ^ (load_row & 15u)) * 16u;
    const unsigned int value_lane = load_row * value_stride_bytes + (position ^ (4u * (load_row & 3u))) * 16u;
    auto load_part = [&](const unsigned char* base, unsigned int stride_bytes, unsigned int lane_offset, unsigned int i,
                         unsigned char* stage) __attribute__((always_inline)) {
        unsigned int offset = lane_offset + kLoadRows * i * stride_bytes;
        asm volatile("" : "+v"(offset));  // a 32-bit offset next to the load keeps its scalar-base form
        __builtin_amdgcn_global_load_lds(reinterpret_cast<const unsigned int*>(base + offset),
                                         (lds_words_t)(stage + (kLoadRows * i + 4u * wave) * kRowBytes), 16, 0, 0);
    };
    auto tile_base = [&](const unsigned char* rows, unsigned int stride_bytes, unsigned int tile) __attribute__((always_inline)) {
        const unsigned char* base = rows + static_cast<size_t>(tile * kKeyTile) * stride_bytes;
        asm("" : "+s"(base));
        return base;
    };
    auto load_tile = [&](unsigned int tile, unsigned int stage) __attribute__((always_inline)) {
        const unsigned char* keys = tile_base(k_bytes, key_stride_bytes, tile);
        const unsigned char* values = tile_base(v_bytes, value_stride_bytes, tile);
#pragma unroll
        for (unsigned int i = 0; i < 4; ++i) load_part(keys, key_stride_bytes, key_lane, i, lds + stage * kTileBytes);
#pragma unroll
        for (unsigned int i = 0; i < 4; ++i) load_part(values, value_stride_bytes, value_lane, i, lds + kPairValueBase + stage * kTileBytes);
    };

    RowState A, B;
    reset(A);
    reset(B);
    const ReadOffsets offsets = read_offsets(lane);

    for (unsigned int early = 0; early < kPairAhead && early < tiles; ++early) load_tile(early, early);
    loads_landed();
    accumulation_loads_landed();
    __syncthreads();

    f32x16_t a_even, b_even, a_odd, b_odd;  // raw scores of the block folded next (even / odd blocks of a tile)
    unsigned int tile = 0, stage = 0;       // stage = tile % 4
    if (interior_tiles > 0 || has_diagonal) {
        score_block_pair(half, a_even, qa, lds, offsets);
        score_block_pair(half, b_even, qb, lds, offsets);
    }
    if (interior_tiles > 0) {
        uint4 operand[kSteps];
        read_key_operands(operand, lds + kBlockBytes, offsets);
        // (the V stages start at an offset the compiler must not know, or it folds it into the reads' immediates,
        // which it then overflows)
        unsigned int value_base = kPairValueBase;
        asm volatile("" : "+s"(value_base));
        const unsigned char* value_origin = lds + value_base;
        float shift_a = begin_block(A, a_even, hi, factor, false, [](unsigned int) { return false; });
        float shift_b = begin_block(B, b_even, hi, factor, false, [](unsigned int) { return false; });
        auto settle = [&](float largest_a, float largest_b) __attribute__((always_inline)) {
            move_reference(A, largest_a);
            move_reference(B, largest_b);
            shift_a = A.reference == -INFINITY ? 0.0f : -A.reference;
            shift_b = B.reference == -INFINITY ? 0.0f : -B.reference;
        };
        // One tile, its stage a constant: the loop below is written out once per stage, so that every LDS address of
        // the schedule is a register that never changes plus an immediate offset.
        auto fold_tile = [&](auto stage_constant) __attribute__((always_inline)) {
            constexpr unsigned int kStage = decltype(stage_constant)::value;
            constexpr unsigned int kNextStage = (kStage + 1) % kPairStages, kSpareStage = (kStage + kPairAhead) % kPairStages;
            const unsigned char* __restrict__ next_keys = lds + kNextStage * kTileBytes;
            constexpr unsigned int values = kStage * kTileBytes;
            unsigned char* __restrict__ key_dest = lds + kSpareStage * kTileBytes;
            unsigned char* __restrict__ value_dest = lds + kPairValueBase + kSpareStage * kTileBytes;
            // The tile three ahead, or (nobody reads it) the last one again when there is none.
            const unsigned int wanted = tile + kPairAhead < tiles ? tile + kPairAhead : tiles - 1;
            const unsigned char* key_rows = tile_base(k_bytes, key_stride_bytes, wanted);
            const unsigned char* value_rows = tile_base(v_bytes, value_stride_bytes, wanted);
            auto issue_keys = [&](unsigned int i) __attribute__((always_inline)) { load_part(key_rows, key_stride_bytes, key_lane, i, key_dest); };
            auto issue_values = [&](unsigned int i) __attribute__((always_inline)) { load_part(value_rows, value_stride_bytes, value_lane, i, value_dest); };
            float largest_a, largest_b;
            bool lagging = fold_pair_block(half, A, B, a_even, b_even, a_odd, b_odd, factor, shift_a, shift_b, largest_a, largest_b, qa, qb, operand,
                                  next_keys, value_origin, values, offsets, issue_keys);
            if (lagging) settle(largest_a, largest_b);
            lagging = fold_pair_block(half, A, B, a_odd, b_odd, a_even, b_even, factor, shift_a, shift_b, largest_a, largest_b, qa, qb, operand,
                                   next_keys + kBlockBytes, value_origin, values + kBlockBytes, offsets, issue_values);
            // (past the wave's last unmasked tile the scores just computed are the diagonal tile's, which the masked path
            // takes as they are, or nobody's)
            if (lagging && tile + 1 < interior_tiles) settle(largest_a, largest_b);
            older_loads_landed();  // the next tile's; the eight of this iteration have another tile's time
            __syncthreads();
        };
        while (tile < interior_tiles) {
            fold_tile(std::integral_constant<unsigned int, 0>{});
            stage = 1;
            if (++tile >= interior_tiles) break;
            fold_tile(std::integral_constant<unsigned int, 1>{});
            stage = 2;
            if (++tile >= interior_tiles) break;
            fold_tile(std::integral_constant<unsigned int, 2>{});
            stage = 3;
            if (++tile >= interior_tiles) break;
            fold_tile(std::integral_constant<unsigned int, 3>{});
            stage = 0;
            ++tile;
        }
    }
    // The tile on the diagonal: block 2 t holds the keys of tile A's rows (B sees all of it), block 2 t + 1 those of
    // tile B's rows (A sees none of it).
    if (has_diagonal) {
        const unsigned int next_stage = (stage + 1) % kPairStages, spare_stage = (stage + kPairAhead) % kPairStages;
        const unsigned char* keys = lds + stage * kTileBytes;
        const unsigned char* values = lds + kPairValueBase + stage * kTileBytes;
        const bool loading = tile + kPairAhead < tiles;
        if (loading) load_tile(tile + kPairAhead, spare_stage);
        const unsigned int key0 = tile * kKeyTile;
        const float edge_a = begin_block(A, a_even, hi, factor, true, [&](unsigned int key_in_block) { return key0 + key_in_block > query_a; });
        finish_block<false>(half, A, a_even, factor, edge_a, values, offsets, a_even, no_query, values);
        const float whole_b = begin_block(B, b_even, hi, factor, false, [](unsigned int) { return false; });
        finish_block<false>(half, B, b_even, factor, whole_b, values, offsets, b_even, no_query, values);
        score_block_pair(half, b_odd, qb, keys + kBlockBytes, offsets);
        const float edge_b = begin_block(B, b_odd, hi, factor, true, [&](unsigned int key_in_block) { return key0 + 32u + key_in_block > query_b; });
        finish_block<false>(half, B, b_odd, factor, edge_b, values + kBlockBytes, offsets, b_odd, no_query, values);
        if (loading) older_loads_landed(); else loads_landed();
        __syncthreads();
        stage = next_stage;
        ++tile;
    }
    // The tiles the waves with later rows still work on: this wave's share of their loads, and their barriers.
    for (; tile < tiles; ++tile) {
        const unsigned int next_stage = (stage + 1) % kPairStages, spare_stage = (stage + kPairAhead) % kPairStages;
        const bool loading = tile + kPairAhead < tiles;
        if (loading) load_tile(tile + kPairAhead, spare_stage);
        if (loading) older_loads_landed(); else loads_landed();
        __syncthreads();
        stage = next_stage;
    }

    // Normalise and store.  Lane (query, hi) holds dims 32db + 8(r / 4) + 4hi + (r % 4).
    auto store = [&](RowState& state, unsigned int query, bool valid) __attribute__((always_inline)) {
        const float sum = swap32_sum(state.running_sum);
        const float inverse = sum > 0.0f ? 1.0f / sum : 0.0f;
        if (!valid) return;
        uint16_t* row = a.out + batch * a.output_batch_stride + static_cast<size_t>(query) * a.output_sequence_stride + head * a.output_head_stride;
#pragma unroll
        for (int db = 0; db < kDimBlocks; ++db)
#pragma unroll
            for (int quad = 0; quad < 4; ++quad) {
                uint2 packed;
                packed.x = pack_pair(half, state.out[db][4 * quad + 0] * inverse, state.out[db][4 * quad + 1] * inverse);
                packed.y = pack_pair(half, state.out[db][4 * quad + 2] * inverse, state.out[db][4 * quad + 3] * inverse);
                *reinterpret_cast<uint2*>(row + 32 * db + 8 * quad + 4 * hi) = packed;
            }
        if (a.lse != nullptr && hi == 0)
            a.lse[(static_cast<size_t>(batch) * a.heads + head) * a.query_len + query] = sum > 0.0f ? (state.reference + fast_log2(sum)) * kLn2 : -INFINITY;
    };
    store(A, query_a, valid_a);
    store(B, query_b, valid_b);
    // (the next tile of the pair starts by loading into stages this one may still be reading)
    __syncthreads();
}

// Workgroup id -> (batch * heads + head, pair of query tiles), as in fmha_prefill.hip; query_tiles counts 256-row tiles.
template <bool CAUSAL, class Half>
SINGE_DEVICE void fmha_prefill_pair_body(const PrefillArgs& a, unsigned char* lds) {
    const unsigned int xcd = blockIdx.x & 7u, within = blockIdx.x >> 3;
    const unsigned int pairs = (a.query_tiles + 1u) / 2u;
    const unsigned int bh = (within / pairs) * 8u + xcd;
    if (bh >= a.batch * a.heads) return;
    const unsigned int light = within % pairs, heavy = a.query_tiles - 1u - light;
    // (one copy of the tile's code for both tiles: written out per stage it is long, and two copies of it would not fit
    // the instruction cache)
#pragma nounroll
    for (unsigned int which = 0; which < (light != heavy ? 2u : 1u); ++which)
        fmha_prefill_pair_tile<CAUSAL, Half>(a, lds, bh, which == 0 ? heavy : light);
}

}  // namespace

#define SINGE_FMHA_PREFILL_PAIR_KERNEL(NAME, CAUSAL, HALF)                                             \
    extern "C" __global__ __launch_bounds__(64 * kPairWaves, 1) void NAME(PrefillArgs args) {          \
        __shared__ __attribute__((aligned(1024))) unsigned char prefill_lds[kPairLdsBytes];            \
        fmha_prefill_pair_body<CAUSAL, prefill::HALF>(args, prefill_lds);                              \
    }

SINGE_FMHA_PREFILL_PAIR_KERNEL(singe_fmha_prefill_pair_bf16_d128_causal, true, Bf16)
SINGE_FMHA_PREFILL_PAIR_KERNEL(singe_fmha_prefill_pair_bf16_d128_full, false, Bf16)
SINGE_FMHA_PREFILL_PAIR_KERNEL(singe_fmha_prefill_pair_f16_d128_causal, true, F16)
SINGE_FMHA_PREFILL_PAIR_KERNEL(singe_fmha_prefill_pair_f16_d128_full, false, F16)
