// Dense flash-attention prefill for long rows, bf16 or f16, head_dim 128 (or 96, 64: -DSINGE_HEAD_DIM=), no options: the same arithmetic and
// register layouts as fmha_prefill.hip (S^T = K . Q^T, per-lane softmax, O^T += V^T . P^T; prefill_core.hip.h), with
// the work laid out the other way round.  There, two waves share a SIMD and each folds keys into 32 query rows;
// what one wave leaves idle the other uses.  Here ONE wave owns a SIMD (up to 512 registers) and folds every key
// block into TWO tiles of 32 query rows, A and B:
//   * each K and V^T operand read from LDS feeds two matrix instructions instead of one, a workgroup's 64-key
//     tile serves 256 query rows instead of 128, and there is one barrier per 64 matrix instructions;
//   * the order of a wave's instructions is the schedule: a block is 32 matrix instructions (8 score products of
//     the NEXT block for A, 8 for B, 8 value products of this block for A, 8 for B) and the vector work of the block
//     (exponentials, sums, packing, the next block's row maxima, LDS operand reads, the tile's loads) is dealt out
//     evenly over the 32 slots between them, each piece before the matrix instruction that needs it
//     (fold_pair_block; prefill_pair_deal.py).  A lone wave issues every instruction itself, the matrix ones
//     included, so the block's instruction count bounds the loop (about 360 issue cycles of four clocks for 256 of
//     matrix work), and on operands that switch many bits the clock the device holds comes before that;
//   * the score accumulators must be in ordinary vector registers (the vector unit reads them) while O^T and Q^T
//     live in the accumulation registers; the compiler gives every matrix instruction of such a kernel an
//     accumulation-register destination, so the score products are written as assembly with the register classes
//     spelled out.  The distance between a score product and the first vector instruction that reads its result is
//     part of the schedule (at least four slots, some thirty instructions), since the compiler does not see a
//     matrix instruction there.
// query/out [batch, query_len, heads, 128], key/value [batch, key_len, kv_heads, 128] with element strides from
// FmhaPrefillConfig; lse [batch, heads, query_len], natural log.  The host sends calls here that fill the chip with
// 256-row tiles; everything else stays on fmha_prefill.hip.  A last tile of fewer than 64 keys re-reads the last key
// in its spare rows and takes the masked path, like the tile on the causal diagonal.
//
// Grid: one workgroup of four waves per (batch, head, pair of 256-row query tiles), tile i from the end and tile i
// from the start; ids laid out as in fmha_prefill.hip.  LDS: four stages of K and four of V (128 KiB), each tile
// loaded three tiles ahead, straight from global memory, and waited for a tile after it was asked for (a wave alone
// on its SIMD has nobody to cover a wait for fresh loads); one barrier per tile.  Behind the stages, 8 KiB a wave that
// its output rows go through on their way out (32 KiB: all of a compute unit's 160 KiB are in use).
#include "kernel_args.h"
#include "prefill_pair.hip.h"

namespace {

using namespace prefill;

// One 256-row query tile of (batch, head) pair `bh`.  RAGGED: key_len is not a multiple of 64 (a build of its own:
// the extra code of the last tile costs the other build instruction-cache room, 4 % under the causal mask).
template <bool CAUSAL, bool RAGGED, class Half>
SINGE_DEVICE void fmha_prefill_pair_tile(const PrefillArgs& a, unsigned char* lds, unsigned int bh, unsigned int query_tile) {
    constexpr unsigned int kLoadRows = 4u * kPairWaves;  // key rows one load instruction of every wave brings in
    const unsigned int tid = threadIdx.x, lane = tid & 63;
    const unsigned int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const unsigned int column = lane & 31, hi = lane >> 5;
    const unsigned int group = a.heads / a.kv_heads;
    const unsigned int batch = bh / a.heads, head = bh % a.heads, kv_head = head / group;
    // Keys that take part: all of them (at least one, and a multiple of 64 unless RAGGED: the host's gate), or (RAGGED) the
    // batch entry's own count, which may be none (singe/src/backend/cpu/normalization/attention.rs:191-276, key_lengths).
    unsigned int key_len = a.key_len;
    if (RAGGED && a.key_lengths != nullptr) {
        const int own = a.key_lengths[batch];
        const unsigned int bound = own > 0 ? static_cast<unsigned int>(own) : 0u;
        key_len = bound < key_len ? bound : key_len;
    }
    key_len = __builtin_amdgcn_readfirstlane(key_len);

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

    // Tiles of keys the workgroup visits, how many of them this wave folds without a mask, and whether one more takes
    // the masked path: under the causal mask the tile that holds the wave's own rows (index first_row / 64), and with or
    // without it a last tile that is not whole.
    unsigned int key_end = key_len;
    if (CAUSAL) {
        const unsigned int reach = query_tile * kPairRows + kPairRows;
        key_end = key_end < reach ? key_end : reach;
    }
    const unsigned int tiles = (key_end + kKeyTile - 1) / kKeyTile, whole_tiles = key_end / kKeyTile;
    unsigned int interior_tiles = whole_tiles;
    if (CAUSAL) interior_tiles = first_row / kKeyTile < whole_tiles ? first_row / kKeyTile : whole_tiles;
    const bool has_masked_tile = interior_tiles < tiles;  // (its index is interior_tiles)
    // The last key tile A and tile B see anything of, as the first key past it.
    const unsigned int reach_a = CAUSAL && first_row + 32u < key_len ? first_row + 32u : key_len;
    const unsigned int reach_b = CAUSAL && first_row + 64u < key_len ? first_row + 64u : key_len;

    // The loads of a tile, as in fmha_prefill.hip: instruction i of wave w fills rows 16 i + 4 w .. + 3 of the stage.
    const unsigned int key_stride_bytes = static_cast<unsigned int>(a.key_sequence_stride) * 2u;
    const unsigned int value_stride_bytes = static_cast<unsigned int>(a.value_sequence_stride) * 2u;
    const unsigned int load_row = 4u * wave + (lane >> 4), position = lane & 15u;
    const unsigned int key_chunk = fetched_chunk(position ^ (load_row & 15u)) * 16u;
    const unsigned int value_chunk = fetched_chunk(position ^ (4u * (load_row & 3u))) * 16u;
    const unsigned int key_lane = load_row * key_stride_bytes + key_chunk, value_lane = load_row * value_stride_bytes + value_chunk;
    // The lane's offsets into a tile, one a load.  A last tile that is not whole has offsets of its own: its rows past
    // the last key re-read that key (they are masked; what lies behind the last key is not this call's to read).  Both
    // sets are worked out here, so that a load in the loop picks one with a single select and no branch.
    unsigned int key_offsets[4], value_offsets[4], key_tail_offsets[4], value_tail_offsets[4];
#pragma unroll
    for (unsigned int i = 0; i < 4; ++i) {
        const unsigned int row = kLoadRows * i + load_row, last = (key_len - 1u) % kKeyTile;
        const unsigned int kept = row < last ? row : last;
        key_offsets[i] = key_lane + kLoadRows * i * key_stride_bytes;
        value_offsets[i] = value_lane + kLoadRows * i * value_stride_bytes;
        key_tail_offsets[i] = kept * key_stride_bytes + key_chunk;
        value_tail_offsets[i] = kept * value_stride_bytes + value_chunk;
    }
    auto load_part = [&](const unsigned char* base, const unsigned int (&whole)[4], const unsigned int (&tailed)[4], bool tail, unsigned int i,
                         unsigned char* stage) __attribute__((always_inline)) {
        unsigned int offset = tail ? tailed[i] : whole[i];
        asm volatile("" : "+v"(offset));  // a 32-bit offset next to the load keeps its scalar-base form
        __builtin_amdgcn_global_load_lds(reinterpret_cast<const unsigned int*>(base + offset),
                                         (lds_words_t)(stage + (kLoadRows * i + 4u * wave) * kRowBytes), 16, 0, 0);
    };
    auto is_tail = [&](unsigned int tile) __attribute__((always_inline)) { return RAGGED && tile * kKeyTile + kKeyTile > key_len; };
    auto tile_base = [&](const unsigned char* rows, unsigned int stride_bytes, unsigned int tile) __attribute__((always_inline)) {
        const unsigned char* base = rows + static_cast<size_t>(tile * kKeyTile) * stride_bytes;
        asm("" : "+s"(base));
        return base;
    };
    auto load_tile = [&](unsigned int tile, unsigned int stage) __attribute__((always_inline)) {
        const unsigned char* keys = tile_base(k_bytes, key_stride_bytes, tile);
        const unsigned char* values = tile_base(v_bytes, value_stride_bytes, tile);
        const bool tail = is_tail(tile);
#pragma unroll
        for (unsigned int i = 0; i < 4; ++i) load_part(keys, key_offsets, key_tail_offsets, tail, i, lds + stage * kTileBytes);
#pragma unroll
        for (unsigned int i = 0; i < 4; ++i)
            load_part(values, value_offsets, value_tail_offsets, tail, i, lds + kPairValueBase + stage * kTileBytes);
    };

    RowState A, B;
    reset(A);
    reset(B);
    if (a.sinks != nullptr) {
        // The head's sink: a score that is always there and weighs no value.  A row starts with it as its reference point
        // and a sum of one (held by one of the row's two lanes), as in fmha_prefill.hip.
        const uint16_t bits = a.sinks[head];
        float sink;
        if constexpr (std::is_same_v<Half, F16>) sink = static_cast<float>(__builtin_bit_cast(_Float16, bits));
        else sink = __builtin_bit_cast(float, static_cast<unsigned int>(bits) << 16);
        A.reference = B.reference = sink * kLog2e;
        A.running_sum = B.running_sum = hi == 0 && A.reference != -INFINITY ? 1.0f : 0.0f;
    }
    const ReadOffsets offsets = read_offsets(lane);

    for (unsigned int early = 0; early < kPairAhead && early < tiles; ++early) load_tile(early, early);
    loads_landed();
    accumulation_loads_landed();
    __syncthreads();

    f32x16_t a_even, b_even, a_odd, b_odd;  // raw scores of the block folded next (even / odd blocks of a tile)
    unsigned int tile = 0, stage = 0;       // stage = tile % 4
    if (interior_tiles > 0 || has_masked_tile) {
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
            const bool tail = is_tail(wanted);
            auto issue_keys = [&](unsigned int i) __attribute__((always_inline)) {
                load_part(key_rows, key_offsets, key_tail_offsets, tail, i, key_dest);
            };
            auto issue_values = [&](unsigned int i) __attribute__((always_inline)) {
                load_part(value_rows, value_offsets, value_tail_offsets, tail, i, value_dest);
            };
            float largest_a, largest_b;
            bool lagging = fold_pair_block(half, A, B, a_even, b_even, a_odd, b_odd, factor, shift_a, shift_b, largest_a, largest_b, qa, qb, operand,
                                  next_keys, value_origin, values, offsets, issue_keys);
            if (lagging) settle(largest_a, largest_b);
            lagging = fold_pair_block(half, A, B, a_odd, b_odd, a_even, b_even, factor, shift_a, shift_b, largest_a, largest_b, qa, qb, operand,
                                   next_keys + kBlockBytes, value_origin, values + kBlockBytes, offsets, issue_values);
            // (past the wave's last unmasked tile the scores just computed are the masked tile's, which that path
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
    // The tile a mask touches: on the causal diagonal block 2 t holds the keys of tile A's rows (B sees all of it) and
    // block 2 t + 1 those of tile B's rows (A sees none of it); a last tile that is not whole ends where the keys end.
    if (has_masked_tile) {
        const unsigned int next_stage = (stage + 1) % kPairStages, spare_stage = (stage + kPairAhead) % kPairStages;
        const unsigned char* keys = lds + stage * kTileBytes;
        const unsigned char* values = lds + kPairValueBase + stage * kTileBytes;
        const bool loading = tile + kPairAhead < tiles;
        if (loading) load_tile(tile + kPairAhead, spare_stage);
        const unsigned int key0 = tile * kKeyTile;
        if constexpr (!RAGGED) {
            // (the causal diagonal: A masked, B whole; then B masked)
            const float edge_a = begin_block(A, a_even, hi, factor, true, [&](unsigned int key_in_block) { return key0 + key_in_block > query_a; });
            finish_block<false>(half, A, a_even, factor, edge_a, values, offsets, a_even, no_query, values);
            const float whole_b = begin_block(B, b_even, hi, factor, false, [](unsigned int) { return false; });
            finish_block<false>(half, B, b_even, factor, whole_b, values, offsets, b_even, no_query, values);
            score_block_pair(half, b_odd, qb, keys + kBlockBytes, offsets);
            const float edge_b = begin_block(B, b_odd, hi, factor, true, [&](unsigned int key_in_block) { return key0 + 32u + key_in_block > query_b; });
            finish_block<false>(half, B, b_odd, factor, edge_b, values + kBlockBytes, offsets, b_odd, no_query, values);
        } else {
            // One block of one row tile, masked by the last key each row sees (its own under the causal mask, and never
            // past the last key there is).
            auto fold = [&](RowState& state, f32x16_t& s, unsigned int query, unsigned int first_key, const unsigned char* block_values) __attribute__((always_inline)) {
                const unsigned int last_seen = CAUSAL && query < key_len - 1u ? query : key_len - 1u;
                const float shift = begin_block(state, s, hi, factor, true, [&](unsigned int key_in_block) { return first_key + key_in_block > last_seen; });
                finish_block<false>(half, state, s, factor, shift, block_values, offsets, s, no_query, block_values);
            };
            if (key0 < reach_a) fold(A, a_even, query_a, key0, values);
            if (key0 < reach_b) fold(B, b_even, query_b, key0, values);
            if (key0 + 32u < reach_a) {
                score_block_pair(half, a_odd, qa, keys + kBlockBytes, offsets);
                fold(A, a_odd, query_a, key0 + 32u, values + kBlockBytes);
            }
            if (key0 + 32u < reach_b) {
                score_block_pair(half, b_odd, qb, keys + kBlockBytes, offsets);
                fold(B, b_odd, query_b, key0 + 32u, values + kBlockBytes);
            }
        }
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

    // Normalise and store (store_rows).  (Storing as soon as a wave's own last tile is folded, up to three tiles before
    // the workgroup's under the causal mask, was measured and is no faster: the wave then waits for its stores with the
    // next tile's loads, and the others wait for it at the barrier.)
    {
        uint16_t* const rows = a.out + batch * a.output_batch_stride + head * a.output_head_stride;
        unsigned char* const staging = lds + kPairLdsBytes + wave * (32u * kRowBytes);
        auto store = [&](RowState& state, unsigned int tile_first, unsigned int query, bool valid) __attribute__((always_inline)) {
            const float sum = swap32_sum(state.running_sum);
            const float inverse = sum > 0.0f ? 1.0f / sum : 0.0f;
            if (a.lse != nullptr && hi == 0 && valid)
                a.lse[(static_cast<size_t>(batch) * a.heads + head) * a.query_len + query] = sum > 0.0f ? (state.reference + fast_log2(sum)) * kLn2 : -INFINITY;
            store_rows(half, state, inverse, lane, staging, [&](unsigned int r) __attribute__((always_inline)) {
                const unsigned int row = tile_first + r;
                return row < a.query_len ? rows + static_cast<size_t>(row) * a.output_sequence_stride : nullptr;
            });
        };
        store(A, first_row, query_a, valid_a);
        store(B, first_row + 32u, query_b, valid_b);
    }
    // (the next tile of the pair starts by loading into stages this one may still be reading)
    __syncthreads();
}

// Workgroup id -> (batch * heads + head, pair of query tiles), as in fmha_prefill.hip; query_tiles counts 256-row tiles.
template <bool CAUSAL, bool RAGGED, class Half>
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
        fmha_prefill_pair_tile<CAUSAL, RAGGED, Half>(a, lds, bh, which == 0 ? heavy : light);
}

}  // namespace

#define SINGE_FMHA_PREFILL_PAIR_KERNEL(NAME, CAUSAL, RAGGED, HALF)                                     \
    extern "C" __global__ __launch_bounds__(64 * kPairWaves, 1) void NAME(PrefillArgs args) {          \
        __shared__ __attribute__((aligned(1024))) unsigned char prefill_lds[kPairLdsBytes + kPairStoreBytes]; \
        fmha_prefill_pair_body<CAUSAL, RAGGED, prefill::HALF>(args, prefill_lds);                      \
    }

#define SINGE_PAIR_NAME(TYPE, FORM) SINGE_PAIR_JOIN(singe_fmha_prefill, pair, TYPE, SINGE_PAIR_DIM, FORM)
SINGE_FMHA_PREFILL_PAIR_KERNEL(SINGE_PAIR_NAME(bf16, causal), true, false, Bf16)
SINGE_FMHA_PREFILL_PAIR_KERNEL(SINGE_PAIR_NAME(bf16, full), false, false, Bf16)
SINGE_FMHA_PREFILL_PAIR_KERNEL(SINGE_PAIR_NAME(f16, causal), true, false, F16)
SINGE_FMHA_PREFILL_PAIR_KERNEL(SINGE_PAIR_NAME(f16, full), false, false, F16)
SINGE_FMHA_PREFILL_PAIR_KERNEL(SINGE_PAIR_NAME(bf16, causal_ragged), true, true, Bf16)
SINGE_FMHA_PREFILL_PAIR_KERNEL(SINGE_PAIR_NAME(bf16, full_ragged), false, true, Bf16)
SINGE_FMHA_PREFILL_PAIR_KERNEL(SINGE_PAIR_NAME(f16, causal_ragged), true, true, F16)
SINGE_FMHA_PREFILL_PAIR_KERNEL(SINGE_PAIR_NAME(f16, full_ragged), false, true, F16)
