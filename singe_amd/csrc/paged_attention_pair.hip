// Attention of ragged queries over a paged KV cache in FlashInfer form (see paged_attention.hip for the op, its
// layouts and its paging checks), for the calls that are prefill-shaped and plain: bf16 or f16, head_dim 128 (or 96, 64: -DSINGE_HEAD_DIM=), a page
// size that is a power of two of at least 16 keys, no cap, no window, no key splits; with or without the fused query
// rotation of rotary_paged_attention (query_rotation.hip.h).  The loop is
// the dense two-tile one (fmha_prefill_pair.hip, prefill_pair.hip.h): a wave alone on its SIMD folds every 32-key
// block into two tiles of 32 packed rows, so a workgroup owns 256 packed rows of one (sequence, kv head) (row r =
// token r / groups, head r % groups) and a key tile staged in LDS serves all of them.
//
// What differs from the dense kernel is where rows and keys come from.  Keys: a tile's sixteen-key groups sit in one
// page each; their ids are fetched four tiles ahead (by vector loads, lane i the id of group i, so that they are
// counted with the tile loads and not with the LDS reads), checked a tile later, and the tile is loaded three
// ahead from the checked ids (an id outside the cache is reported and replaced by page 0).  Rows: a row's key
// position is max(keys - queries + token, 0) (bottom-right causal alignment), so under the mask a wave's 64 rows (eight
// tokens at eight heads a kv head) end within a few keys of each other: the tiles every row of the wave sees whole run
// through the scheduled loop, the one or two behind them through the 32-row kernel's masked block functions, tile A
// and tile B each with its own positions.
#include "kernel_args.h"
#include "paged_locate.hip.h"
#include "paging.hip.h"
#include "prefill_pair.hip.h"
#include "query_rotation.hip.h"

namespace {

using namespace prefill;

template <int FORM, bool ROTATE, class Half>
SINGE_DEVICE void paged_attention_pair_body(const PagedAttentionArgs& a, unsigned char* lds) {
    static_assert(FORM == kCsrI32 || FORM == kCsrI64, "the FlashInfer form");
    const unsigned int tid = threadIdx.x, lane = tid & 63;
    const unsigned int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const unsigned int column = lane & 31, hi = lane >> 5;
    const unsigned int groups = a.heads / a.kv_heads;

    unsigned int unit, row_tile, split;
    if (!locate<FORM, kPairRows>(a, unit, row_tile, split)) return;
    unit = __builtin_amdgcn_readfirstlane(unit);
    row_tile = __builtin_amdgcn_readfirstlane(row_tile);
    const unsigned int sequence = unit / a.kv_heads, kv_head = unit % a.kv_heads;
    const unsigned int first_row = row_tile * kPairRows;

    const SequenceSpan span = load_span<FORM>(sequence, a.query_offsets, a.page_offsets, a.last_page_lengths, a.query_lengths,
                                              a.tokens, a.page_table, a.page_size);
    if (!span.valid) {
        if (tid == 0) report_index_error(a.status);
        return;
    }
    const long long query_start = span.query_start, page_start = span.page_start;
    const unsigned int queries = __builtin_amdgcn_readfirstlane(span.queries), keys = __builtin_amdgcn_readfirstlane(span.keys);
    const unsigned int packed = queries * groups;
    if (first_row >= packed) return;

    // Key position of packed row r: max(keys - queries + r / groups, 0).
    auto position_of = [&](unsigned int row) __attribute__((always_inline)) {
        const long long position = static_cast<long long>(keys) - static_cast<long long>(queries) + row / groups;
        return position < 0 ? 0u : static_cast<unsigned int>(position);
    };
    const bool causal = a.causal != 0;
    // The wave's two tiles: A holds rows wave_first_row .. + 31, B the 32 after them.
    const unsigned int wave_first_row = first_row + wave * 64u;
    struct Tile {
        unsigned int row, token, head, position;  // of this lane's row (the workgroup's first row when it has none)
        bool valid;
        unsigned int high;  // position of the tile's last row: the last key any of its rows sees under the mask
        bool live;          // the tile has rows
    };
    auto tile_of = [&](unsigned int first) __attribute__((always_inline)) {
        Tile t;
        t.row = first + column;
        t.valid = t.row < packed;
        const unsigned int row = t.valid ? t.row : first_row;
        t.token = row / groups;
        t.head = row % groups;
        t.position = position_of(row);
        t.live = first < packed;
        const unsigned int last = first + 31u < packed ? first + 31u : packed - 1u;
        t.high = __builtin_amdgcn_readfirstlane(position_of(t.live ? last : first_row));
        return t;
    };
    const Tile ta = tile_of(wave_first_row), tb = tile_of(wave_first_row + 32u);
    const bool wave_live = ta.live;
    const unsigned int wave_low = __builtin_amdgcn_readfirstlane(position_of(wave_live ? wave_first_row : first_row));
    const unsigned int wave_high = tb.live ? tb.high : ta.high;

    // Tiles of keys the workgroup visits; the ones this wave folds (under the mask, up to the last key its last row
    // sees); and the ones of those that no mask touches for any of its rows.
    const unsigned int group_last_row = first_row + kPairRows - 1 < packed ? first_row + kPairRows - 1 : packed - 1u;
    unsigned int key_end = keys;
    if (causal) {
        const unsigned int reach = position_of(group_last_row) + 1u;
        key_end = key_end < reach ? key_end : reach;
    }
    const unsigned int tiles = __builtin_amdgcn_readfirstlane((key_end + kKeyTile - 1) / kKeyTile);
    unsigned int wave_tiles = 0, interior_tiles = 0;
    if (wave_live) {
        wave_tiles = tiles;
        interior_tiles = keys / kKeyTile;  // tiles t with 64 t + 64 <= keys
        if (causal) {
            const unsigned int seen = wave_high / kKeyTile + 1u, unmasked = (wave_low + 1u) / kKeyTile;  // 64 t + 63 <= wave_low
            wave_tiles = wave_tiles < seen ? wave_tiles : seen;
            interior_tiles = interior_tiles < unmasked ? interior_tiles : unmasked;
        }
        interior_tiles = interior_tiles < wave_tiles ? interior_tiles : wave_tiles;
    }
    wave_tiles = __builtin_amdgcn_readfirstlane(wave_tiles);
    interior_tiles = __builtin_amdgcn_readfirstlane(interior_tiles);

    // Q^T of both tiles, straight into accumulation registers (the host sends positive scales only).
    const float factor = a.scale_log2e;
    const Half half{};
    u32x4_t qa[kSteps], qb[kSteps];
    {
        auto row_of = [&](const Tile& t) __attribute__((always_inline)) {
            return a.query_rows + ((static_cast<size_t>(query_start) + t.token) * a.heads + kv_head * groups + t.head) * kHeadDim + 8 * hi;
        };
        if constexpr (ROTATE) {
            // The query arrives before its norm and rotation (query_rotation.hip.h): loaded into vector registers, turned
            // there, parked in LDS (the fourth stage, which nobody loads before the first tile is folded: 8 KiB a wave,
            // a lane's eight chunks 1 KiB apart) and read back straight into the accumulation registers, so that Q^T is
            // born in that class here too.
            unsigned char* const parked = lds + (wave < 2 ? 0 : kPairValueBase) + kPairAhead * kTileBytes + (wave & 1u) * 8192u + lane * 16u;
            auto turned = [&](const Tile& t, u32x4_t (&q)[kSteps]) __attribute__((always_inline)) {
                const uint16_t* row = row_of(t);
                uint4 bits[kSteps];
#pragma unroll
                for (int s = 0; s < kSteps; ++s) {
                    bits[s] = *reinterpret_cast<const uint4*>(row + 16 * s);
                    if (!t.valid) bits[s] = make_uint4(0, 0, 0, 0);
                }
                rotate_query(half, bits, a, static_cast<size_t>(query_start) + t.token, t.valid, hi);
#pragma unroll
                for (int s = 0; s < kSteps; ++s) *reinterpret_cast<uint4*>(parked + 1024 * s) = bits[s];
#pragma unroll
                for (int s = 0; s < kSteps; ++s) q[s] = lds_to_accumulation(lds_address(parked + 1024 * s));
            };
            turned(ta, qa);
            turned(tb, qb);
        } else {
            const uint16_t* row_a = row_of(ta);
            const uint16_t* row_b = row_of(tb);
#pragma unroll
            for (int s = 0; s < kSteps; ++s) qa[s] = load_to_accumulation(row_a + 16 * s);
#pragma unroll
            for (int s = 0; s < kSteps; ++s) qb[s] = load_to_accumulation(row_b + 16 * s);
        }
    }
    const uint4 no_query[kSteps] = {};  // the masked path's folding functions take a Q^T they do not read

    // Loads: instruction i of wave w fills rows 16 i + 4 w .. + 3 of a stage; the sixteen keys of instruction i's
    // group sit in one page (paged_attention.hip, GROUPED).
    const unsigned int load_row = 4u * wave + (lane >> 4), chunk_position = lane & 15u;
    const unsigned int key_chunk = fetched_chunk(chunk_position ^ (load_row & 15u)) * 16u;
    const unsigned int value_chunk = fetched_chunk(chunk_position ^ (4u * (load_row & 3u))) * 16u;
    const unsigned int page_bytes = a.page_size * a.kv_heads * kGlobalRowBytes;  // (the host sends pages below 4 GiB)
    const unsigned int head_bytes = kv_head * kGlobalRowBytes, slot_bytes = a.kv_heads * kGlobalRowBytes;
    const unsigned char* const key_bytes = reinterpret_cast<const unsigned char*>(a.key_cache);
    const unsigned char* const value_bytes = reinterpret_cast<const unsigned char*>(a.value_cache);
    const unsigned int last_group = tiles > 0 ? (keys - 1u) & ~15u : 0u;  // first key of the sixteen that hold the last one
    const unsigned int key_lane = load_row * slot_bytes + key_chunk, value_lane = load_row * slot_bytes + value_chunk;
    // Where the four groups of a tile start in either cache, in bytes.
    struct Pages {
        unsigned long long start[4];
    };
    // First key of the group instruction i of a tile reads: its own, or the last group of the sequence.
    auto group_of = [&](unsigned int tile, unsigned int i) __attribute__((always_inline)) {
        const unsigned int first = tile * kKeyTile + 16u * i;
        return first < last_group ? first : last_group;
    };
    // The id of one group of a tile a lane (group lane % 4), on its way until the loads before it have landed, and
    // where the group starts in its page.  All of this is lane work: the wave is alone on its SIMD, where a scalar
    // instruction costs the issue slot a vector one does, and four lanes do four groups at once.
    struct Lookup {
        RawPage<FORM> raw;
        unsigned int in_page;
    };
    auto lookup = [&](unsigned int tile) __attribute__((always_inline)) {
        const unsigned int group = group_of(tile, lane & 3u);
        Lookup l;
        l.raw = read_raw_page<FORM>(a.pages, static_cast<size_t>(page_start) + (group >> a.page_shift));
        l.in_page = (group & (a.page_size - 1u)) * slot_bytes + head_bytes;
        return l;
    };
    auto check = [&](const Lookup& l, Pages& pages) __attribute__((always_inline)) {
        const unsigned long long mine = static_cast<unsigned long long>(l.raw);  // negative ids wrap above any cache
        const bool valid = mine < static_cast<unsigned long long>(a.cache_pages);
        // (an id outside the cache is reported and replaced by page 0: what that holds is not used by a caller that checks)
        if (__builtin_amdgcn_ballot_w64(!valid) != 0) report_index_error(a.status);
        const unsigned long long start = static_cast<unsigned long long>(valid ? static_cast<unsigned int>(mine) : 0u) * page_bytes + l.in_page;
        const unsigned int low = static_cast<unsigned int>(start), upper = static_cast<unsigned int>(start >> 32);
#pragma unroll
        for (unsigned int i = 0; i < 4; ++i)
            pages.start[i] = (static_cast<unsigned long long>(static_cast<unsigned int>(__builtin_amdgcn_readlane(upper, i))) << 32) |
                             static_cast<unsigned int>(__builtin_amdgcn_readlane(low, i));
    };
    // The lane's offsets inside a group, for K and for V; the tile that holds the sequence's last key has offsets of its
    // own, one a group: rows past that key re-read it, and a group that lies past it is the last group again.  Both are
    // worked out here, so that a load in the loop picks one with a single select and no branch.
    unsigned int key_tail_lane[4], value_tail_lane[4];
#pragma unroll
    for (unsigned int i = 0; i < 4; ++i) {
        const unsigned int last = tiles > 0 ? keys - 1u - group_of((keys - 1u) / kKeyTile, i) : 0u;
        const unsigned int kept = load_row < last ? load_row : last;
        key_tail_lane[i] = kept * slot_bytes + key_chunk;
        value_tail_lane[i] = kept * slot_bytes + value_chunk;
    }
    // `tail`: the tile holds the sequence's last key and is not whole.
    auto load_part = [&](const unsigned char* cache, unsigned int lane_offset, const unsigned int (&tail_lane)[4], bool tail, const Pages& pages,
                         unsigned int i, unsigned char* stage) __attribute__((always_inline)) {
        const unsigned char* base = cache + pages.start[i];
        unsigned int offset = tail ? tail_lane[i] : lane_offset;
        asm("" : "+s"(base));
        asm volatile("" : "+v"(offset));
        __builtin_amdgcn_global_load_lds(reinterpret_cast<const unsigned int*>(base + offset),
                                         (lds_words_t)(stage + (16u * i + 4u * wave) * kRowBytes), 16, 0, 0);
    };
    auto is_tail = [&](unsigned int tile) __attribute__((always_inline)) { return tile * kKeyTile + kKeyTile > keys; };
    auto load_tile = [&](unsigned int tile, const Pages& pages, unsigned int stage) __attribute__((always_inline)) {
#pragma unroll
        for (unsigned int i = 0; i < 4; ++i) load_part(key_bytes, key_lane, key_tail_lane, is_tail(tile), pages, i, lds + stage * kTileBytes);
#pragma unroll
        for (unsigned int i = 0; i < 4; ++i)
            load_part(value_bytes, value_lane, value_tail_lane, is_tail(tile), pages, i, lds + kPairValueBase + stage * kTileBytes);
    };

    RowState A, B;
    reset(A);
    reset(B);
    const ReadOffsets offsets = read_offsets(lane);

    // The first three tiles, and the ids of the fourth: `ready` holds the checked ids of the tile that is loaded next
    // (tile + 3 at the top of tile's iteration; past the last tile, the last tile's again).
    Pages ready = {};
    {
        Lookup raw[kPairAhead + 1];
#pragma unroll
        for (unsigned int early = 0; early <= kPairAhead; ++early)
            if (tiles > 0) raw[early] = lookup(early < tiles ? early : tiles - 1u);
#pragma unroll
        for (unsigned int early = 0; early <= kPairAhead; ++early) {
            if (tiles > 0) check(raw[early], ready);
            if (early < kPairAhead && early < tiles) load_tile(early, ready, early);
        }
    }
    loads_landed();
    accumulation_loads_landed();
    __syncthreads();

    // Folds block `block` of one row tile on the masked path.
    auto fold_masked = [&](RowState& state, f32x16_t& s, const Tile& t, unsigned int block, const unsigned char* values) __attribute__((always_inline)) {
        const unsigned int key0 = block * 32u;
        const float shift = begin_block(state, s, hi, factor, true, [&](unsigned int key_in_block) {
            const unsigned int key = key0 + key_in_block;
            return key >= keys || (causal && key > t.position);
        });
        finish_block<false>(half, state, s, factor, shift, values, offsets, s, no_query, values);
    };
    // Whether a row tile has anything in a block.
    auto needs = [&](const Tile& t, unsigned int block) __attribute__((always_inline)) {
        return t.live && block * 32u < key_end && (!causal || block * 32u <= t.high);
    };

    f32x16_t a_even, b_even, a_odd, b_odd;  // raw scores of the block folded next (even / odd blocks of a tile)
    unsigned int tile = 0, stage = 0;       // stage = tile % 4
    if (wave_tiles > 0) {
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
        auto fold_tile = [&](auto stage_constant) __attribute__((always_inline)) {
            constexpr unsigned int kStage = decltype(stage_constant)::value;
            constexpr unsigned int kNextStage = (kStage + 1) % kPairStages, kSpareStage = (kStage + kPairAhead) % kPairStages;
            const unsigned char* __restrict__ next_keys = lds + kNextStage * kTileBytes;
            constexpr unsigned int values = kStage * kTileBytes;
            unsigned char* __restrict__ key_dest = lds + kSpareStage * kTileBytes;
            unsigned char* __restrict__ value_dest = lds + kPairValueBase + kSpareStage * kTileBytes;
            // The tile three ahead (`ready` holds its ids), or (nobody reads it) the last one again; the ids of the one
            // after it go out first and are back with the loads that the end of the iteration waits for.
            const unsigned int wanted = tile + kPairAhead < tiles ? tile + kPairAhead : tiles - 1u;
            const unsigned int after = tile + kPairAhead + 1u < tiles ? tile + kPairAhead + 1u : tiles - 1u;
            const Lookup fresh = lookup(after);
            const bool tail = is_tail(wanted);
            const Pages now = ready;
            auto issue_keys = [&](unsigned int i) __attribute__((always_inline)) { load_part(key_bytes, key_lane, key_tail_lane, tail, now, i, key_dest); };
            auto issue_values = [&](unsigned int i) __attribute__((always_inline)) { load_part(value_bytes, value_lane, value_tail_lane, tail, now, i, value_dest); };
            float largest_a, largest_b;
            bool lagging = fold_pair_block(half, A, B, a_even, b_even, a_odd, b_odd, factor, shift_a, shift_b, largest_a, largest_b, qa, qb, operand,
                                           next_keys, value_origin, values, offsets, issue_keys);
            if (lagging) settle(largest_a, largest_b);
            lagging = fold_pair_block(half, A, B, a_odd, b_odd, a_even, b_even, factor, shift_a, shift_b, largest_a, largest_b, qa, qb, operand,
                                      next_keys + kBlockBytes, value_origin, values + kBlockBytes, offsets, issue_values);
            // (past the wave's last unmasked tile the scores just computed are a masked tile's, which that path takes
            // as they are, or nobody's)
            if (lagging && tile + 1 < interior_tiles) settle(largest_a, largest_b);
            older_loads_landed();  // the next tile's and the ids; the eight of this iteration have another tile's time
            check(fresh, ready);
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
    // A tile outside the scheduled loop: this wave's share of the loads three tiles on and of the ids four tiles on,
    // whatever `work` the wave has in the tile, the wait and the barrier.
    auto plain_tile = [&](auto&& work) __attribute__((always_inline)) {
        const unsigned int next_stage = (stage + 1) % kPairStages, spare_stage = (stage + kPairAhead) % kPairStages;
        const bool loading = tile + kPairAhead < tiles, looking = tile + kPairAhead + 1u < tiles;
        Lookup fresh = {};
        if (looking) fresh = lookup(tile + kPairAhead + 1u);
        if (loading) load_tile(tile + kPairAhead, ready, spare_stage);
        work(next_stage);
        if (loading) older_loads_landed(); else loads_landed();
        if (looking) check(fresh, ready);
        __syncthreads();
        stage = next_stage;
        ++tile;
    };
    // The tiles a mask touches for some row of the wave (under the causal mask: the last one or two it folds; without
    // it: a last tile that is not whole), each row tile with its own positions.
    while (tile < wave_tiles) {
        plain_tile([&](unsigned int next_stage) __attribute__((always_inline)) {
            const unsigned char* keys_here = lds + stage * kTileBytes;
            const unsigned char* values = lds + kPairValueBase + stage * kTileBytes;
            const unsigned int block = 2u * tile;
            if (needs(ta, block)) fold_masked(A, a_even, ta, block, values);
            if (needs(tb, block)) fold_masked(B, b_even, tb, block, values);
            if (needs(ta, block + 1u)) {
                score_block_pair(half, a_odd, qa, keys_here + kBlockBytes, offsets);
                fold_masked(A, a_odd, ta, block + 1u, values + kBlockBytes);
            }
            if (needs(tb, block + 1u)) {
                score_block_pair(half, b_odd, qb, keys_here + kBlockBytes, offsets);
                fold_masked(B, b_odd, tb, block + 1u, values + kBlockBytes);
            }
            if (tile + 1u < wave_tiles) {
                score_block_pair(half, a_even, qa, lds + next_stage * kTileBytes, offsets);
                score_block_pair(half, b_even, qb, lds + next_stage * kTileBytes, offsets);
            }
        });
    }
    // The tiles the waves with later rows still work on.
    while (tile < tiles) plain_tile([](unsigned int) {});

    // Normalise and store; a row that sees no key stays zero and has a log-sum-exp of -inf.
    auto store = [&](RowState& state, const Tile& t) __attribute__((always_inline)) {
        const float sum = swap32_sum(state.running_sum);
        const float inverse = sum > 0.0f ? 1.0f / sum : 0.0f;
        if (!t.valid) return;
        const size_t flat = (static_cast<size_t>(query_start) + t.token) * a.heads + kv_head * groups + t.head;
        uint16_t* row = a.output + flat * kHeadDim;
#pragma unroll
        for (int db = 0; db < kDimBlocks; ++db)
#pragma unroll
            for (int quad = 0; quad < 4; ++quad) {
                if (32 * db + 8 * quad >= kHeadDim) continue;  // (the last dim block of an odd multiple of 16 is half)
                uint2 packed_bits;
                packed_bits.x = pack_pair(half, state.out[db][4 * quad + 0] * inverse, state.out[db][4 * quad + 1] * inverse);
                packed_bits.y = pack_pair(half, state.out[db][4 * quad + 2] * inverse, state.out[db][4 * quad + 3] * inverse);
                *reinterpret_cast<uint2*>(row + 32 * db + 8 * quad + 4 * hi) = packed_bits;
            }
        if (a.lse != nullptr && hi == 0) a.lse[flat] = sum > 0.0f ? state.reference + fast_log2(sum) : -INFINITY;
    };
    store(A, ta);
    store(B, tb);
}

}  // namespace

#define SINGE_PAGED_ATTENTION_PAIR_KERNEL(NAME, FORM, ROTATE, HALF)                                 \
    extern "C" __global__ __launch_bounds__(64 * prefill::kPairWaves, 1) void NAME(PagedAttentionArgs args) { \
        __shared__ __attribute__((aligned(1024))) unsigned char paged_lds[prefill::kPairLdsBytes];  \
        paged_attention_pair_body<FORM, ROTATE, prefill::HALF>(args, paged_lds);                    \
    }

#define SINGE_PAIR_NAME(OP, TYPE, FORM) SINGE_PAIR_JOIN(singe_##OP, pair, TYPE, SINGE_PAIR_DIM, FORM)
SINGE_PAGED_ATTENTION_PAIR_KERNEL(SINGE_PAIR_NAME(paged_attention, bf16, i32), kCsrI32, false, Bf16)
SINGE_PAGED_ATTENTION_PAIR_KERNEL(SINGE_PAIR_NAME(paged_attention, bf16, i64), kCsrI64, false, Bf16)
SINGE_PAGED_ATTENTION_PAIR_KERNEL(SINGE_PAIR_NAME(paged_attention, f16, i32), kCsrI32, false, F16)
SINGE_PAGED_ATTENTION_PAIR_KERNEL(SINGE_PAIR_NAME(paged_attention, f16, i64), kCsrI64, false, F16)
// (with the query's norm and rotation fused in)
SINGE_PAGED_ATTENTION_PAIR_KERNEL(SINGE_PAIR_NAME(rotary_paged_attention, bf16, i32), kCsrI32, true, Bf16)
SINGE_PAGED_ATTENTION_PAIR_KERNEL(SINGE_PAIR_NAME(rotary_paged_attention, bf16, i64), kCsrI64, true, Bf16)
SINGE_PAGED_ATTENTION_PAIR_KERNEL(SINGE_PAIR_NAME(rotary_paged_attention, f16, i32), kCsrI32, true, F16)
SINGE_PAGED_ATTENTION_PAIR_KERNEL(SINGE_PAIR_NAME(rotary_paged_attention, f16, i64), kCsrI64, true, F16)
