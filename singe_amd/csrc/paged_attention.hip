// Attention of ragged queries over a paged KV cache in FlashInfer form: decode, prefill and chunked
// prefill in one kernel, the gfx950 counterpart of singe_paged_attention
// (singe/src/backend/cuda/kernel_plan/source/paged_attention.rs:544-868) and of the CPU attend_paged
// (singe/src/backend/cpu/normalization/attention.rs:424-538).
//
// query_rows/output [tokens, heads, D] bf16 or f16; caches [pages, page_size, kv_heads, D], D = 128 or 64 (one build
// each); sequence b
// holds queries query_offsets[b] .. query_offsets[b+1] and the keys of pages
// pages[page_offsets[b] .. page_offsets[b+1]], all full but the last, which holds last_page_lengths[b];
// lse [tokens, heads] f32, base two, -inf for a row that sees no key.  Queries are a sequence's LAST
// tokens: query q sits at key position max(keys - queries + q, 0) (bottom-right causal alignment, with
// the CPU path's saturating subtraction: attention.rs:482-488).
//
// A workgroup owns 128 packed rows of one (sequence, kv head): the query heads that share the kv head,
// a token's heads consecutive (row r = token r / groups, head r % groups), so a key tile is staged once
// for the whole group.  The grid covers every sequence's longest possible run of rows; workgroups past
// their sequence's rows return at once.  Keys are gathered row by row, each lane placing its own row in its
// page, straight from the cache into the same permuted LDS tiles as the dense kernel (three K stages, two V
// stages, page ids looked up three tiles ahead) and folded by the same block-pipelined core
// (prefill_blocks.hip.h).
//
// The same body also serves paged_kv_prefill_attention of the singe-kernel surface
// (singe-kernel/src/cpu/attention.rs:1248-1341): paging as a [batch, stride] block table with per-sequence
// query offsets, query lengths and key lengths, queries aligned with a sequence's FIRST keys, and a
// natural-log lse that is -1e20 for a row without keys.
//
// Paging values come from device memory, so they are checked here: a value that would address outside
// the queries, the page table or the cache sets the status word to 1 (first writer wins; the word may
// be null) and nothing is read through it (paged_attention.rs:41-54, 210-262, 739-755).
#include "kernel_args.h"
#include "paging.hip.h"
#include "paged_locate.hip.h"
#include "prefill_blocks.hip.h"
#include "query_rotation.hip.h"

namespace {

using namespace prefill;

// Whether the interior tiles read their K operands a block ahead (prefill_blocks.hip.h).
constexpr bool kPagedOperandsAhead = true;

template <bool SOFTCAP, int FORM, bool GROUPED, bool ROTATE, class Half>
SINGE_DEVICE void paged_attention_body(const PagedAttentionArgs& a, unsigned char* lds) {
    const unsigned int tid = threadIdx.x, lane = tid & 63;
    const unsigned int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // uniform, and known to be
    const unsigned int column = lane & 31, hi = lane >> 5;
    const unsigned int groups = a.heads / a.kv_heads;

    unsigned int unit, row_tile, split;
    if (!locate<FORM, kQueryTile>(a, unit, row_tile, split)) return;
    unit = __builtin_amdgcn_readfirstlane(unit);  // the same in every lane, and known to the compiler to be
    row_tile = __builtin_amdgcn_readfirstlane(row_tile);
    const unsigned int sequence = unit / a.kv_heads, kv_head = unit % a.kv_heads;
    const unsigned int first_row = row_tile * kQueryTile;

    // The sequence's paging values, refused when any would address outside the kernel's buffers.
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

    // Key position of packed row r: max(keys - queries + r / groups, 0); the block-table form aligns
    // queries with the FIRST keys instead (key > query index is hidden, cpu/attention.rs:1283).
    auto position_of = [&](unsigned int row) __attribute__((always_inline)) {
        if constexpr (FORM == kTable) return row / groups;
        const long long position = static_cast<long long>(keys) - static_cast<long long>(queries) + row / groups;
        return position < 0 ? 0u : static_cast<unsigned int>(position);
    };
    const unsigned int my_row = first_row + wave * 32u + column;
    const bool row_valid = my_row < packed;
    const unsigned int my_token = (row_valid ? my_row : first_row) / groups, my_head = (row_valid ? my_row : first_row) % groups;
    const unsigned int my_position = position_of(row_valid ? my_row : first_row);
    const bool causal = a.causal != 0, windowed = a.window >= 0;
    // (positions fit 31 bits: a wider window hides nothing, and is held there so that key + window cannot wrap)
    const unsigned int window = !windowed ? 0u : a.window > 0x7fffffffll ? 0x7fffffffu : static_cast<unsigned int>(a.window);

    // Rows of this wave: none when the wave starts past the sequence's rows.
    const unsigned int wave_first_row = first_row + wave * 32u;
    const bool wave_live = wave_first_row < packed;
    const unsigned int wave_last_row = wave_live ? (wave_first_row + 31u < packed ? wave_first_row + 31u : packed - 1u) : first_row;
    const unsigned int wave_low = __builtin_amdgcn_readfirstlane(position_of(wave_live ? wave_first_row : first_row));
    const unsigned int wave_high = __builtin_amdgcn_readfirstlane(position_of(wave_last_row));

    // Keys this workgroup must visit, in tiles; and the blocks of them this wave folds: under the causal
    // mask a block wholly after the wave's last position contributes nothing.
    const unsigned int group_last_row = first_row + kQueryTile - 1 < packed ? first_row + kQueryTile - 1 : packed - 1u;
    unsigned int key_end = keys;
    if (causal) {
        const unsigned int reach = position_of(group_last_row) + 1u;
        key_end = key_end < reach ? key_end : reach;
    }
    unsigned int first_tile = 0;
    if (windowed) {
        const unsigned int low = position_of(first_row) + 1u;  // keys below low - window are hidden from every row
        first_tile = low > window ? (low - window) / kKeyTile : 0u;
    }
    unsigned int tiles = (key_end + kKeyTile - 1) / kKeyTile;
    if (a.splits > 1) {
        // This workgroup's share of the tiles; a share may be empty.
        const unsigned int share = tiles > first_tile ? (tiles - first_tile + a.splits - 1) / a.splits : 0u;
        first_tile += split * share;
        tiles = tiles < first_tile + share ? tiles : first_tile + share;
    }
    first_tile = __builtin_amdgcn_readfirstlane(first_tile);
    tiles = __builtin_amdgcn_readfirstlane(tiles);
    unsigned int wave_blocks = 0;
    if (wave_live) {
        wave_blocks = (key_end + 31u) / 32u;
        if (causal) {
            const unsigned int seen = wave_high / 32u + 1u;
            wave_blocks = wave_blocks < seen ? wave_blocks : seen;
        }
        wave_blocks = wave_blocks < 2u * tiles ? wave_blocks : 2u * tiles;  // a share ends with its last tile
    }
    wave_blocks = __builtin_amdgcn_readfirstlane(wave_blocks);

    // Q^T as the MFMA B operand; a negative scale moves into Q (see fmha_prefill.hip).
    const float factor = SOFTCAP ? 1.0f : fabsf(a.scale_log2e);
    const unsigned int flip = (SOFTCAP ? a.softcap_scale : a.scale_log2e) < 0.0f ? 0x80008000u : 0u;
    const Half half{};
    uint4 q[kSteps];
    {
        const uint16_t* row = a.query_rows + ((static_cast<size_t>(query_start) + my_token) * a.heads + kv_head * groups + my_head) * kHeadDim + 8 * hi;
        uint4 bits[kSteps];
#pragma unroll
        for (int s = 0; s < kSteps; ++s) {
            bits[s] = *reinterpret_cast<const uint4*>(row + 16 * s);
            if (!row_valid) bits[s] = make_uint4(0, 0, 0, 0);
        }
        if constexpr (ROTATE) {
            rotate_query(half, bits, a, static_cast<size_t>(query_start) + my_token, row_valid, hi);
        }
#pragma unroll
        for (int s = 0; s < kSteps; ++s) {
            bits[s].x ^= flip; bits[s].y ^= flip; bits[s].z ^= flip; bits[s].w ^= flip;
            q[s] = bits[s];
        }
    }

    // A tile load is 1024 16-byte chunks per operand: instruction i of wave w fills rows 16 i + 4 w .. + 3,
    // lane l the chunk position l % 16 of row 16 i + 4 w + l / 16, fetched from the chunk the row's
    // permutation puts there (prefill_blocks.hip.h).  A row is key (tile, row) of the sequence, found in page
    // pages[page_start + key / page_size] at slot key % page_size; rows past the sequence's last key re-read
    // that key and are masked, so nothing the sequence does not own reaches LDS.  Page ids are looked up
    // three tiles ahead and checked then; K is loaded two tiles ahead and V one, from the same ids.
    //
    // GROUPED (the page size is 16, 32, 64, ... keys): the sixteen rows of an instruction, keys 16-aligned, sit
    // in one page, so its id is one scalar load, checked and multiplied on the scalar unit, and a load's
    // address is a scalar base (page, the group's first slot, the kv head) plus a per-lane offset that never
    // changes (row in the group, chunk): no vector arithmetic per load.  Otherwise each lane looks up and
    // places its own row.
    const unsigned int load_row = 4u * wave + (lane >> 4), chunk_position = lane & 15u;
    const unsigned int key_chunk = (chunk_position ^ (load_row & 15u)) * 16u, value_chunk = (chunk_position ^ (4u * (load_row & 3u))) * 16u;
    // At head_dim 64 a cache row has eight chunks: the lanes whose LDS position holds one of the other eight fetch nothing.
    const bool key_lane_live = key_chunk < kGlobalRowBytes, value_lane_live = value_chunk < kGlobalRowBytes;
    const size_t page_bytes = static_cast<size_t>(a.page_size) * a.kv_heads * kGlobalRowBytes;
    const unsigned int head_bytes = kv_head * kGlobalRowBytes, slot_bytes = a.kv_heads * kGlobalRowBytes;
    const unsigned char* const key_bytes = reinterpret_cast<const unsigned char*>(a.key_cache);
    const unsigned char* const value_bytes = reinterpret_cast<const unsigned char*>(a.value_cache);
    const bool shifted = a.page_shift >= 0;
    const unsigned int last_group = (keys - 1u) & ~15u;  // first key of the sixteen that hold the last one (keys > 0 where used)
    struct Pages {
        unsigned int id[4];
    };
    struct RawPages {
        RawPage<FORM> value[4];  // as loaded: nothing computes on them until they are checked, a tile later
    };
    auto key_of = [&](unsigned int tile, unsigned int i) __attribute__((always_inline)) {
        const unsigned int key = tile * kKeyTile + 16u * i + load_row;
        return key < keys ? key : keys - 1u;
    };
    // GROUPED: first key of the group instruction i of a tile reads: its own, or the last group of the sequence.
    auto group_of = [&](unsigned int tile, unsigned int i) __attribute__((always_inline)) {
        const unsigned int first = tile * kKeyTile + 16u * i;
        return first < last_group ? first : last_group;
    };
    auto lookup = [&](unsigned int tile, RawPages& raw) __attribute__((always_inline)) {
#pragma unroll
        for (unsigned int i = 0; i < 4; ++i) {
            if constexpr (GROUPED) {
                raw.value[i] = read_raw_page_uniform<FORM>(a.pages, static_cast<size_t>(page_start) + (group_of(tile, i) >> a.page_shift));
            } else {
                const unsigned int key = key_of(tile, i);
                const unsigned int entry = shifted ? key >> a.page_shift : key / a.page_size;
                raw.value[i] = read_raw_page<FORM>(a.pages, static_cast<size_t>(page_start) + entry);
            }
        }
    };
    auto check = [&](const RawPages& raw, Pages& pages) __attribute__((always_inline)) {
#pragma unroll
        for (unsigned int i = 0; i < 4; ++i) {
            const unsigned long long page = static_cast<unsigned long long>(raw.value[i]);  // negative ids wrap above any cache
            const bool valid = page < static_cast<unsigned long long>(a.cache_pages);
            if (!valid) report_index_error(a.status);
            pages.id[i] = valid ? static_cast<unsigned int>(page) : kNoPage;
        }
    };
    const unsigned int key_lane = load_row * slot_bytes + key_chunk, value_lane = load_row * slot_bytes + value_chunk;
    auto load = [&](const unsigned char* cache, unsigned int chunk, unsigned int lane_offset, bool lane_live, unsigned int tile,
                    const Pages& pages, unsigned char* stage) __attribute__((always_inline)) {
        // (only the load itself is predicated, so that the scalar address arithmetic stays outside the branch)
        const bool fetch = kGlobalRowBytes == kRowBytes || lane_live;
#pragma unroll
        for (unsigned int i = 0; i < 4; ++i) {
            if constexpr (GROUPED) {
                if (pages.id[i] == kNoPage) continue;
                const unsigned int first = tile * kKeyTile + 16u * i, group = group_of(tile, i);
                const unsigned char* base = cache + (pages.id[i] * page_bytes + ((group & (a.page_size - 1u)) * slot_bytes + head_bytes));
                unsigned int offset = lane_offset;
                if (first + 15u >= keys) {  // the group holds the sequence's last key, or lies past it
                    const unsigned int last = keys - 1u - group;
                    offset = (load_row < last ? load_row : last) * slot_bytes + chunk;
                }
                // Both pinned as they are (a scalar, a 32-bit per-lane offset) so the load keeps its
                // scalar-base form (see fmha_prefill.hip).
                asm("" : "+s"(base));
                asm volatile("" : "+v"(offset));
                if (fetch)
                    __builtin_amdgcn_global_load_lds(reinterpret_cast<const unsigned int*>(base + offset),
                                                     (lds_words_t)(stage + (16u * i + 4u * wave) * kRowBytes), 16, 0, 0);
            } else {
                const unsigned int key = key_of(tile, i);
                const unsigned int slot = shifted ? key & (a.page_size - 1u) : key % a.page_size;
                const size_t offset = pages.id[i] * page_bytes + (slot * slot_bytes + head_bytes + chunk);
                if (pages.id[i] != kNoPage && fetch)
                    __builtin_amdgcn_global_load_lds(reinterpret_cast<const unsigned int*>(cache + offset),
                                                     (lds_words_t)(stage + (16u * i + 4u * wave) * kRowBytes), 16, 0, 0);
            }
        }
    };
    auto load_keys = [&](unsigned int tile, const Pages& pages, unsigned char* stage) __attribute__((always_inline)) {
        load(key_bytes, key_chunk, key_lane, key_lane_live, tile, pages, stage);
    };
    auto load_values = [&](unsigned int tile, const Pages& pages, unsigned char* stage) __attribute__((always_inline)) {
        load(value_bytes, value_chunk, value_lane, value_lane_live, tile, pages, stage);
    };

    RowState state;
    reset(state);
    const ReadOffsets offsets = read_offsets(lane);

    Pages behind = {}, ahead = {};  // of tile + 1 and tile + 2 at the top of tile's iteration
    RawPages fresh = {};            // of tile + 3, on their way during it
    if (first_tile < tiles) {
        RawPages raw_first = {}, raw_behind = {}, raw_ahead = {};
        lookup(first_tile, raw_first);
        if (first_tile + 1 < tiles) lookup(first_tile + 1, raw_behind);
        if (first_tile + 2 < tiles) lookup(first_tile + 2, raw_ahead);
        Pages first;
        check(raw_first, first);
        if (first_tile + 1 < tiles) check(raw_behind, behind);
        if (first_tile + 2 < tiles) check(raw_ahead, ahead);
        load_keys(first_tile, first, lds);
        load_values(first_tile, first, lds + kValueBase);
        if (first_tile + 1 < tiles) load_keys(first_tile + 1, behind, lds + kTileBytes);
    }
    loads_landed();
    __syncthreads();

    // Folds block `block` (scores in `s`, values at `values`) with the masks' edges applied.
    auto fold = [&](unsigned int block, f32x16_t& s, const unsigned char* values) __attribute__((always_inline)) {
        const unsigned int key0 = block * 32u;
        if constexpr (SOFTCAP) {
            // Scores become cap * tanh(score * scale / cap) before the softmax
            // (singe/src/backend/cuda/kernel_plan/source/tensor_core.rs:49-54).
            const float cap_scale = fabsf(a.softcap_scale);
#pragma unroll
            for (int r = 0; r < 16; ++r) s[r] = fast_tanh(s[r] * cap_scale) * a.softcap_log2e;
        }
        const bool edge = (causal && key0 + 31u > wave_low) || key0 + 32u > keys || windowed;
        const float shift = begin_block(state, s, hi, factor, edge, [&](unsigned int key_in_block) {
            const unsigned int key = key0 + key_in_block;
            return key >= keys || (causal && key > my_position) || (windowed && key + window <= my_position);
        });
        finish_block<false>(half, state, s, factor, shift, values, offsets, s, q, values);
    };

    // One block ahead, as in the dense kernel: `scores` holds those of the block that is folded next.
    f32x16_t scores;
    if (2u * first_tile < wave_blocks) score_block(half, scores, q, lds, offsets);
    unsigned int key_stage = 0, value_stage = 0;
    // Names the stages a tile's iteration works on and loads into.
    auto enter = [&]() __attribute__((always_inline)) {
        const unsigned int next_key_stage = key_stage + 1 == kKeyStages ? 0 : key_stage + 1;
        const unsigned int spare_key_stage = next_key_stage + 1 == kKeyStages ? 0 : next_key_stage + 1;
        TileStages stages;
        stages.keys = lds + key_stage * kTileBytes;
        stages.next_keys = lds + next_key_stage * kTileBytes;
        stages.values = lds + kValueBase + value_stage * kTileBytes;
        stages.key_dest = lds + spare_key_stage * kTileBytes;
        stages.value_dest = lds + kValueBase + (value_stage ^ 1u) * kTileBytes;
        key_stage = next_key_stage;
        value_stage ^= 1u;
        return stages;
    };
    unsigned int tile = first_tile;
    // Starts a tile's loads: ids for tile + 3, K of tile + 2, V of tile + 1.
    auto issue = [&](unsigned char* key_dest, unsigned char* value_dest) __attribute__((always_inline)) {
        if (tile + 3 < tiles) lookup(tile + 3, fresh);
        if (tile + 2 < tiles) load_keys(tile + 2, ahead, key_dest);
        if (tile + 1 < tiles) load_values(tile + 1, behind, value_dest);
    };
    // Ends a tile's iteration: the ids looked up at its start have had the whole tile to arrive, this wave's
    // loads have landed, and the barrier hands the stages on.
    auto leave = [&]() __attribute__((always_inline)) {
        __builtin_amdgcn_sched_barrier(0);
        behind = ahead;
        if (tile + 3 < tiles) check(fresh, ahead);
        loads_landed();
        __syncthreads();
    };

    // Tiles no mask touches for this wave, with another block to come after them: straight-line code.  With a
    // window, the tiles that reach back past the window of the wave's last row come before them and take the
    // masked path; a cap is applied to each block's scores before they are folded.
    unsigned int interior_end = wave_blocks > 2 ? (wave_blocks - 1) / 2 : 0;  // tiles t with 2 t + 2 < wave_blocks
    if (causal) {
        const unsigned int unmasked = (wave_low + 1) / kKeyTile;  // tiles t with 64 t + 63 <= wave_low
        interior_end = interior_end < unmasked ? interior_end : unmasked;
    }
    {
        const unsigned int whole = keys / kKeyTile;  // tiles t with 64 t + 64 <= keys
        interior_end = interior_end < whole ? interior_end : whole;
    }
    unsigned int interior_begin = first_tile;
    if (windowed && wave_high + 1u > window) {
        // Tile t lies inside every row's window when 64 t + window > wave_high.
        const unsigned int inside = (wave_high + 1u - window + kKeyTile - 1) / kKeyTile;
        interior_begin = inside > first_tile ? inside : first_tile;
    }
    uint4 operand[kSteps];
    for (; tile < interior_begin && tile < interior_end; ++tile) {
        const TileStages stages = enter();
        fold_edge_tile(half, scores, q, offsets, 2u * tile, wave_blocks, stages.keys, stages.next_keys, stages.values, stages.key_dest,
                       stages.value_dest, issue, fold);
        leave();
    }
    if (kPagedOperandsAhead && tile < interior_end) read_key_operands(operand, lds + key_stage * kTileBytes + kBlockBytes, offsets);
    for (; tile < interior_end; ++tile) {
        const TileStages stages = enter();
        if constexpr (SOFTCAP) {
            const float cap_scale = fabsf(a.softcap_scale), cap_log2e = a.softcap_log2e;
            fold_interior_tile<kPagedOperandsAhead>(half, state, scores, operand, q, offsets, hi, factor, stages.keys, stages.next_keys, stages.values,
                                                    stages.key_dest, stages.value_dest, issue, [&](f32x16_t& s, unsigned int) {
#pragma unroll
                                                        for (int r = 0; r < 16; ++r) s[r] = fast_tanh(s[r] * cap_scale) * cap_log2e;
                                                    });
        } else {
            fold_interior_tile<kPagedOperandsAhead>(half, state, scores, operand, q, offsets, hi, factor, stages.keys, stages.next_keys, stages.values,
                                                    stages.key_dest, stages.value_dest, issue);
        }
        leave();
    }
    // Tiles on a mask's edge and the last ones (and, for waves that have run out of blocks, the workgroup's
    // remaining loads and barriers).
    for (; tile < tiles; ++tile) {
        const TileStages stages = enter();
        fold_edge_tile(half, scores, q, offsets, 2u * tile, wave_blocks, stages.keys, stages.next_keys, stages.values, stages.key_dest,
                       stages.value_dest, issue, fold);
        leave();
    }

    // Normalise and store; a row that sees no key stays zero and has a log-sum-exp of -inf
    // (paged_attention.rs:811-821, attention.rs:503-515).
    const float sum = swap32_sum(state.running_sum);
    const float inverse = sum > 0.0f ? 1.0f / sum : 0.0f;
    if (row_valid && a.splits > 1) {
        const size_t flat = (static_cast<size_t>(query_start) + my_token) * a.heads + kv_head * groups + my_head;
        const size_t slot = static_cast<size_t>(split) * a.tokens * a.heads + flat;
        float* row = a.partial_out + slot * kHeadDim;
#pragma unroll
        for (int db = 0; db < kDimBlocks; ++db)
#pragma unroll
            for (int quad = 0; quad < 4; ++quad)
                if (32 * db + 8 * quad < kHeadDim)
                    *reinterpret_cast<float4*>(row + 32 * db + 8 * quad + 4 * hi) =
                    make_float4(state.out[db][4 * quad + 0] * inverse, state.out[db][4 * quad + 1] * inverse,
                                state.out[db][4 * quad + 2] * inverse, state.out[db][4 * quad + 3] * inverse);
        if (hi == 0) a.partial_lse[slot] = sum > 0.0f ? state.reference + fast_log2(sum) : -INFINITY;
    } else if (row_valid) {
        const size_t flat = (static_cast<size_t>(query_start) + my_token) * a.heads + kv_head * groups + my_head;
        uint16_t* row = a.output + flat * kHeadDim;
#pragma unroll
        for (int db = 0; db < kDimBlocks; ++db)
#pragma unroll
            for (int quad = 0; quad < 4; ++quad) {
                if (32 * db + 8 * quad >= kHeadDim) continue;
                uint2 packed_bits;
                packed_bits.x = pack_pair(half, state.out[db][4 * quad + 0] * inverse, state.out[db][4 * quad + 1] * inverse);
                packed_bits.y = pack_pair(half, state.out[db][4 * quad + 2] * inverse, state.out[db][4 * quad + 3] * inverse);
                *reinterpret_cast<uint2*>(row + 32 * db + 8 * quad + 4 * hi) = packed_bits;
            }
        if (a.lse != nullptr && hi == 0) {
            const float lse2 = state.reference + fast_log2(sum);
            if constexpr (FORM == kTable)  // natural log, -1e20 for a row without keys (cpu/attention.rs:1304-1317)
                a.lse[flat] = sum > 0.0f ? lse2 * 0.69314718055994530942f : -1.0e20f;
            else
                a.lse[flat] = sum > 0.0f ? lse2 : -INFINITY;
        }
    }
}

// Merges the key splits of every row of a (unit, row tile): each share's output weighs 2^(lse - largest) over
// the sum of those (the merge of the reference's own split kernels, kernel_plan/source/mla.rs:497-560), the row's
// log-sum-exp is largest + log2 of that sum.  Workgroup ids map as in the attention kernel without splits; `shares`
// (at most 64) is the number of shares.
template <int FORM, class Half>
SINGE_DEVICE void combine_body(const PagedAttentionArgs& a, unsigned int shares) {
    unsigned int unit, row_tile, split;
    if (!locate<FORM, kQueryTile>(a, unit, row_tile, split)) return;
    const unsigned int sequence = unit / a.kv_heads, kv_head = unit % a.kv_heads, groups = a.heads / a.kv_heads;
    const SequenceSpan span = load_span<FORM>(sequence, a.query_offsets, a.page_offsets, a.last_page_lengths, a.query_lengths,
                                              a.tokens, a.page_table, a.page_size);
    if (!span.valid) return;  // reported by the attention kernel
    // A wave per row, rows of the tile four apart; a lane takes two of the row's values (the first 32 lanes at head_dim 64).
    const unsigned int wave = threadIdx.x >> 6, lane = threadIdx.x & 63u;
    const unsigned int packed = span.queries * groups;
    const size_t rows_total = static_cast<size_t>(a.tokens) * a.heads;
    for (unsigned int row = row_tile * kQueryTile + wave; row < packed && row < (row_tile + 1u) * kQueryTile; row += 4u) {
        const size_t flat = (static_cast<size_t>(span.query_start) + row / groups) * a.heads + kv_head * groups + row % groups;
        // The shares' log-sum-exps, one per lane (at most 64 shares), and their largest.
        const float mine = lane < shares ? a.partial_lse[lane * rows_total + flat] : -INFINITY;
        float largest = mine;
#pragma unroll
        for (int step = 32; step > 0; step >>= 1) largest = fmaxf(largest, __shfl_xor(largest, step, 64));
        const float weight = mine == -INFINITY ? 0.0f : fast_exp2(mine - largest);  // an empty share weighs nothing
        float total = weight;
#pragma unroll
        for (int step = 32; step > 0; step >>= 1) total += __shfl_xor(total, step, 64);
        float2 merged = make_float2(0.0f, 0.0f);
        const bool holds_values = 2u * lane < static_cast<unsigned int>(kHeadDim);
        // Four shares' values are asked for together; what a share that weighs nothing holds is not used.
        const float* mine_of = a.partial_out + flat * kHeadDim + (holds_values ? 2u * lane : 0u);
        const size_t share_stride = rows_total * kHeadDim;
        auto fold = [&](unsigned int s, const float2& part) __attribute__((always_inline)) {
            const float w = __shfl(weight, s, 64);
            merged.x = w == 0.0f ? merged.x : fmaf(w, part.x, merged.x);
            merged.y = w == 0.0f ? merged.y : fmaf(w, part.y, merged.y);
        };
        unsigned int s = 0;
        for (; s + 4 <= shares; s += 4) {
            float2 part[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) part[i] = *reinterpret_cast<const float2*>(mine_of + (s + i) * share_stride);
#pragma unroll
            for (int i = 0; i < 4; ++i) fold(s + i, part[i]);
        }
        for (; s < shares; ++s) fold(s, *reinterpret_cast<const float2*>(mine_of + s * share_stride));
        const float inverse = total > 0.0f ? 1.0f / total : 0.0f;
        if (holds_values) reinterpret_cast<unsigned int*>(a.output + flat * kHeadDim)[lane] = pack_pair(Half{}, merged.x * inverse, merged.y * inverse);
        if (a.lse != nullptr && lane == 0) a.lse[flat] = total > 0.0f ? largest + fast_log2(total) : -INFINITY;
    }
}

}  // namespace

// The merge of key splits: the same argument block as the attention kernel, whose `splits` counts the shares
// here while workgroup ids map as without splits.
#define SINGE_PAGED_COMBINE_KERNEL(NAME, FORM, HALF)                                         \
    extern "C" __global__ __launch_bounds__(256) void NAME(PagedAttentionArgs args) {        \
        const unsigned int shares = args.splits;                                             \
        args.splits = 1;                                                                     \
        combine_body<FORM, prefill::HALF>(args, shares);                                     \
    }

// Names carry the head dimension of the build: singe_paged_attention_bf16_d128_i32, ..._d64_i32.
#define SINGE_PASTE4_(a, b, c, d) a##b##c##d
#define SINGE_PASTE4(a, b, c, d) SINGE_PASTE4_(a, b, c, d)
#define SINGE_PAGED_NAME(STEM, TAIL) SINGE_PASTE4(STEM, _d, SINGE_HEAD_DIM, TAIL)
#if SINGE_HEAD_DIM == 128
// (the merge kernels of the head_dim 128 build keep their first names)
SINGE_PAGED_COMBINE_KERNEL(singe_paged_attention_combine_bf16_i32, kCsrI32, Bf16)
SINGE_PAGED_COMBINE_KERNEL(singe_paged_attention_combine_bf16_i64, kCsrI64, Bf16)
SINGE_PAGED_COMBINE_KERNEL(singe_paged_attention_combine_f16_i32, kCsrI32, F16)
SINGE_PAGED_COMBINE_KERNEL(singe_paged_attention_combine_f16_i64, kCsrI64, F16)
#else
SINGE_PAGED_COMBINE_KERNEL(SINGE_PAGED_NAME(singe_paged_attention_combine_bf16, _i32), kCsrI32, Bf16)
SINGE_PAGED_COMBINE_KERNEL(SINGE_PAGED_NAME(singe_paged_attention_combine_bf16, _i64), kCsrI64, Bf16)
SINGE_PAGED_COMBINE_KERNEL(SINGE_PAGED_NAME(singe_paged_attention_combine_f16, _i32), kCsrI32, F16)
SINGE_PAGED_COMBINE_KERNEL(SINGE_PAGED_NAME(singe_paged_attention_combine_f16, _i64), kCsrI64, F16)
#endif

#define SINGE_PAGED_ATTENTION_KERNEL(NAME, SOFTCAP, FORM, GROUPED, ROTATE, HALF)                           \
    extern "C" __global__ __launch_bounds__(256, 2) void NAME(PagedAttentionArgs args) {                    \
        __shared__ __attribute__((aligned(1024))) unsigned char paged_lds[prefill::kStagedLdsBytes];        \
        paged_attention_body<SOFTCAP, FORM, GROUPED, ROTATE, prefill::HALF>(args, paged_lds);              \
    }

// _p16: the page size is a power of two of at least 16 keys (page ids on the scalar unit).
SINGE_PAGED_ATTENTION_KERNEL(SINGE_PAGED_NAME(singe_paged_attention_bf16, _i32), false, kCsrI32, false, false, Bf16)
SINGE_PAGED_ATTENTION_KERNEL(SINGE_PAGED_NAME(singe_paged_attention_bf16, _i64), false, kCsrI64, false, false, Bf16)
SINGE_PAGED_ATTENTION_KERNEL(SINGE_PAGED_NAME(singe_paged_attention_bf16, _softcap_i32), true, kCsrI32, false, false, Bf16)
SINGE_PAGED_ATTENTION_KERNEL(SINGE_PAGED_NAME(singe_paged_attention_bf16, _softcap_i64), true, kCsrI64, false, false, Bf16)
SINGE_PAGED_ATTENTION_KERNEL(SINGE_PAGED_NAME(singe_paged_attention_bf16, _i32_p16), false, kCsrI32, true, false, Bf16)
SINGE_PAGED_ATTENTION_KERNEL(SINGE_PAGED_NAME(singe_paged_attention_bf16, _i64_p16), false, kCsrI64, true, false, Bf16)
SINGE_PAGED_ATTENTION_KERNEL(SINGE_PAGED_NAME(singe_paged_attention_bf16, _softcap_i32_p16), true, kCsrI32, true, false, Bf16)
SINGE_PAGED_ATTENTION_KERNEL(SINGE_PAGED_NAME(singe_paged_attention_bf16, _softcap_i64_p16), true, kCsrI64, true, false, Bf16)
// paged_kv_prefill_attention_bf16 of the singe-kernel surface: same gather, block-table paging.
SINGE_PAGED_ATTENTION_KERNEL(SINGE_PAGED_NAME(singe_paged_kv_prefill_bf16, /**/), false, kTable, false, false, Bf16)
SINGE_PAGED_ATTENTION_KERNEL(SINGE_PAGED_NAME(singe_paged_kv_prefill_bf16, _p16), false, kTable, true, false, Bf16)
SINGE_PAGED_ATTENTION_KERNEL(SINGE_PAGED_NAME(singe_paged_kv_prefill_f16, /**/), false, kTable, false, false, F16)
SINGE_PAGED_ATTENTION_KERNEL(SINGE_PAGED_NAME(singe_paged_kv_prefill_f16, _p16), false, kTable, true, false, F16)
// rotary_paged_attention: the query is normalised and rotated on its way into the registers.
SINGE_PAGED_ATTENTION_KERNEL(SINGE_PAGED_NAME(singe_rotary_paged_attention_bf16, _i32), false, kCsrI32, false, true, Bf16)
SINGE_PAGED_ATTENTION_KERNEL(SINGE_PAGED_NAME(singe_rotary_paged_attention_bf16, _i64), false, kCsrI64, false, true, Bf16)
SINGE_PAGED_ATTENTION_KERNEL(SINGE_PAGED_NAME(singe_rotary_paged_attention_bf16, _i32_p16), false, kCsrI32, true, true, Bf16)
SINGE_PAGED_ATTENTION_KERNEL(SINGE_PAGED_NAME(singe_rotary_paged_attention_bf16, _i64_p16), false, kCsrI64, true, true, Bf16)
SINGE_PAGED_ATTENTION_KERNEL(SINGE_PAGED_NAME(singe_rotary_paged_attention_bf16, _softcap_i32), true, kCsrI32, false, true, Bf16)
SINGE_PAGED_ATTENTION_KERNEL(SINGE_PAGED_NAME(singe_rotary_paged_attention_bf16, _softcap_i64), true, kCsrI64, false, true, Bf16)
SINGE_PAGED_ATTENTION_KERNEL(SINGE_PAGED_NAME(singe_rotary_paged_attention_bf16, _softcap_i32_p16), true, kCsrI32, true, true, Bf16)
SINGE_PAGED_ATTENTION_KERNEL(SINGE_PAGED_NAME(singe_rotary_paged_attention_bf16, _softcap_i64_p16), true, kCsrI64, true, true, Bf16)
SINGE_PAGED_ATTENTION_KERNEL(SINGE_PAGED_NAME(singe_rotary_paged_attention_f16, _i32), false, kCsrI32, false, true, F16)
SINGE_PAGED_ATTENTION_KERNEL(SINGE_PAGED_NAME(singe_rotary_paged_attention_f16, _i64), false, kCsrI64, false, true, F16)
SINGE_PAGED_ATTENTION_KERNEL(SINGE_PAGED_NAME(singe_rotary_paged_attention_f16, _i32_p16), false, kCsrI32, true, true, F16)
SINGE_PAGED_ATTENTION_KERNEL(SINGE_PAGED_NAME(singe_rotary_paged_attention_f16, _i64_p16), false, kCsrI64, true, true, F16)
SINGE_PAGED_ATTENTION_KERNEL(SINGE_PAGED_NAME(singe_rotary_paged_attention_f16, _softcap_i32), true, kCsrI32, false, true, F16)
SINGE_PAGED_ATTENTION_KERNEL(SINGE_PAGED_NAME(singe_rotary_paged_attention_f16, _softcap_i64), true, kCsrI64, false, true, F16)
SINGE_PAGED_ATTENTION_KERNEL(SINGE_PAGED_NAME(singe_rotary_paged_attention_f16, _softcap_i32_p16), true, kCsrI32, true, true, F16)
SINGE_PAGED_ATTENTION_KERNEL(SINGE_PAGED_NAME(singe_rotary_paged_attention_f16, _softcap_i64_p16), true, kCsrI64, true, true, F16)
// f16 operands: the same kernels on v_mfma_f32_32x32x16_f16.
SINGE_PAGED_ATTENTION_KERNEL(SINGE_PAGED_NAME(singe_paged_attention_f16, _i32), false, kCsrI32, false, false, F16)
SINGE_PAGED_ATTENTION_KERNEL(SINGE_PAGED_NAME(singe_paged_attention_f16, _i64), false, kCsrI64, false, false, F16)
SINGE_PAGED_ATTENTION_KERNEL(SINGE_PAGED_NAME(singe_paged_attention_f16, _softcap_i32), true, kCsrI32, false, false, F16)
SINGE_PAGED_ATTENTION_KERNEL(SINGE_PAGED_NAME(singe_paged_attention_f16, _softcap_i64), true, kCsrI64, false, false, F16)
SINGE_PAGED_ATTENTION_KERNEL(SINGE_PAGED_NAME(singe_paged_attention_f16, _i32_p16), false, kCsrI32, true, false, F16)
SINGE_PAGED_ATTENTION_KERNEL(SINGE_PAGED_NAME(singe_paged_attention_f16, _i64_p16), false, kCsrI64, true, false, F16)
SINGE_PAGED_ATTENTION_KERNEL(SINGE_PAGED_NAME(singe_paged_attention_f16, _softcap_i32_p16), true, kCsrI32, true, false, F16)
SINGE_PAGED_ATTENTION_KERNEL(SINGE_PAGED_NAME(singe_paged_attention_f16, _softcap_i64_p16), true, kCsrI64, true, false, F16)
