// Attention of ragged queries over a paged KV cache in FlashInfer form: decode, prefill and chunked
// prefill in one kernel, the gfx950 counterpart of singe_paged_attention
// (singe/src/backend/cuda/kernel_plan/source/paged_attention.rs:544-868) and of the CPU attend_paged
// (singe/src/backend/cpu/normalization/attention.rs:424-538).
//
// query_rows/output [tokens, heads, 128] bf16; caches [pages, page_size, kv_heads, 128] bf16; sequence b
// holds queries query_offsets[b] .. query_offsets[b+1] and the keys of pages
// pages[page_offsets[b] .. page_offsets[b+1]], all full but the last, which holds last_page_lengths[b];
// lse [tokens, heads] f32, base two, -inf for a row that sees no key.  Queries are a sequence's LAST
// tokens: query q sits at key position max(keys - queries + q, 0) (bottom-right causal alignment, with
// the CPU path's saturating subtraction: attention.rs:482-488).
//
// A workgroup owns 128 packed rows of one (sequence, kv head): the query heads that share the kv head,
// a token's heads consecutive (row r = token r / groups, head r % groups), so a key tile is staged once
// for the whole group.  The grid covers every sequence's longest possible run of rows; workgroups past
// their sequence's rows return at once.  Keys are gathered page by page into the same padded LDS tiles
// as the dense kernel and folded by the shared core (prefill_core.hip.h).
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
#include "prefill_core.hip.h"

namespace {

using namespace prefill;

template <bool SOFTCAP, int FORM>
SINGE_DEVICE void paged_attention_body(const PagedAttentionArgs& a, unsigned char* lds) {
    const unsigned int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const unsigned int column = lane & 31, hi = lane >> 5;
    const unsigned int groups = a.heads / a.kv_heads;

    // Workgroup i runs on XCD i % 8: the row tiles of one (sequence, kv head) share an XCD and its L2.
    const unsigned int xcd = blockIdx.x & 7u, within = blockIdx.x >> 3;
    const unsigned int unit = (within / a.row_tiles) * 8u + xcd;
    if (unit >= a.sequences * a.kv_heads) return;
    const unsigned int sequence = unit / a.kv_heads, kv_head = unit % a.kv_heads;
    const unsigned int first_row = (within % a.row_tiles) * kQueryTile;

    // The sequence's paging values, refused when any would address outside the kernel's buffers.
    const SequenceSpan span = load_span<FORM>(sequence, a.query_offsets, a.page_offsets, a.last_page_lengths, a.query_lengths,
                                              a.tokens, a.page_table, a.page_size);
    if (!span.valid) {
        if (tid == 0) report_index_error(a.status);
        return;
    }
    const long long query_start = span.query_start, page_start = span.page_start;
    const unsigned int queries = span.queries, keys = span.keys;
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
    const unsigned int window = windowed ? static_cast<unsigned int>(a.window) : 0u;

    // Rows of this wave: none when the wave starts past the sequence's rows.
    const unsigned int wave_first_row = first_row + wave * 32u;
    const bool wave_live = wave_first_row < packed;
    const unsigned int wave_last_row = wave_live ? (wave_first_row + 31u < packed ? wave_first_row + 31u : packed - 1u) : first_row;
    const unsigned int wave_low = position_of(wave_live ? wave_first_row : first_row), wave_high = position_of(wave_last_row);

    // Keys this workgroup must visit.
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
    const unsigned int end_tile = (key_end + kKeyTile - 1) / kKeyTile;

    // Q^T as the MFMA B operand; a negative scale moves into Q (see fmha_prefill.hip).
    const float factor = SOFTCAP ? 1.0f : fabsf(a.scale_log2e);
    const unsigned int flip = (SOFTCAP ? a.softcap_scale : a.scale_log2e) < 0.0f ? 0x80008000u : 0u;
    bf16x8_t q[8];
    {
        const uint16_t* row = a.query_rows + ((static_cast<size_t>(query_start) + my_token) * a.heads + kv_head * groups + my_head) * kHeadDim + 8 * hi;
#pragma unroll
        for (int s = 0; s < 8; ++s) {
            uint4 bits = *reinterpret_cast<const uint4*>(row + 16 * s);
            if (!row_valid) bits = make_uint4(0, 0, 0, 0);
            bits.x ^= flip; bits.y ^= flip; bits.z ^= flip; bits.w ^= flip;
            q[s] = __builtin_bit_cast(bf16x8_t, bits);
        }
    }

    // Tile loads: 1024 16-byte chunks per operand per tile, four per thread (rows load_row + 16 i).
    // The page of each row is looked up one tile ahead of the row itself, so the gather never waits on
    // two dependent round trips.
    const unsigned int load_row = tid >> 4, load_col = tid & 15u;
    const unsigned int page_elements = a.page_size * a.kv_heads * kHeadDim;  // fits 32 bits (checked by the host)
    // When the page size divides the tile (1, 2, ..., 64 keys) a thread's rows sit at the same slots of
    // their pages in every tile and a tile covers a whole number of pages, so only the page ids change from
    // tile to tile; other page sizes divide per row.
    const bool regular = a.page_shift >= 0 && a.page_size <= static_cast<unsigned int>(kKeyTile);
    const unsigned int pages_per_tile = regular ? static_cast<unsigned int>(kKeyTile) >> a.page_shift : 0u;
    auto slot_of = [&](unsigned int key) __attribute__((always_inline)) { return regular ? key & (a.page_size - 1u) : key % a.page_size; };
    auto entry_of = [&](unsigned int key) __attribute__((always_inline)) { return regular ? key >> a.page_shift : key / a.page_size; };
    unsigned int row_offset0 = 0, row_offset1 = 0, row_offset2 = 0, row_offset3 = 0;  // (slot * kv_heads + kv_head) * 128 + column
    if (regular) {
        row_offset0 = (slot_of(load_row) * a.kv_heads + kv_head) * kHeadDim + load_col * 8u;
        row_offset1 = (slot_of(load_row + 16u) * a.kv_heads + kv_head) * kHeadDim + load_col * 8u;
        row_offset2 = (slot_of(load_row + 32u) * a.kv_heads + kv_head) * kHeadDim + load_col * 8u;
        row_offset3 = (slot_of(load_row + 48u) * a.kv_heads + kv_head) * kHeadDim + load_col * 8u;
    }
    uint4 k0, k1, k2, k3, v0, v1, v2, v3;
    unsigned long long page0, page1, page2, page3;  // of the rows of the tile that is fetched next
    auto lookup_row = [&](unsigned int tile, unsigned int i, unsigned long long& page) __attribute__((always_inline)) {
        const unsigned int key = tile * kKeyTile + load_row + 16u * i;
        page = 0;
        if (key < keys) {
            // The tile's first table entry is the same for every lane; the row adds a small offset.
            const size_t tile_entry = static_cast<size_t>(page_start) + (regular ? tile * pages_per_tile : 0u);
            page = read_page<FORM>(a.pages, tile_entry + (regular ? entry_of(load_row + 16u * i) : entry_of(key)));
        }
    };
    auto lookup = [&](unsigned int tile) __attribute__((always_inline)) {
        lookup_row(tile, 0, page0);
        lookup_row(tile, 1, page1);
        lookup_row(tile, 2, page2);
        lookup_row(tile, 3, page3);
    };
    auto fetch_row = [&](unsigned int tile, unsigned int i, unsigned long long page, unsigned int row_offset, uint4& key_bits,
                         uint4& value_bits) __attribute__((always_inline)) {
        const unsigned int key = tile * kKeyTile + load_row + 16u * i;
        const bool wanted = key < keys;
        const bool valid = wanted && page < static_cast<unsigned long long>(a.cache_pages);  // negative pages wrap above it
        if (wanted && !valid) report_index_error(a.status);
        key_bits = make_uint4(0, 0, 0, 0);
        value_bits = make_uint4(0, 0, 0, 0);
        if (valid) {
            if (!regular) row_offset = (slot_of(key) * a.kv_heads + kv_head) * kHeadDim + load_col * 8u;
            // One 32 x 32 -> 64-bit multiply-add places the page; everything else is 32-bit.
            const size_t offset = static_cast<size_t>(static_cast<unsigned int>(page)) * page_elements + row_offset;
            key_bits = *reinterpret_cast<const uint4*>(a.key_cache + offset);
            value_bits = *reinterpret_cast<const uint4*>(a.value_cache + offset);
        }
    };
    auto fetch = [&](unsigned int tile) __attribute__((always_inline)) {
        fetch_row(tile, 0, page0, row_offset0, k0, v0);
        fetch_row(tile, 1, page1, row_offset1, k1, v1);
        fetch_row(tile, 2, page2, row_offset2, k2, v2);
        fetch_row(tile, 3, page3, row_offset3, k3, v3);
    };
    auto stash_row = [&](unsigned char* keys_at, unsigned char* values_at, unsigned int i, const uint4& key_bits, const uint4& value_bits) __attribute__((always_inline)) {
        const unsigned int row = load_row + 16u * i;
        *reinterpret_cast<uint4*>(keys_at + row * kKeyRowBytes + load_col * 16) = key_bits;
        *reinterpret_cast<uint4*>(values_at + row * kValueRowBytes + load_col * 16) = value_bits;
    };
    auto stash = [&](unsigned char* keys_at, unsigned char* values_at) __attribute__((always_inline)) {
        stash_row(keys_at, values_at, 0, k0, v0);
        stash_row(keys_at, values_at, 1, k1, v1);
        stash_row(keys_at, values_at, 2, k2, v2);
        stash_row(keys_at, values_at, 3, k3, v3);
    };

    RowState state;
    reset(state);
    const unsigned int key_read = key_read_offset(lane), value_read = value_read_offset(lane);

    auto fold = [&](unsigned int tile, const unsigned char* keys_at, const unsigned char* values_at) __attribute__((always_inline)) {
        const unsigned int key0 = tile * kKeyTile;
        // A 32-key block is dead for the wave when every row's mask hides all of it.
        auto block_live = [&](unsigned int base) __attribute__((always_inline)) {
            if (!wave_live || base >= keys) return false;
            if (causal && base > wave_high) return false;
            if (windowed && base + 31u + window <= wave_low) return false;
            return true;
        };
        const bool live0 = block_live(key0), live1 = block_live(key0 + 32u);
        if (!live0 && !live1) return;
        const bool edge = !live0 || (causal && key0 + kKeyTile - 1 > wave_low) || key0 + kKeyTile > keys || windowed;
        fold_staged_keys<SOFTCAP>(state, q, keys_at, values_at, key_read, value_read, hi, factor, live1, edge,
                                  [&](unsigned int block, unsigned int key_in_block) {
                                      const unsigned int key = key0 + 32 * block + key_in_block;
                                      return (block == 0 && !live0) || key >= keys || (causal && key > my_position) ||
                                             (windowed && key + window <= my_position);
                                  },
                                  fabsf(a.softcap_scale), a.softcap_log2e);
    };

    unsigned char* const keys0 = lds;
    unsigned char* const values0 = lds + kKeyStageBytes;
    unsigned char* const keys1 = lds + kStageBytes;
    unsigned char* const values1 = lds + kStageBytes + kKeyStageBytes;
    if (first_tile < end_tile) {
        lookup(first_tile);
        fetch(first_tile);
        if (first_tile + 1 < end_tile) lookup(first_tile + 1);
        stash(keys0, values0);
    }
    __syncthreads();
    for (unsigned int tile = first_tile; tile < end_tile; tile += 2) {
        if (tile + 1 < end_tile) {
            fetch(tile + 1);
            if (tile + 2 < end_tile) lookup(tile + 2);
        }
        fold(tile, keys0, values0);
        if (tile + 1 < end_tile) stash(keys1, values1);
        __syncthreads();
        if (tile + 1 >= end_tile) break;
        if (tile + 2 < end_tile) {
            fetch(tile + 2);
            if (tile + 3 < end_tile) lookup(tile + 3);
        }
        fold(tile + 1, keys1, values1);
        if (tile + 2 < end_tile) stash(keys0, values0);
        __syncthreads();
    }

    // Normalise and store; a row that sees no key stays zero and has a log-sum-exp of -inf
    // (paged_attention.rs:811-821, attention.rs:503-515).
    const float sum = swap32_sum(state.running_sum);
    const float inverse = sum > 0.0f ? 1.0f / sum : 0.0f;
    if (row_valid) {
        const size_t flat = (static_cast<size_t>(query_start) + my_token) * a.heads + kv_head * groups + my_head;
        uint16_t* row = a.output + flat * kHeadDim;
#pragma unroll
        for (int db = 0; db < 4; ++db)
#pragma unroll
            for (int quad = 0; quad < 4; ++quad) {
                uint2 packed_bits;
                packed_bits.x = pack_pair(state.out[db][4 * quad + 0] * inverse, state.out[db][4 * quad + 1] * inverse);
                packed_bits.y = pack_pair(state.out[db][4 * quad + 2] * inverse, state.out[db][4 * quad + 3] * inverse);
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

}  // namespace

#define SINGE_PAGED_ATTENTION_KERNEL(NAME, SOFTCAP, FORM)                                              \
    extern "C" __global__ __launch_bounds__(256, 2) void NAME(PagedAttentionArgs args) {                \
        __shared__ __attribute__((aligned(16))) unsigned char paged_lds[2 * prefill::kStageBytes];     \
        paged_attention_body<SOFTCAP, FORM>(args, paged_lds);                                          \
    }

SINGE_PAGED_ATTENTION_KERNEL(singe_paged_attention_bf16_d128_i32, false, kCsrI32)
SINGE_PAGED_ATTENTION_KERNEL(singe_paged_attention_bf16_d128_i64, false, kCsrI64)
SINGE_PAGED_ATTENTION_KERNEL(singe_paged_attention_bf16_d128_softcap_i32, true, kCsrI32)
SINGE_PAGED_ATTENTION_KERNEL(singe_paged_attention_bf16_d128_softcap_i64, true, kCsrI64)
// paged_kv_prefill_attention_bf16 of the singe-kernel surface: same gather, block-table paging.
SINGE_PAGED_ATTENTION_KERNEL(singe_paged_kv_prefill_bf16_d128, false, kTable)
