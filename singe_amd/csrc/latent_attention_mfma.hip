// Latent attention over paged caches on the matrix cores: bf16 or f16, latent width 512, positional width 64
// (DeepSeek's absorbed MLA).  The same op as latent_attention.hip (CPU: singe/src/backend/cpu/normalization/
// attention.rs:540-679; kernel plan: singe/src/backend/cuda/kernel_plan/source/mla.rs), built for the one shape that
// matters in practice.  The `_any` kernels (ANY below) run the same loop for every other width the reference's
// tensor-core plan takes with a positional part of at most 64 (latent a multiple of 32 up to 512, positional a multiple
// of 8: mla.rs:75, 140-146): rows keep their 512 + 64 places in LDS, a lane whose chunk lies past a row's real width
// loads nothing and finds the zeros the stages were filled with at the start, Q^T is zero there, and the outputs past
// the latent width are not stored; narrower shapes pay for the full width's products.
//
// Every head of a token attends over the same cache rows, so the rows of a sequence, (query, head) pairs in
// query-major order, are tiled 128 to a workgroup and the cache is read once per tile of rows instead of once
// per head.  A workgroup is eight waves; wave w owns rows 16 w .. 16 w + 15 of the tile for the whole of the
// keys.  Keys come in tiles of 32, straight from global memory into LDS (global_load_lds_dwordx4), one tile
// ahead of the one being worked on; all eight waves read every tile.
//
//   S^T[key, row] = C[key, :] . Q[row, :]   v_mfma_f32_16x16x32: A = cache rows from LDS (ds_read_b128),
//                                           B = the wave's Q^T, 18 steps of 32 dims (16 latent, 2 positional)
//                                           held in registers; two products of 16 keys each.
//   O^T[dim, row] += C^T[dim, key] . P^T    A = the latent part of the same LDS rows, transposed on the way
//                                           out by ds_read_b64_tr_b16; B = the weights, packed from the score
//                                           registers with no lane traffic: lane (row, g) holds keys
//                                           4 g .. 4 g + 3 of either 16-key half, which is what the A operand's
//                                           lane group g is made to read.  32 products of 16 dims.
//
// LDS rows are unpadded (the direct loads write 1 KiB runs); bank conflicts are kept down by permuting the 16-byte
// chunks of a row, on the global side of the load and again in the read offsets: latent chunk c of key k sits at
// c ^ f(k), f a permutation of 0..15 (chunk_flip below) that spreads the 16 keys of a score operand over all banks
// and, through f(k) >> 1, the 8 keys that one pass of a transposed read serves: lanes 0-15 go with lanes 32-47 there,
// so keys 0-3 with 8-11 and 4-7 with 12-15 (measured: SQ_LDS_BANK_CONFLICT drops from 28 % of the LDS cycles to 0
// against a permutation that only separates keys 0-7 and 8-15).  Positional chunk c (of 8) sits at c ^ (k & 7).
#include "common.hip.h"
#include "kernel_args.h"
#include "paging.hip.h"
#include "prefill_core.hip.h"

namespace latent_mfma {

using prefill::Bf16;
using prefill::F16;
using prefill::kMaxLag;
using prefill::pack_pair;
using prefill::v4i16_t;

constexpr int kLatent = 512, kPositional = 64;
constexpr int kWaves = 8, kRows = 16 * kWaves;  // rows of a workgroup
constexpr int kKeys = 32;                      // keys per tile
constexpr int kLatentRowBytes = kLatent * 2, kPositionalRowBytes = kPositional * 2;
constexpr int kLatentTileBytes = kKeys * kLatentRowBytes;          // 32 KiB
constexpr int kPositionalTileBytes = kKeys * kPositionalRowBytes;  // 4 KiB
constexpr int kStageBytes = kLatentTileBytes + kPositionalTileBytes;
// The first steps of Q^T live in LDS, one 16-byte slot per (step, lane) that only its own lane touches, to leave the
// wave registers for the operands in flight.
constexpr int kParkedSteps = 8;
constexpr int kParkedBytes = kParkedSteps * 1024 * kWaves;
constexpr int kLdsBytes = 2 * kStageBytes + kParkedBytes;
constexpr int kLatentSteps = kLatent / 32, kSteps = (kLatent + kPositional) / 32;
constexpr int kDimBlocks = kLatent / 16;

typedef unsigned int __attribute__((address_space(3))) * lds_words_t;
typedef v4i16_t __attribute__((address_space(3))) * lds_v4_t;

SINGE_DEVICE f32x4_t mma(Bf16, uint4 a, uint4 b, f32x4_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
}
SINGE_DEVICE f32x4_t mma(F16, uint4 a, uint4 b, f32x4_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(prefill::f16x8v_t, a), __builtin_bit_cast(prefill::f16x8v_t, b), c, 0, 0, 0);
}

// One direct-to-LDS load: every active lane's 16 bytes at `source` go to the wave's `dest` + 16 * lane.  Written as
// text so that the compiler keeps counting its own LDS reads and loads as usual (it makes every LDS read after the
// built-in form wait for all of them, and the first one for the load itself); the kernel waits for these loads with
// vmcnt(0) before the barrier that hands a stage on.
SINGE_DEVICE void load_to_lds(const unsigned char* source, unsigned char* dest) {
    const unsigned int base = __builtin_amdgcn_readfirstlane(static_cast<unsigned int>(reinterpret_cast<__UINTPTR_TYPE__>((lds_words_t)dest)));
    // M0 carries the LDS base of the load; it is read when the load issues, so the statement puts back what M0 held
    // and the compiler's own uses of M0 around it are not disturbed.
    unsigned int kept;
    asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, off\n\ts_mov_b32 m0, %0"
                 : "=&s"(kept) : "s"(base), "v"(source) : "memory");
}

// The same with the address in two parts, a base every lane shares (kept in scalar registers) and a 32-bit offset per
// lane: a wave-uniform row costs no 64-bit address per lane, in registers or in arithmetic.
SINGE_DEVICE void load_to_lds(const unsigned char* shared_base, unsigned int lane_offset, unsigned char* dest) {
    const unsigned int base = __builtin_amdgcn_readfirstlane(static_cast<unsigned int>(reinterpret_cast<__UINTPTR_TYPE__>((lds_words_t)dest)));
    const unsigned long long bits = reinterpret_cast<unsigned long long>(shared_base);
    // (the built-in returns an int: through unsigned int first, or a low word with its top bit set would fill the high word)
    const unsigned int low_word = __builtin_amdgcn_readfirstlane(static_cast<unsigned int>(bits));
    const unsigned int high_word = __builtin_amdgcn_readfirstlane(static_cast<unsigned int>(bits >> 32));
    const unsigned long long scalar = static_cast<unsigned long long>(low_word) | (static_cast<unsigned long long>(high_word) << 32);
    unsigned int kept;
    asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, %3\n\ts_mov_b32 m0, %0"
                 : "=&s"(kept) : "s"(base), "v"(lane_offset), "s"(scalar) : "memory");
}

// The same with the destination as the byte address in LDS that M0 takes (a pointer into LDS costs a null test and a
// select on its way there).
SINGE_DEVICE void load_to_lds(const unsigned char* shared_base, unsigned int lane_offset, unsigned int lds_byte_address) {
    const unsigned int base = __builtin_amdgcn_readfirstlane(lds_byte_address);
    const unsigned long long bits = reinterpret_cast<unsigned long long>(shared_base);
    const unsigned int low_word = __builtin_amdgcn_readfirstlane(static_cast<unsigned int>(bits));
    const unsigned int high_word = __builtin_amdgcn_readfirstlane(static_cast<unsigned int>(bits >> 32));
    const unsigned long long scalar = static_cast<unsigned long long>(low_word) | (static_cast<unsigned long long>(high_word) << 32);
    unsigned int kept;
    asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, %3\n\ts_mov_b32 m0, %0"
                 : "=&s"(kept) : "s"(base), "v"(lane_offset), "s"(scalar) : "memory");
}

// Where the chunk permutation of a latent row puts things: see the header comment.
SINGE_DEVICE unsigned int chunk_flip(unsigned int key) {
    const unsigned int pair = (key & 3u) | ((((key >> 2) ^ (key >> 3)) & 1u) << 2);
    return (pair << 1) | ((key >> 3) & 1u);
}

// Workgroup units map to (sequence, row tile) in sequence order: sequence s owns max(1, ceil(rows_s / 128)) units (one
// even without rows, so that its paging values are checked), which every wave finds for itself by a prefix sum over
// the query offsets, 64 sequences at a time.  Returns false for a unit past the last sequence's.
template <int FORM>
SINGE_DEVICE bool find_unit(const LatentAttentionArgs& a, unsigned int unit, unsigned int& sequence, unsigned int& row_tile) {
    const unsigned int lane = threadIdx.x & 63u;
    unsigned int base = 0;
    for (unsigned int first = 0; first < a.sequences; first += 64u) {
        const unsigned int s = first + lane;
        unsigned int mine = 0;
        if (s < a.sequences) {
            long long count = read_index<FORM>(a.query_offsets, s + 1) - read_index<FORM>(a.query_offsets, s);
            count = count < 0 ? 0 : count > static_cast<long long>(a.tokens) ? static_cast<long long>(a.tokens) : count;
            const unsigned long long tiles = (static_cast<unsigned long long>(count) * a.heads + kRows - 1) / kRows;
            mine = tiles == 0 ? 1u : static_cast<unsigned int>(tiles);
        }
        unsigned int through = mine;  // inclusive prefix sum over the wave
#pragma unroll
        for (int step = 1; step < 64; step <<= 1) {
            const unsigned int below = __shfl_up(through, step, 64);
            if (lane >= static_cast<unsigned int>(step)) through += below;
        }
        const unsigned int total = __shfl(through, 63, 64);
        if (unit < base + total) {
            const unsigned long long holds = __ballot(unit < base + through);  // first lane whose range reaches the unit
            const unsigned int owner = static_cast<unsigned int>(__builtin_ctzll(holds));
            const unsigned int owner_through = __shfl(through, owner, 64), owner_mine = __shfl(mine, owner, 64);
            sequence = first + owner;
            row_tile = unit - (base + owner_through - owner_mine);
            return true;
        }
        base += total;
    }
    return false;
}

// What a wave needs to know of the keys it loads for one tile: its four latent rows (wave-uniform) and, for waves
// 0-3, each lane's positional row.
template <int FORM>
struct TilePages {
    RawPage<FORM> latent[4];
    RawPage<FORM> positional;
};

// IN_PAGE: the page size is a power of two of at least 32 keys, so the 32 keys of a tile lie in one page: one page id a
// tile (instead of one a row), no division, and a key's place follows from the tile's.  A wave issues its instructions in
// order, one every four or five clocks whatever their kind, so the scalar arithmetic of the paging is time the matrix
// cores do not get from that wave.
template <class Half, int FORM, bool ANY, bool IN_PAGE>
SINGE_DEVICE void latent_tile_rows(const LatentAttentionArgs& a, unsigned char* lds) {
    const unsigned int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63u;
    // The widths of a row in global memory: the built shape, or (ANY) whatever the problem says.
    const unsigned int latent_row_bytes = ANY ? 2u * a.latent_dim : static_cast<unsigned int>(kLatentRowBytes);
    const unsigned int positional_row_bytes = ANY ? 2u * a.position_dim : static_cast<unsigned int>(kPositionalRowBytes);
    const unsigned int latent_chunks = ANY ? a.latent_dim / 8u : 64u, positional_chunks = ANY ? a.position_dim / 8u : 8u;
    if constexpr (ANY) {
        // Chunks past a row's real width are never loaded: they read as the zeros put here.
        for (unsigned int at = threadIdx.x * 16u; at < 2u * kStageBytes; at += 64u * kWaves * 16u)
            *reinterpret_cast<uint4*>(lds + at) = make_uint4(0, 0, 0, 0);
        __syncthreads();
    }
    const unsigned int column = lane & 15u, g = lane >> 4;  // row of the wave, lane group
    const unsigned int splits = a.splits > 1 ? a.splits : 1u;
    // Workgroup i runs on XCD i % 8.  Without key splits, units (row tiles, in sequence order) are dealt to the
    // XCDs in bands of a.unit_band neighbours, so that the workgroups an XCD runs side by side are row tiles of the
    // same sequence walking the same keys, and the cache rows one of them brings into the XCD's L2 serve the others.
    // With key splits the units are few and their shares read different keys: the shares of a unit are neighbouring
    // workgroups and so go round the XCDs, which keeps every XCD busy however few units there are (and share s of
    // every unit still meets the same few XCDs when the count of shares is a power of two).
    unsigned int split = 0, unit;
    if (splits > 1) {
        split = blockIdx.x % splits;
        unit = blockIdx.x / splits;
    } else {
        const unsigned int xcd = blockIdx.x & 7u, within = blockIdx.x >> 3;
        unit = ((within / a.unit_band) * 8u + xcd) * a.unit_band + within % a.unit_band;
    }
    unsigned int sequence, row_tile;
    if (!find_unit<FORM>(a, unit, sequence, row_tile)) return;
    sequence = __builtin_amdgcn_readfirstlane(sequence);
    row_tile = __builtin_amdgcn_readfirstlane(row_tile);
    const SequenceSpan span = load_span<FORM>(sequence, a.query_offsets, a.page_offsets, a.last_page_lengths, nullptr, a.tokens,
                                              a.page_table, a.page_size);
    if (!span.valid) {
        if (threadIdx.x == 0) report_index_error(a.status);
        return;
    }
    const unsigned long long rows = static_cast<unsigned long long>(span.queries) * a.heads;
    const unsigned long long first_row = static_cast<unsigned long long>(row_tile) * kRows;
    if (first_row >= rows) return;
    const unsigned int keys = span.keys;

    // Queries are the sequence's last tokens, with the CPU path's saturating position (attention.rs:619-627).
    auto position_of = [&](unsigned long long row) __attribute__((always_inline)) {
        const long long raw = static_cast<long long>(keys) - static_cast<long long>(span.queries) + static_cast<long long>(row / a.heads);
        return raw < 0 ? 0u : static_cast<unsigned int>(raw);
    };
    const unsigned long long my_row = first_row + 16u * wave + column;
    const bool row_valid = my_row < rows;
    const unsigned long long safe_row = row_valid ? my_row : first_row;
    const size_t flat = (static_cast<size_t>(span.query_start) + safe_row / a.heads) * a.heads + safe_row % a.heads;
    const unsigned int my_position = position_of(safe_row);
    const bool causal = a.causal != 0;

    // Keys the workgroup visits, and how far this wave's rows see.
    const unsigned long long group_last = first_row + kRows - 1 < rows ? first_row + kRows - 1 : rows - 1;
    unsigned int key_end = keys;
    if (causal) {
        const unsigned int reach = position_of(group_last) + 1u;
        key_end = key_end < reach ? key_end : reach;
    }
    // With key splits this workgroup takes one share of the tiles; a share may be empty.
    unsigned int first_tile = 0, tiles = (key_end + kKeys - 1) / kKeys;
    if (splits > 1) {
        const unsigned int share = (tiles + splits - 1) / splits;
        first_tile = split * share;
        tiles = tiles < first_tile + share ? tiles : first_tile + share;
    }
    const unsigned long long wave_first = first_row + 16u * wave;
    const bool wave_live = wave_first < rows;
    const unsigned long long wave_last = wave_first + 15u < rows ? wave_first + 15u : rows - 1;
    unsigned int wave_end = 0;  // keys before this take part for some row of the wave
    if (wave_live) {
        wave_end = keys;
        if (causal) {
            const unsigned int reach = position_of(wave_last) + 1u;
            wave_end = wave_end < reach ? wave_end : reach;
        }
    }
    wave_end = __builtin_amdgcn_readfirstlane(wave_end);
    const unsigned int wave_low = __builtin_amdgcn_readfirstlane(wave_live ? position_of(wave_first) : 0u);

    // Q^T: lane (row, g) holds dims 32 s + 8 g .. + 8 of its row for every step s.
    const Half half{};
    uint4 q[kSteps - kParkedSteps];  // steps kParkedSteps and up
    unsigned char* parked = lds + 2 * kStageBytes + wave * (kParkedSteps * 1024) + 16u * lane;
    {
        const unsigned char* latent_row = static_cast<const unsigned char*>(a.latent_queries) + flat * latent_row_bytes + 16u * g;
        const unsigned char* positional_row = static_cast<const unsigned char*>(a.positional_queries) + flat * positional_row_bytes + 16u * g;
#pragma unroll
        for (int s = 0; s < kSteps; ++s) {
            // (ANY: the lane's chunk of the step, 4 s + g of the latent part or 4 (s - 16) + g of the positional one, may lie past the row)
            const bool real = !ANY || (s < kLatentSteps ? 4u * s + g < latent_chunks : 4u * (s - kLatentSteps) + g < positional_chunks);
            uint4 bits = make_uint4(0, 0, 0, 0);
            if (real)
                bits = s < kLatentSteps ? *reinterpret_cast<const uint4*>(latent_row + 64 * s)
                                        : *reinterpret_cast<const uint4*>(positional_row + 64 * (s - kLatentSteps));
            if (!row_valid) bits = make_uint4(0, 0, 0, 0);
            if (s < kParkedSteps)
                *reinterpret_cast<uint4*>(parked + 1024 * s) = bits;
            else
                q[s - kParkedSteps] = bits;
        }
    }

    // Loading a tile: wave w brings latent rows w, w + 8, w + 16, w + 24 (one 1 KiB instruction each) and, for
    // w < 4, the positional parts of rows 8 w .. 8 w + 7 (lane l: row 8 w + l / 8, chunk position l % 8).
    const unsigned char* latent_cache = static_cast<const unsigned char*>(a.latent_cache);
    const unsigned char* positional_cache = static_cast<const unsigned char*>(a.positional_cache);
    const unsigned int positional_row = 8u * wave + (lane >> 3);
    auto key_of = [&](unsigned int tile, unsigned int row) __attribute__((always_inline)) {
        const unsigned int key = tile * kKeys + row;
        return key < keys ? key : keys - 1u;  // rows past the end re-read the last key and are masked
    };
    // A key's entry in the sequence's pages and its place in the page; a power-of-two page size takes the shift.
    const int page_shift = a.page_shift;
    auto entry_of = [&](unsigned int key) __attribute__((always_inline)) { return page_shift >= 0 ? key >> page_shift : key / a.page_size; };
    auto place_of = [&](unsigned int key) __attribute__((always_inline)) {
        return page_shift >= 0 ? key & (a.page_size - 1u) : key % a.page_size;
    };
    auto lookup = [&](unsigned int tile) __attribute__((always_inline)) {
        TilePages<FORM> pages;
        if constexpr (IN_PAGE) {
            // (the tile's first key is one of the sequence's: tile < tiles)
            pages.latent[0] = read_raw_page_uniform<FORM>(a.pages, static_cast<size_t>(span.page_start) + ((tile * kKeys) >> page_shift));
            return pages;
        }
#pragma unroll
        for (int i = 0; i < 4; ++i)
            pages.latent[i] = read_raw_page_uniform<FORM>(a.pages, static_cast<size_t>(span.page_start) + entry_of(key_of(tile, wave + 8u * i)));
        pages.positional = 0;
        if (wave < 4) pages.positional = read_raw_page<FORM>(a.pages, static_cast<size_t>(span.page_start) + entry_of(key_of(tile, positional_row)));
        return pages;
    };
    // A key behind a bad page id is read as zeros; the status word tells the caller.
    // In pieces, so that a tile's iteration can spread them between its first score products: piece 0-3 one latent
    // row each, piece 4 the positional parts.
    const unsigned int positional_chunk = 16u * ((lane & 7u) ^ (positional_row & 7u));
    // Rows w and w + 16 of a tile permute their chunks alike, and so do w + 8 and w + 24.
    const unsigned int lane_chunk[2] = {16u * (lane ^ chunk_flip(wave & 15u)), 16u * (lane ^ chunk_flip((wave + 8u) & 15u))};
    // IN_PAGE: where the tile that is being loaded starts in either cache and the last of its rows that holds a key of
    // the sequence (rows past it re-read it and are masked): the same for every lane, worked out once a tile (locate_tile, from the id that lookup asked for a tile earlier) in scalar arithmetic.
    struct TileSource {
        const unsigned char* latent;
        const unsigned char* positional;
        unsigned int last;
    };
    TileSource source = {};
    auto locate_tile = [&](unsigned int tile, const TilePages<FORM>& pages) __attribute__((always_inline)) {
        if constexpr (IN_PAGE) {
            const unsigned long long page = static_cast<unsigned long long>(pages.latent[0]);
            unsigned int low = static_cast<unsigned int>(page);
            // An id outside the cache is reported and replaced by page 0 (what that holds is not used by a caller that
            // checks the status word), so that the loads need no test of their own.
            const bool outside = static_cast<unsigned int>(page >> 32) != 0u || low >= a.cache_pages;
            if (outside && lane == 0) report_index_error(a.status);
            low = __builtin_amdgcn_readfirstlane(outside ? 0u : low);  // (said to be the same for every lane: scalar arithmetic from here on)
            const unsigned int first_key = tile * kKeys;
            const size_t slot = (static_cast<size_t>(low) << page_shift) + (first_key & (a.page_size - 1u));
            source.last = keys - 1u - first_key;
            source.latent = latent_cache + slot * latent_row_bytes;
            source.positional = positional_cache + slot * positional_row_bytes;
        }
    };
    const unsigned int lds_start = static_cast<unsigned int>(reinterpret_cast<__UINTPTR_TYPE__>((lds_words_t)lds));  // the byte address M0 takes
    // (stage_at: the stage's byte offset from there)
    auto issue_piece = [&](int piece, unsigned int tile, const TilePages<FORM>& pages, unsigned char* __restrict__ stage, unsigned int stage_at)
                           __attribute__((always_inline)) {
        if constexpr (IN_PAGE) {
            const TileSource& from = source;
            if (piece < 4) {
                const unsigned int row = wave + 8u * piece, kept = row < from.last ? row : from.last;
                if (!ANY || lane_chunk[piece & 1] < 16u * latent_chunks)
                    load_to_lds(from.latent + kept * latent_row_bytes, lane_chunk[piece & 1], lds_start + stage_at + row * kLatentRowBytes);
            } else if (wave < 4) {
                const unsigned int kept = positional_row < from.last ? positional_row : from.last;
                if (!ANY || positional_chunk < 16u * positional_chunks)
                    load_to_lds(from.positional, kept * positional_row_bytes + positional_chunk,
                                lds_start + stage_at + kLatentTileBytes + 8u * wave * kPositionalRowBytes);
            }
            return;
        }
        if (piece < 4) {
            const int i = piece;
            const unsigned int row = wave + 8u * i;
            const unsigned long long page = static_cast<unsigned long long>(pages.latent[i]);
            unsigned char* dest = stage + row * kLatentRowBytes;
            if (page < static_cast<unsigned long long>(a.cache_pages)) {
                const size_t slot = static_cast<size_t>(page) * a.page_size + place_of(key_of(tile, row));
                if (!ANY || lane_chunk[i & 1] < 16u * latent_chunks) load_to_lds(latent_cache + slot * latent_row_bytes, lane_chunk[i & 1], dest);
            } else {
                if (lane == 0) report_index_error(a.status);
                *reinterpret_cast<uint4*>(dest + 16u * lane) = make_uint4(0, 0, 0, 0);
            }
        } else if (wave < 4) {
            const unsigned long long page = static_cast<unsigned long long>(pages.positional);
            unsigned char* dest = stage + kLatentTileBytes + 8u * wave * kPositionalRowBytes;
            if (page < static_cast<unsigned long long>(a.cache_pages)) {
                const size_t slot = static_cast<size_t>(page) * a.page_size + place_of(key_of(tile, positional_row));
                // (the lane's chunk is made opaque here: added to the cache's address ahead of the loop it would be a
                // 64-bit value per lane to keep)
                unsigned int chunk = positional_chunk;
                asm volatile("" : "+v"(chunk));
                const unsigned char* source = positional_cache + (slot * positional_row_bytes + chunk);
                if (!ANY || positional_chunk < 16u * positional_chunks) load_to_lds(source, dest);
            } else {
                report_index_error(a.status);
                *reinterpret_cast<uint4*>(dest + 16u * lane) = make_uint4(0, 0, 0, 0);
            }
        }
    };

    auto issue = [&](unsigned int tile, const TilePages<FORM>& pages, unsigned char* __restrict__ stage, unsigned int stage_at) __attribute__((always_inline)) {
        locate_tile(tile, pages);
#pragma unroll
        for (int piece = 0; piece < 5; ++piece) issue_piece(piece, tile, pages, stage, stage_at);
    };

    // Read offsets.  Score operand of step s, 16-key half t: row 16 t + column, chunk (4 s + g) ^ flip.  Transposed
    // operand of dim block db: rows 4 g + column / 4 (and 16 more), chunk (2 db + (column & 3) / 2) ^ flip, the
    // low or high 8 bytes of it by column & 1.  A flip touches the low four bits of a chunk index only, so the
    // offsets repeat every 256 bytes of a row: four registers serve the score operands, eight the transposed ones,
    // and the rest of an address is an immediate.
    unsigned int score_at[4], positional_at[2], value_at[8];
    {
        const unsigned int score_row = column * kLatentRowBytes, score_flip = chunk_flip(column);
#pragma unroll
        for (unsigned int i = 0; i < 4; ++i) score_at[i] = score_row + 16u * ((4u * i + g) ^ score_flip);
        const unsigned int positional_row_at = kLatentTileBytes + column * kPositionalRowBytes, positional_flip = column & 7u;
#pragma unroll
        for (unsigned int i = 0; i < 2; ++i) positional_at[i] = positional_row_at + 16u * ((4u * i + g) ^ positional_flip);
        const unsigned int value_key = 4u * g + (column >> 2);
        const unsigned int value_row = value_key * kLatentRowBytes + 8u * (column & 1u);
        const unsigned int value_flip = chunk_flip(value_key), value_chunk = (column & 3u) >> 1;
#pragma unroll
        for (unsigned int i = 0; i < 8; ++i) value_at[i] = value_row + 16u * ((2u * i + value_chunk) ^ value_flip);
    }

    f32x4_t out[kDimBlocks];  // lane (row, g): dims 16 db + 4 g + r of its row
#pragma unroll
    for (int db = 0; db < kDimBlocks; ++db) out[db] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
    float reference = -INFINITY, running_sum = 0.0f;  // the sum of this lane's keys only
    const float scale_log2e = a.scale * kLog2e;

    auto fold = [&](unsigned int tile, const unsigned char* __restrict__ stage, auto&& between) __attribute__((always_inline)) {
        const unsigned int key0 = tile * kKeys;
        f32x4_t s[2] = {f32x4_t{0.0f, 0.0f, 0.0f, 0.0f}, f32x4_t{0.0f, 0.0f, 0.0f, 0.0f}};
        // The operands of a step are read a step before its products (two sets taking turns), and the order is
        // pinned: left to itself the compiler, short of registers, reads each operand right before its use and the
        // matrix core waits out every LDS round trip.
        uint4 operand[2][2], parked_q[2];
        auto read_step = [&](int step, int slot) __attribute__((always_inline)) {
            const unsigned char* at = step < kLatentSteps ? stage + score_at[step & 3] + 256 * (step >> 2) : stage + positional_at[step & 1];
            const int half_stride = step < kLatentSteps ? 16 * kLatentRowBytes : 16 * kPositionalRowBytes;
            operand[slot][0] = *reinterpret_cast<const uint4*>(at);
            operand[slot][1] = *reinterpret_cast<const uint4*>(at + half_stride);
            if (step < kParkedSteps) parked_q[slot] = *reinterpret_cast<const uint4*>(parked + 1024 * step);
        };
        read_step(0, 0);
#pragma unroll
        for (int step = 0; step < kSteps; ++step) {
            if (step + 1 < kSteps) read_step(step + 1, (step + 1) % 2);
            __builtin_amdgcn_sched_barrier(0);
            const uint4 mine = step < kParkedSteps ? parked_q[step % 2] : q[step < kParkedSteps ? 0 : step - kParkedSteps];
            s[0] = mma(half, operand[step % 2][0], mine, s[0]);
            s[1] = mma(half, operand[step % 2][1], mine, s[1]);
            between(step);  // the caller's paging arithmetic and loads, while the products run
            __builtin_amdgcn_sched_barrier(0);
        }
        // Register r of half t is key key0 + 16 t + 4 g + r against the lane's row.
        float x[8];
        const bool edge = key0 + kKeys > keys || (causal && key0 + kKeys - 1u > wave_low);
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int r = 0; r < 4; ++r) x[4 * t + r] = s[t][r] * scale_log2e;
        if (edge) {
            // (a statement the compiler may not run ahead of the test: it would otherwise turn the branch into eight
            // tests and selects on every tile, and a wave's instruction count is what bounds its time)
            asm volatile("s_nop 0");
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const unsigned int key = key0 + 16u * t + 4u * g + r;
                    if (key >= keys || (causal && key > my_position)) x[4 * t + r] = -INFINITY;
                }
        }
        float largest = fmaxf(fmaxf(fmaxf(x[0], x[1]), fmaxf(x[2], x[3])), fmaxf(fmaxf(x[4], x[5]), fmaxf(x[6], x[7])));
        largest = across_groups_max(largest);  // the four lanes of a row agree from here on
        if (__any(largest > reference + kMaxLag || (reference == -INFINITY && largest != -INFINITY))) {
            const float moved = fmaxf(reference, largest);
            const float base = moved == -INFINITY ? 0.0f : moved;
            const float rescale = fast_exp2(reference - base);
            running_sum *= rescale;
#pragma unroll
            for (int db = 0; db < kDimBlocks; ++db)
#pragma unroll
                for (int r = 0; r < 4; ++r) out[db][r] *= rescale;
            reference = moved;
        }
        const float shift = reference == -INFINITY ? 0.0f : -reference;
        float p[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            p[i] = fast_exp2(x[i] + shift);
            running_sum += p[i];
        }
        // The weights, rounded as the value product takes them: slots 8 g .. 8 g + 3 are keys 4 g .. 4 g + 3, slots
        // 8 g + 4 .. 8 g + 7 keys 16 + 4 g .. 16 + 4 g + 3.
        const uint4 weights = make_uint4(pack_pair(half, p[0], p[1]), pack_pair(half, p[2], p[3]), pack_pair(half, p[4], p[5]),
                                         pack_pair(half, p[6], p[7]));
        // The transposed operands likewise, two dim blocks ahead (a ring of three).
        v4i16_t low[3], high[3];
        auto read_block = [&](int db, int slot) __attribute__((always_inline)) {
            const unsigned char* at = stage + value_at[db & 7] + 256 * (db >> 3);
            low[slot] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4_t)(at));
            high[slot] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4_t)(at + 16 * kLatentRowBytes));
        };
        read_block(0, 0);
        read_block(1, 1);
#pragma unroll
        for (int db = 0; db < kDimBlocks; ++db) {
            if (db + 2 < kDimBlocks) read_block(db + 2, (db + 2) % 3);
            __builtin_amdgcn_sched_barrier(0);
            const prefill::v8i16_t both = __builtin_shufflevector(low[db % 3], high[db % 3], 0, 1, 2, 3, 4, 5, 6, 7);
            out[db] = mma(half, __builtin_bit_cast(uint4, both), weights, out[db]);
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    if (first_tile < tiles) {
        TilePages<FORM> pages = lookup(first_tile);
        issue(first_tile, pages, lds + (first_tile & 1u) * kStageBytes, (first_tile & 1u) * kStageBytes);
        if (first_tile + 1 < tiles) pages = lookup(first_tile + 1);
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
        __syncthreads();
        for (unsigned int tile = first_tile; tile < tiles; ++tile) {
            unsigned char* stage = lds + (tile & 1u) * kStageBytes;
            unsigned char* other = lds + ((tile & 1u) ^ 1u) * kStageBytes;
            const unsigned int other_at = ((tile & 1u) ^ 1u) * kStageBytes;
            // The next tile's loads go out one piece after each of the first score steps, the page ids of the tile
            // after it once those have been used: address arithmetic in the shadow of the products.
            auto between = [&](int step) __attribute__((always_inline)) {
                if (step < 5) {
                    if constexpr (IN_PAGE) {
                        // (past the last tile: the last one again, into the stage nobody reads any more, so that a piece
                        // carries no test; `pages` then still holds the last tile's id)
                        const unsigned int wanted = tile + 1 < tiles ? tile + 1 : tiles - 1u;
                        if (step == 0) locate_tile(wanted, pages);
                        issue_piece(step, wanted, pages, other, other_at);
                    } else if (tile + 1 < tiles) {
                        issue_piece(step, tile + 1, pages, other, other_at);
                    }
                } else if (step == 6) {
                    if (tile + 2 < tiles) pages = lookup(tile + 2);
                }
            };
            if (tile * kKeys < wave_end) {
                fold(tile, stage, between);
            } else {
#pragma unroll
                for (int step = 0; step < 7; ++step) between(step);
            }
            __builtin_amdgcn_s_waitcnt(0x0F70);  // this wave's loads have landed
            __syncthreads();                     // and everyone has finished reading
        }
    }

    // Normalise and store; a row that sees no key stays zero and has a log-sum-exp of -inf.
    const float sum = across_groups_sum(running_sum);
    const float inverse = sum > 0.0f ? 1.0f / sum : 0.0f;
    if (row_valid && splits > 1) {
        const size_t slot = static_cast<size_t>(split) * a.tokens * a.heads + flat;
        float* row = a.partial_out + slot * kLatent + 4u * g;
#pragma unroll
        for (int db = 0; db < kDimBlocks; ++db)
            *reinterpret_cast<float4*>(row + 16 * db) =
                make_float4(out[db][0] * inverse, out[db][1] * inverse, out[db][2] * inverse, out[db][3] * inverse);
        if (g == 0) a.partial_lse[slot] = sum > 0.0f ? reference + fast_log2(sum) : -INFINITY;
    } else if (row_valid) {
        unsigned char* row = static_cast<unsigned char*>(a.output) + flat * latent_row_bytes + 8u * g;
#pragma unroll
        for (int db = 0; db < kDimBlocks; ++db) {
            // (a test a dim block, not a way out of the loop: a loop that may end early is not unrolled, and an output
            // indexed by a variable lives in scratch memory for the whole kernel)
            if (ANY && 2u * db >= latent_chunks) continue;  // dims past the latent width
            uint2 packed;
            packed.x = pack_pair(half, out[db][0] * inverse, out[db][1] * inverse);
            packed.y = pack_pair(half, out[db][2] * inverse, out[db][3] * inverse);
            *reinterpret_cast<uint2*>(row + 32 * db) = packed;
        }
        if (a.lse != nullptr && g == 0) a.lse[flat] = sum > 0.0f ? reference + fast_log2(sum) : -INFINITY;
    }
}

// Merges the shares of a row: out = sum_s 2^(lse_s - m) o_s / sum_s 2^(lse_s - m), lse = m + log2 of that sum
// (the merge of the reference's own split kernels, kernel_plan/source/mla.rs:497-560).  One wave per (token, head)
// row, lane l dims 8 l .. 8 l + 7, kCombineBlocks workgroups of four waves to a row tile, so that a tile's 128 rows
// are merged side by side rather than one after another; a row whose shares are all empty stays zero with a
// log-sum-exp of -inf.  Lane s holds share s's weight (the host allows 64 shares at most), and the shares' values
// are asked for four at a time.
constexpr unsigned int kCombineBlocks = kRows / 4;

template <class Half, int FORM, bool ANY>
SINGE_DEVICE void latent_combine_rows(const LatentAttentionArgs& a) {
    const unsigned int wave = threadIdx.x >> 6, lane = threadIdx.x & 63u;
    // Workgroups map to (sequence, row tile) as in the attention kernel, so only rows that kernel wrote are read.
    unsigned int sequence, row_tile;
    if (!find_unit<FORM>(a, blockIdx.x / kCombineBlocks, sequence, row_tile)) return;
    const SequenceSpan span = load_span<FORM>(sequence, a.query_offsets, a.page_offsets, a.last_page_lengths, nullptr, a.tokens,
                                              a.page_table, a.page_size);
    if (!span.valid) return;  // the attention kernel has reported it
    const unsigned long long rows = static_cast<unsigned long long>(span.queries) * a.heads;
    const size_t rows_total = static_cast<size_t>(a.tokens) * a.heads;
    const unsigned long long local = static_cast<unsigned long long>(row_tile) * kRows + 4u * (blockIdx.x % kCombineBlocks) + wave;
    if (local >= rows) return;
    const size_t row = (static_cast<size_t>(span.query_start) + local / a.heads) * a.heads + local % a.heads;
    const float mine = lane < a.splits ? a.partial_lse[lane * rows_total + row] : -INFINITY;
    float largest = mine;
#pragma unroll
    for (int step = 32; step >= 1; step >>= 1) largest = fmaxf(largest, __shfl_xor(largest, step, 64));
    // An empty share weighs nothing (its values are zeros).
    const float weight = mine == -INFINITY ? 0.0f : fast_exp2(mine - largest);
    float total = weight;
#pragma unroll
    for (int step = 32; step >= 1; step >>= 1) total += __shfl_xor(total, step, 64);
    float acc[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
    const float* part = a.partial_out + row * kLatent + 8u * lane;
    const size_t share_stride = rows_total * kLatent;
    auto fold = [&](float w, const float4& low, const float4& high) __attribute__((always_inline)) {
        acc[0] = fmaf(w, low.x, acc[0]); acc[1] = fmaf(w, low.y, acc[1]);
        acc[2] = fmaf(w, low.z, acc[2]); acc[3] = fmaf(w, low.w, acc[3]);
        acc[4] = fmaf(w, high.x, acc[4]); acc[5] = fmaf(w, high.y, acc[5]);
        acc[6] = fmaf(w, high.z, acc[6]); acc[7] = fmaf(w, high.w, acc[7]);
    };
    unsigned int s = 0;
    for (; s + 4 <= a.splits; s += 4) {
        float4 low[4], high[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float* from = part + (s + i) * share_stride;
            low[i] = *reinterpret_cast<const float4*>(from);
            high[i] = *reinterpret_cast<const float4*>(from + 4);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) fold(__shfl(weight, s + i, 64), low[i], high[i]);
    }
    for (; s < a.splits; ++s) {
        const float* from = part + s * share_stride;
        fold(__shfl(weight, s, 64), *reinterpret_cast<const float4*>(from), *reinterpret_cast<const float4*>(from + 4));
    }
    const float inverse = total > 0.0f ? 1.0f / total : 0.0f;
    const Half half{};
    uint4 packed;
    packed.x = pack_pair(half, acc[0] * inverse, acc[1] * inverse);
    packed.y = pack_pair(half, acc[2] * inverse, acc[3] * inverse);
    packed.z = pack_pair(half, acc[4] * inverse, acc[5] * inverse);
    packed.w = pack_pair(half, acc[6] * inverse, acc[7] * inverse);
    // (a share's rows are 512 values apart whatever the latent width; the output's rows are as wide as the problem's)
    if (!ANY || 8u * lane < a.latent_dim)
        *reinterpret_cast<uint4*>(static_cast<unsigned char*>(a.output) + row * (ANY ? 2u * a.latent_dim : static_cast<unsigned int>(kLatentRowBytes)) + 16u * lane) = packed;
    if (a.lse != nullptr && lane == 0) a.lse[row] = total > 0.0f ? largest + fast_log2(total) : -INFINITY;
}

template <class Half, bool ANY>
SINGE_DEVICE void latent_tile_body(const LatentAttentionArgs& a, unsigned char* lds) {
    const bool in_page = a.page_shift >= 5;  // a power of two of at least a tile's 32 keys
    if (a.wide_index) {
        if (in_page) latent_tile_rows<Half, kCsrI64, ANY, true>(a, lds);
        else latent_tile_rows<Half, kCsrI64, ANY, false>(a, lds);
    } else {
        if (in_page) latent_tile_rows<Half, kCsrI32, ANY, true>(a, lds);
        else latent_tile_rows<Half, kCsrI32, ANY, false>(a, lds);
    }
}

}  // namespace latent_mfma

#define SINGE_LATENT_MFMA_KERNEL(NAME, HALF, ANY)                                                         \
    extern "C" __global__ __launch_bounds__(64 * latent_mfma::kWaves, 2) void NAME(LatentAttentionArgs args) { \
        __shared__ __attribute__((aligned(1024))) unsigned char latent_lds[latent_mfma::kLdsBytes];         \
        latent_mfma::latent_tile_body<prefill::HALF, ANY>(args, latent_lds);                               \
    }

#define SINGE_LATENT_COMBINE_KERNEL(NAME, HALF, ANY)                                             \
    extern "C" __global__ __launch_bounds__(256) void NAME(LatentAttentionArgs args) {          \
        if (args.wide_index)                                                                    \
            latent_mfma::latent_combine_rows<prefill::HALF, kCsrI64, ANY>(args);                \
        else                                                                                    \
            latent_mfma::latent_combine_rows<prefill::HALF, kCsrI32, ANY>(args);                \
    }

SINGE_LATENT_COMBINE_KERNEL(singe_paged_mla_attention_combine_bf16, Bf16, false)
SINGE_LATENT_COMBINE_KERNEL(singe_paged_mla_attention_combine_f16, F16, false)
SINGE_LATENT_MFMA_KERNEL(singe_paged_mla_attention_bf16_l512_p64, Bf16, false)
SINGE_LATENT_MFMA_KERNEL(singe_paged_mla_attention_f16_l512_p64, F16, false)
// Any latent width that is a multiple of 32 up to 512 with a positional width that is a multiple of 8 up to 64.
SINGE_LATENT_MFMA_KERNEL(singe_paged_mla_attention_bf16_any, Bf16, true)
SINGE_LATENT_MFMA_KERNEL(singe_paged_mla_attention_f16_any, F16, true)
SINGE_LATENT_COMBINE_KERNEL(singe_paged_mla_attention_combine_bf16_any, Bf16, true)
SINGE_LATENT_COMBINE_KERNEL(singe_paged_mla_attention_combine_f16_any, F16, true)
