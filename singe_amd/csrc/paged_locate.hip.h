// Which (sequence, kv head, row tile, key split) a workgroup of the paged attention kernels works on.
#pragma once

#include "kernel_args.h"
#include "paging.hip.h"

namespace {

constexpr unsigned int kNoPage = 0xFFFFFFFFu;  // a table entry outside the cache: reported, never read through

// Workgroup id -> (unit = sequence * kv_heads + kv head, row tile, key split); false for ids past the units.
// Workgroup i runs on XCD i % 8: the row tiles of one (sequence, kv head) share an XCD and its L2.
//
// Plain form (a.compact == 0; calls where no sequence can have more than one row tile, decoding above all): the grid
// covers every sequence's longest possible run of rows.  Within an XCD the order is band by band of 32 row tiles:
// every unit's tiles 0 .. 31 (a unit's side by side, walking its keys together), then every unit's tiles 32 .. 63,
// and so on.  The splits of one (unit, row tile) are neighbours.
//
// Compact form (a.compact != 0): the row tiles of all sequences form one list in sequence order (or longest sequence
// first, see a.longest_first), sequence s owning
// max(1, ceil(queries_s * groups / ROWS)) of them (ROWS: the rows of a workgroup, 128 or 256) (one even without queries, so that its paging values are checked),
// and the grid covers a bound on the list's length instead of sequences x the longest possible sequence; a workgroup
// finds its entry by a prefix sum over the sequences' query counts, 64 sequences at a time.  The list is cut into
// bands of 32 entries; (band, kv head) pairs go round the XCDs, so a band's tiles for one kv head are neighbours on
// one XCD and walk their keys side by side.
// a.longest_first (at most 64 sequences, several row tiles each: chunks of a prefill): the compact list takes the
// sequences longest first (by pages held, ties by index), so that the workgroups with the most keys to walk start
// first and the short ones fill the chip's last round.  Lane s learns how many list entries come before sequence s's
// own (`mine` of them) in that order; any values give some order, and a sequence's own checks report the ones that
// make no sense.  (Decode-shaped calls keep the sequences' own order: their workgroups are short, and the two loads
// and the ranking in front of everything else cost them more than the order gains: 62 -> 70 us on the decode
// benchmark's shape.)
template <int FORM>
SINGE_DEVICE unsigned int entries_before_longest_first(const PagedAttentionArgs& a, unsigned int mine) {
    const unsigned int s = threadIdx.x & 63u;
    unsigned int held = 0;
    if (s < a.sequences) {
        long long count;
        if constexpr (FORM == kTable) count = read_index<FORM>(a.last_page_lengths, s);  // the block-table form's key counts
        else count = read_index<FORM>(a.page_offsets, s + 1) - read_index<FORM>(a.page_offsets, s);
        held = count < 0 ? 0u : count > 0x7fffffffll ? 0x7fffffffu : static_cast<unsigned int>(count);
    }
    unsigned int before = 0;
    for (unsigned int other = 0; other < a.sequences; ++other) {
        const unsigned int other_held = __builtin_amdgcn_readlane(held, other), other_mine = __builtin_amdgcn_readlane(mine, other);
        if (other_held > held || (other_held == held && other < s)) before += other_mine;
    }
    return before;
}

template <int FORM, unsigned int ROWS>
SINGE_DEVICE bool locate(const PagedAttentionArgs& a, unsigned int& unit, unsigned int& row_tile, unsigned int& split) {
    constexpr unsigned int kBand = 32;
    const unsigned int xcd = blockIdx.x & 7u;
    unsigned int within = blockIdx.x >> 3;
    split = within % a.splits;
    within /= a.splits;
    if (a.compact != 0) {
        const unsigned int bands = (a.row_tiles + kBand - 1) / kBand;
        const unsigned int pair = xcd + 8u * (within / kBand);
        if (pair >= a.kv_heads * bands) return false;
        const unsigned int kv_head = pair % a.kv_heads, entry = (pair / a.kv_heads) * kBand + within % kBand;
        if (entry >= a.row_tiles) return false;
        const unsigned int lane = threadIdx.x & 63u, groups = a.heads / a.kv_heads;
        auto tiles_of = [&](unsigned int s) __attribute__((always_inline)) {
            long long count;
            if constexpr (FORM == kTable) count = read_index<FORM>(a.query_lengths, s);
            else count = read_index<FORM>(a.query_offsets, s + 1) - read_index<FORM>(a.query_offsets, s);
            count = count < 0 ? 0 : count > static_cast<long long>(a.tokens) ? static_cast<long long>(a.tokens) : count;
            const unsigned long long tiles = (static_cast<unsigned long long>(count) * groups + ROWS - 1) / ROWS;
            return tiles == 0 ? 1u : static_cast<unsigned int>(tiles);
        };
        if (a.longest_first != 0) {
            const unsigned int mine = lane < a.sequences ? tiles_of(lane) : 0u;
            const unsigned int before = entries_before_longest_first<FORM>(a, mine);
            const unsigned long long holds = __ballot(entry >= before && entry - before < mine);
            if (holds == 0) return false;
            const unsigned int owner = static_cast<unsigned int>(__builtin_ctzll(holds));
            unit = owner * a.kv_heads + kv_head;
            row_tile = entry - __shfl(before, owner, 64);
            return true;
        }
        unsigned int base = 0;
        for (unsigned int first = 0; first < a.sequences; first += 64u) {
            const unsigned int s = first + lane;
            const unsigned int mine = s < a.sequences ? tiles_of(s) : 0u;
            unsigned int through = mine;  // inclusive prefix sum over the wave
#pragma unroll
            for (int step = 1; step < 64; step <<= 1) {
                const unsigned int below = __shfl_up(through, step, 64);
                if (lane >= static_cast<unsigned int>(step)) through += below;
            }
            const unsigned int total = __shfl(through, 63, 64);
            if (entry < base + total) {
                const unsigned long long holds = __ballot(entry < base + through);  // first lane whose range reaches the entry
                const unsigned int owner = static_cast<unsigned int>(__builtin_ctzll(holds));
                const unsigned int owner_through = __shfl(through, owner, 64), owner_mine = __shfl(mine, owner, 64);
                unit = (first + owner) * a.kv_heads + kv_head;
                row_tile = entry - (base + owner_through - owner_mine);
                return true;
            }
            base += total;
        }
        return false;
    }
    const unsigned int units_per_xcd = (a.sequences * a.kv_heads + 7u) / 8u;
    const unsigned int full_bands = a.row_tiles / kBand, band = within / (units_per_xcd * kBand);
    unsigned int local_unit;
    if (band < full_bands) {
        const unsigned int rest = within % (units_per_xcd * kBand);
        local_unit = rest / kBand;
        row_tile = band * kBand + rest % kBand;
    } else {
        const unsigned int rest = within - full_bands * units_per_xcd * kBand, tail = a.row_tiles - full_bands * kBand;
        local_unit = rest / tail;
        row_tile = full_bands * kBand + rest % tail;
    }
    unit = local_unit * 8u + xcd;
    return unit < a.sequences * a.kv_heads;
}

}  // namespace
