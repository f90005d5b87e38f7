// Reading and checking one sequence's paging values on the device, shared by the paged kernels.
// Paging arrives as FlashInfer CSR vectors of i32 or i64 (singe/src/tensor/neural.rs:409-457), or as the
// block table of the singe-kernel surface: u32 table rows plus i32 per-sequence query offsets, query
// lengths and key lengths (singe-kernel/src/cpu/attention.rs:1248-1276).
#pragma once

#include "common.hip.h"

enum : int { kCsrI32 = 0, kCsrI64 = 1, kTable = 2 };

template <int FORM>
SINGE_DEVICE long long read_index(const void* values, size_t at) {
    if constexpr (FORM == kCsrI64)
        return static_cast<const long long*>(values)[at];
    else
        return static_cast<long long>(static_cast<const int*>(values)[at]);
}

template <int FORM>
SINGE_DEVICE unsigned long long read_page(const void* pages, size_t at) {
    if constexpr (FORM == kTable)
        return static_cast<const unsigned int*>(pages)[at];
    else
        return static_cast<unsigned long long>(read_index<FORM>(pages, at));  // negative ids wrap above any cache
}

// A page id as it sits in memory, and the load of one with no arithmetic on the result (a consumer that
// wants to keep the load in flight widens it later: static_cast<unsigned long long> sign-extends the CSR
// forms, so negative ids wrap above any cache, and zero-extends a block table's u32).
template <int FORM> struct RawPageType { typedef int type; };
template <> struct RawPageType<kCsrI64> { typedef long long type; };
template <> struct RawPageType<kTable> { typedef unsigned int type; };
template <int FORM> using RawPage = typename RawPageType<FORM>::type;

template <int FORM>
SINGE_DEVICE RawPage<FORM> read_raw_page(const void* pages, size_t at) {
    return static_cast<const RawPage<FORM>*>(pages)[at];
}

// The same load from an address every lane shares, through the constant address space (paging vectors are
// not written while a kernel that reads them runs), which lets it run on the scalar unit.
template <int FORM>
SINGE_DEVICE RawPage<FORM> read_raw_page_uniform(const void* pages, size_t at) {
    typedef const RawPage<FORM> __attribute__((address_space(4))) * constant_pages_t;
    return ((constant_pages_t)pages)[at];
}

struct SequenceSpan {
    long long query_start;  // first token of the sequence in the packed queries
    long long page_start;   // first entry of the sequence in `pages`
    unsigned int queries;
    unsigned int keys;
    bool valid;             // false: some value would address outside the queries or the page table
};

// The checks of paged_attention.rs:210-238 (CPU: spec/neural/attention.rs:372-406): offsets monotone
// inside [0, tokens] / [0, page_table], last_page_length in [0, page_size] unless the sequence has no
// pages.  keys = (page_count - 1) * page_size + last_page_length (paged_attention.rs:256).
template <int FORM>
SINGE_DEVICE SequenceSpan load_span(unsigned int sequence, const void* query_offsets, const void* page_offsets,
                                    const void* last_page_lengths, const void* query_lengths, unsigned int tokens,
                                    unsigned int page_table, unsigned int page_size) {
    SequenceSpan span;
    long long query_count, key_count;
    if constexpr (FORM == kTable) {
        span.query_start = read_index<FORM>(query_offsets, sequence);
        query_count = read_index<FORM>(query_lengths, sequence);
        key_count = read_index<FORM>(last_page_lengths, sequence);
        span.page_start = static_cast<long long>(sequence) * page_table;
        span.valid = !(span.query_start < 0 || query_count < 0 || span.query_start + query_count > static_cast<long long>(tokens) ||
                       key_count < 0 || key_count > static_cast<long long>(page_table) * page_size);
    } else {
        span.query_start = read_index<FORM>(query_offsets, sequence);
        const long long query_end = read_index<FORM>(query_offsets, sequence + 1);
        span.page_start = read_index<FORM>(page_offsets, sequence);
        const long long page_end = read_index<FORM>(page_offsets, sequence + 1);
        const long long last_length = read_index<FORM>(last_page_lengths, sequence);
        span.valid = !(span.query_start < 0 || query_end < span.query_start || query_end > static_cast<long long>(tokens) ||
                       span.page_start < 0 || page_end < span.page_start || page_end > static_cast<long long>(page_table) ||
                       (page_end > span.page_start && (last_length < 0 || last_length > static_cast<long long>(page_size))));
        query_count = query_end - span.query_start;
        const long long page_count = page_end - span.page_start;
        key_count = page_count == 0 ? 0 : (page_count - 1) * page_size + last_length;
    }
    span.queries = span.valid ? static_cast<unsigned int>(query_count) : 0u;
    span.keys = span.valid ? static_cast<unsigned int>(key_count) : 0u;
    return span;
}

// Workgroup units in sequence order: sequence s owns max(1, ceil(rows_s * heads / rows_per_unit)) of them (one even
// without rows, so that its paging values are checked), rows_s being its query count (from the offsets, or from
// `query_lengths` in the block-table form; counts that make no sense are held to [0, tokens] and their sequence's
// checks report them).  Every wave finds the owner of `unit` for itself by a prefix sum over the sequences, 64 at a
// time; false for a unit past the last sequence's.  A grid of tokens * heads / rows_per_unit + sequences units
// covers them all.
template <int FORM>
SINGE_DEVICE bool find_row_unit(const void* query_offsets, const void* query_lengths, unsigned int sequences, unsigned int tokens,
                                unsigned int heads, unsigned int rows_per_unit, unsigned int unit, unsigned int& sequence,
                                unsigned int& unit_of_sequence) {
    const unsigned int lane = threadIdx.x & 63u;
    unsigned int base = 0;
    for (unsigned int first = 0; first < sequences; first += 64u) {
        const unsigned int s = first + lane;
        unsigned int mine = 0;
        if (s < sequences) {
            long long count;
            if constexpr (FORM == kTable) count = read_index<FORM>(query_lengths, s);
            else count = read_index<FORM>(query_offsets, s + 1) - read_index<FORM>(query_offsets, s);
            count = count < 0 ? 0 : count > static_cast<long long>(tokens) ? static_cast<long long>(tokens) : count;
            const unsigned long long units = (static_cast<unsigned long long>(count) * heads + rows_per_unit - 1) / rows_per_unit;
            mine = units == 0 ? 1u : static_cast<unsigned int>(units);
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
            unit_of_sequence = unit - (base + owner_through - owner_mine);
            return true;
        }
        base += total;
    }
    return false;
}
