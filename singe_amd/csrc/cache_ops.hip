// The steps either side of paged attention in a decode layer:
//
//  * singe_rotary_cache_write_*: rotates queries and keys and appends keys and values to the paged cache in
//    one launch, the gfx950 counterpart of the reference's rotary_cache_write kernel
//    (singe/src/backend/cuda/kernel_plan/source/rotary_cache.rs:249-427): query [T, H, D], key / value
//    [T, G, D], angles cos / sin [T, D / 2], one (page, slot) per token, caches [P, S, G, D]; half-split
//    pairs (p, p + D / 2): first = a cos - b sin, second = b cos + a sin, after an optional RMS
//    normalisation with an optional per-element weight (rotary_cache.rs:92-185).
//  * singe_paging_indices: turns FlashInfer CSR paging (query offsets, page offsets, pages, last page
//    lengths) into per-sequence packed offsets, query lengths, key lengths and a dense page table
//    [sequences, width], the form block-table kernels read (kernel_plan/source/paged_attention.rs:325-398).
//
// Both are bound by memory traffic and small; sixteen lanes take one head.
#include "common.hip.h"
#include "kernel_args.h"
#include "paging.hip.h"

namespace cache_ops {

template <uint32_t ELEMENT>
struct Element;
template <>
struct Element<kElementF32> {
    typedef float type;
    static SINGE_DEVICE float load(const type* at) { return *at; }
    static SINGE_DEVICE void store(type* at, float value) { *at = value; }
};
template <>
struct Element<kElementBf16> {
    typedef unsigned short type;
    static SINGE_DEVICE float load(const type* at) { return __builtin_bit_cast(float, static_cast<unsigned int>(*at) << 16); }
    static SINGE_DEVICE void store(type* at, float value) { *at = f32_to_bf16_bits(value); }
};
template <>
struct Element<kElementF16> {
    typedef _Float16 type;
    static SINGE_DEVICE float load(const type* at) { return static_cast<float>(*at); }
    static SINGE_DEVICE void store(type* at, float value) { *at = static_cast<_Float16>(value); }
};

SINGE_DEVICE float table_value(const void* table, uint32_t table_type, size_t at) {
    if (table_type == kElementF32) return static_cast<const float*>(table)[at];
    if (table_type == kElementBf16) return Element<kElementBf16>::load(static_cast<const unsigned short*>(table) + at);
    return Element<kElementF16>::load(static_cast<const _Float16*>(table) + at);
}

// Rotates one head: sixteen lanes, lane `part` takes pairs part, part + 16, ...
template <class E>
SINGE_DEVICE void rotate_head(typename E::type* to, const typename E::type* from, const RotaryCacheArgs& a, size_t token,
                              unsigned int part, bool has_norm, float eps, const void* weight) {
    const unsigned int half = a.head_dim / 2;
    float scale = 1.0f;
    if (has_norm) {
        float squares = 0.0f;
        for (unsigned int pair = part; pair < half; pair += 16) {
            const float first = E::load(from + pair), second = E::load(from + pair + half);
            squares += first * first + second * second;
        }
#pragma unroll
        for (int step = 1; step < 16; step <<= 1) squares += __shfl_xor(squares, step, 16);
        scale = rsqrtf(squares / static_cast<float>(a.head_dim) + eps);
    }
    for (unsigned int pair = part; pair < half; pair += 16) {
        float first = E::load(from + pair), second = E::load(from + pair + half);
        if (has_norm) {
            first *= scale;
            second *= scale;
            if (weight != nullptr) {
                first *= E::load(static_cast<const typename E::type*>(weight) + pair);
                second *= E::load(static_cast<const typename E::type*>(weight) + pair + half);
            }
        }
        const float cosine = table_value(a.cos, a.table_type, token * half + pair);
        const float sine = table_value(a.sin, a.table_type, token * half + pair);
        E::store(to + pair, first * cosine - second * sine);
        E::store(to + pair + half, second * cosine + first * sine);
    }
}

template <uint32_t ELEMENT>
SINGE_DEVICE void rotary_cache_write_body(const RotaryCacheArgs& a) {
    typedef Element<ELEMENT> E;
    typedef typename E::type T;
    const unsigned int part = threadIdx.x & 15u;
    const unsigned long long item = static_cast<unsigned long long>(blockIdx.x) * (blockDim.x / 16) + (threadIdx.x >> 4);
    const unsigned int total_heads = a.query_heads + 2 * a.cache_heads;
    if (item >= static_cast<unsigned long long>(a.tokens) * total_heads) return;
    const size_t token = static_cast<size_t>(item / total_heads);
    const unsigned int local = static_cast<unsigned int>(item % total_heads);
    if (local < a.query_heads) {
        const size_t at = (token * a.query_heads + local) * a.head_dim;
        rotate_head<E>(static_cast<T*>(a.query_out) + at, static_cast<const T*>(a.query) + at, a, token, part, a.has_query_norm != 0,
                       a.query_eps, a.query_weight);
        return;
    }
    // Where the token goes: a negative page or slot counts from the end (rotary_cache.rs:376-381).
    long long page = a.wide_index ? static_cast<const long long*>(a.pages)[token] : static_cast<const int*>(a.pages)[token];
    long long slot = a.wide_index ? static_cast<const long long*>(a.slots)[token] : static_cast<const int*>(a.slots)[token];
    if (page < 0) page += a.cache_pages;
    if (slot < 0) slot += a.page_slots;
    if (page < 0 || page >= static_cast<long long>(a.cache_pages) || slot < 0 || slot >= static_cast<long long>(a.page_slots)) {
        if (part == 0) report_index_error(a.status);
        return;
    }
    const size_t cell = (static_cast<size_t>(page) * a.page_slots + static_cast<size_t>(slot)) * a.cache_heads;
    if (local < a.query_heads + a.cache_heads) {
        const unsigned int head = local - a.query_heads;
        rotate_head<E>(static_cast<T*>(a.key_cache) + (cell + head) * a.head_dim,
                       static_cast<const T*>(a.key) + (token * a.cache_heads + head) * a.head_dim, a, token, part, a.has_key_norm != 0,
                       a.key_eps, a.key_weight);
        return;
    }
    const unsigned int head = local - a.query_heads - a.cache_heads;
    const T* from = static_cast<const T*>(a.value) + (token * a.cache_heads + head) * a.head_dim;
    T* to = static_cast<T*>(a.value_cache) + (cell + head) * a.head_dim;
    for (unsigned int dim = part; dim < a.head_dim; dim += 16) to[dim] = from[dim];
}

// The same step sixteen bytes at a time, for head dimensions that are a whole number of chunk pairs (a multiple of 16
// elements in a 16-bit type, of 8 in f32) with every operand on a 16-byte boundary.  A head is dealt to a.group_lanes
// neighbouring lanes (a power of two); lane c < a.head_lanes holds chunk c of the head's first half and chunk c of its
// second half, which are each other's rotation partners, so a head moves as two loads and two stores per lane and the
// only lane traffic is the norm's sum of squares.
template <class E>
struct Chunk {
    static constexpr int kCount = 16 / sizeof(typename E::type);
    float value[kCount];
    static SINGE_DEVICE Chunk load(const typename E::type* from) {
        const uint4 raw = *reinterpret_cast<const uint4*>(from);
        typename E::type lanes[kCount];
        __builtin_memcpy(lanes, &raw, 16);
        Chunk chunk;
#pragma unroll
        for (int i = 0; i < kCount; ++i) chunk.value[i] = E::load(lanes + i);
        return chunk;
    }
    SINGE_DEVICE void store(typename E::type* to) const {
        typename E::type lanes[kCount];
#pragma unroll
        for (int i = 0; i < kCount; ++i) E::store(lanes + i, value[i]);
        uint4 raw;
        __builtin_memcpy(&raw, lanes, 16);
        *reinterpret_cast<uint4*>(to) = raw;
    }
};

// COUNT consecutive angles of a table row, widened to f32.
template <int COUNT>
SINGE_DEVICE void table_chunk(float (&out)[COUNT], const void* table, uint32_t table_type, size_t at) {
    if (table_type == kElementF32) {
        const float4* from = reinterpret_cast<const float4*>(static_cast<const float*>(table) + at);
#pragma unroll
        for (int i = 0; i < COUNT / 4; ++i) {
            const float4 four = from[i];
            out[4 * i] = four.x; out[4 * i + 1] = four.y; out[4 * i + 2] = four.z; out[4 * i + 3] = four.w;
        }
        return;
    }
    unsigned short lanes[COUNT];
    if constexpr (COUNT == 8) {
        const uint4 raw = *reinterpret_cast<const uint4*>(static_cast<const unsigned short*>(table) + at);
        __builtin_memcpy(lanes, &raw, 16);
    } else {
        const uint2 raw = *reinterpret_cast<const uint2*>(static_cast<const unsigned short*>(table) + at);
        __builtin_memcpy(lanes, &raw, 8);
    }
#pragma unroll
    for (int i = 0; i < COUNT; ++i)
        out[i] = table_type == kElementBf16 ? Element<kElementBf16>::load(lanes + i)
                                            : Element<kElementF16>::load(reinterpret_cast<const _Float16*>(lanes + i));
}

template <class E>
SINGE_DEVICE void rotate_head_chunks(typename E::type* to, const typename E::type* from, const RotaryCacheArgs& a, size_t token,
                                     unsigned int chunk, bool live, bool has_norm, float eps, const void* weight) {
    constexpr int kCount = Chunk<E>::kCount;
    const unsigned int half = a.head_dim / 2, at = chunk * kCount;
    Chunk<E> first, second;
    if (live) {
        first = Chunk<E>::load(from + at);
        second = Chunk<E>::load(from + half + at);
    }
    if (has_norm) {
        float squares = 0.0f;
        if (live) {
#pragma unroll
            for (int i = 0; i < kCount; ++i) squares += first.value[i] * first.value[i] + second.value[i] * second.value[i];
        }
        for (unsigned int step = 1; step < a.group_lanes; step <<= 1) squares += __shfl_xor(squares, step, 64);
        const float scale = rsqrtf(squares / static_cast<float>(a.head_dim) + eps);
        if (live) {
#pragma unroll
            for (int i = 0; i < kCount; ++i) {
                first.value[i] *= scale;
                second.value[i] *= scale;
            }
            if (weight != nullptr) {
                const Chunk<E> low = Chunk<E>::load(static_cast<const typename E::type*>(weight) + at);
                const Chunk<E> high = Chunk<E>::load(static_cast<const typename E::type*>(weight) + half + at);
#pragma unroll
                for (int i = 0; i < kCount; ++i) {
                    first.value[i] *= low.value[i];
                    second.value[i] *= high.value[i];
                }
            }
        }
    }
    if (!live) return;
    float cosine[kCount], sine[kCount];
    table_chunk<kCount>(cosine, a.cos, a.table_type, token * half + at);
    table_chunk<kCount>(sine, a.sin, a.table_type, token * half + at);
    Chunk<E> low, high;
#pragma unroll
    for (int i = 0; i < kCount; ++i) {
        low.value[i] = first.value[i] * cosine[i] - second.value[i] * sine[i];
        high.value[i] = second.value[i] * cosine[i] + first.value[i] * sine[i];
    }
    low.store(to + at);
    high.store(to + half + at);
}

template <uint32_t ELEMENT>
SINGE_DEVICE void rotary_cache_write_chunks_body(const RotaryCacheArgs& a) {
    typedef Element<ELEMENT> E;
    typedef typename E::type T;
    constexpr int kCount = Chunk<E>::kCount;
    // A group of lanes never straddles a wave (its width divides 64), and lanes of a group leave together where a
    // shuffle follows, so the norm's exchange meets whole groups.
    const unsigned long long thread = static_cast<unsigned long long>(blockIdx.x) * blockDim.x + threadIdx.x;
    const unsigned long long item = thread / a.group_lanes;
    const unsigned int chunk = static_cast<unsigned int>(thread % a.group_lanes);
    const bool live = chunk < a.head_lanes;
    const unsigned int total_heads = a.query_heads + 2 * a.cache_heads;
    if (item >= static_cast<unsigned long long>(a.tokens) * total_heads) return;
    const size_t token = static_cast<size_t>(item / total_heads);
    const unsigned int local = static_cast<unsigned int>(item % total_heads);
    if (local < a.query_heads) {
        const size_t at = (token * a.query_heads + local) * a.head_dim;
        rotate_head_chunks<E>(static_cast<T*>(a.query_out) + at, static_cast<const T*>(a.query) + at, a, token, chunk, live,
                              a.has_query_norm != 0, a.query_eps, a.query_weight);
        return;
    }
    long long page = a.wide_index ? static_cast<const long long*>(a.pages)[token] : static_cast<const int*>(a.pages)[token];
    long long slot = a.wide_index ? static_cast<const long long*>(a.slots)[token] : static_cast<const int*>(a.slots)[token];
    if (page < 0) page += a.cache_pages;
    if (slot < 0) slot += a.page_slots;
    if (page < 0 || page >= static_cast<long long>(a.cache_pages) || slot < 0 || slot >= static_cast<long long>(a.page_slots)) {
        if (chunk == 0) report_index_error(a.status);
        return;
    }
    const size_t cell = (static_cast<size_t>(page) * a.page_slots + static_cast<size_t>(slot)) * a.cache_heads;
    if (local < a.query_heads + a.cache_heads) {
        const unsigned int head = local - a.query_heads;
        rotate_head_chunks<E>(static_cast<T*>(a.key_cache) + (cell + head) * a.head_dim,
                              static_cast<const T*>(a.key) + (token * a.cache_heads + head) * a.head_dim, a, token, chunk, live,
                              a.has_key_norm != 0, a.key_eps, a.key_weight);
        return;
    }
    if (!live) return;
    const unsigned int head = local - a.query_heads - a.cache_heads, half = a.head_dim / 2;
    const T* from = static_cast<const T*>(a.value) + (token * a.cache_heads + head) * a.head_dim + chunk * kCount;
    T* to = static_cast<T*>(a.value_cache) + (cell + head) * a.head_dim + chunk * kCount;
    const uint4 low = *reinterpret_cast<const uint4*>(from), high = *reinterpret_cast<const uint4*>(from + half);
    *reinterpret_cast<uint4*>(to) = low;
    *reinterpret_cast<uint4*>(to + half) = high;
}

template <bool WIDE>
SINGE_DEVICE void paging_indices_body(const PagingIndicesArgs& a) {
    constexpr int FORM = WIDE ? kCsrI64 : kCsrI32;
    const unsigned long long index = static_cast<unsigned long long>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (index >= static_cast<unsigned long long>(a.sequences) * a.width) return;
    const unsigned int sequence = static_cast<unsigned int>(index / a.width), entry = static_cast<unsigned int>(index % a.width);
    a.page_table[index] = 0;
    if (entry == 0) {
        // Offsets clamped into [0, tokens] and made monotone, so what is written stays inside every buffer
        // whatever the input holds (paged_attention.rs:366-378).
        long long running = 0, sequence_start = 0;
        for (unsigned int other = 0; other <= sequence + 1; ++other) {
            long long offset = read_index<FORM>(a.query_offsets, other);
            offset = offset < 0 ? 0 : (offset > static_cast<long long>(a.tokens) ? static_cast<long long>(a.tokens) : offset);
            if (offset > running) running = offset;
            if (other == sequence) sequence_start = running;
        }
        a.packed_offsets[sequence] = static_cast<int>(sequence_start * a.row_elements);
        if (sequence + 1 == a.sequences) a.packed_offsets[sequence + 1] = static_cast<int>(running * a.row_elements);
        a.query_lengths[sequence] = static_cast<int>(running - sequence_start);
        a.key_lengths[sequence] = 0;
    }
    const SequenceSpan span = load_span<FORM>(sequence, a.query_offsets, a.page_offsets, a.last_page_lengths, nullptr, a.tokens,
                                              a.page_count, a.page_size);
    if (!span.valid) {
        report_index_error(a.status);
        return;
    }
    if (entry == 0) a.key_lengths[sequence] = static_cast<int>(span.keys);
    const long long page_end = read_index<FORM>(a.page_offsets, sequence + 1);
    const long long table_entry = span.page_start + entry;
    if (table_entry < page_end) {
        const long long page = read_index<FORM>(a.pages, static_cast<size_t>(table_entry));
        if (page < 0 || page >= static_cast<long long>(a.cache_pages)) {
            report_index_error(a.status);
            return;
        }
        a.page_table[index] = static_cast<int>(page);
    }
}

// A decode step in FlashInfer form, token by token, for the block-table decode kernels: thread i checks sequence i's
// paging values (reporting what paged_attention.rs:210-238 refuses), gives token i its row (the page list of the
// sequence that owns it and the keys it sees: all of them, or under the causal mask those up to its own position,
// counted from the end as the CPU path does, attention.rs:483), and checks page-table entry i (an id outside the
// cache is reported when a sequence with queries reads it; the decode kernels themselves mask such keys).
template <int FORM>
SINGE_DEVICE void paged_decode_rows_body(const DecodeRowsArgs& a) {
    const unsigned long long index = static_cast<unsigned long long>(blockIdx.x) * blockDim.x + threadIdx.x;
    auto span_of = [&](unsigned int sequence) __attribute__((always_inline)) {
        return load_span<FORM>(sequence, a.query_offsets, a.page_offsets, a.last_page_lengths, nullptr, a.tokens, a.page_table, a.page_size);
    };
    // The last sequence whose offset is at most `value`, by bisection (sequences without queries or pages share an
    // offset with their successor, and the last of them is the one that holds the value).
    auto owner_of = [&](const void* offsets, long long value) __attribute__((always_inline)) {
        unsigned int low = 0, high = a.sequences;  // offsets[low] <= value (or low == 0), offsets[high] > value (or high == sequences)
        while (high - low > 1) {
            const unsigned int middle = (low + high) / 2;
            if (read_index<FORM>(offsets, middle) <= value) low = middle; else high = middle;
        }
        return low;
    };
    // (every load below is asked for before anything waits: the kernel is a chain of memory round trips)
    const long long page = index < a.page_table ? read_index<FORM>(a.pages, index) : 0;
    SequenceSpan own;
    own.valid = false, own.query_start = 0, own.page_start = 0, own.queries = 0, own.keys = 0;
    if (index < a.sequences) {
        own = span_of(static_cast<unsigned int>(index));
        if (!own.valid) report_index_error(a.status);
    }
    if (index < a.tokens) {
        const long long token = static_cast<long long>(index);
        // One token a sequence, in order, is the usual step: then the token's owner is the sequence of its own index,
        // whose values are here already; otherwise the owner is searched for.
        SequenceSpan span = own;
        if (!(index < a.sequences && own.valid && own.query_start == token && own.queries == 1u))
            span = span_of(owner_of(a.query_offsets, token));
        unsigned int start = 0, begin = 0;
        long long length = -1;  // no valid sequence owns the token: its row is left alone
        if (span.valid && token >= span.query_start && token - span.query_start < static_cast<long long>(span.queries)) {
            start = static_cast<unsigned int>(span.page_start);
            length = span.keys;
            // The token's position among the keys, counted from the end and held at the first key (attention.rs:483).
            const long long raw = static_cast<long long>(span.keys) - static_cast<long long>(span.queries) + (token - span.query_start);
            const long long position = raw < 0 ? 0 : raw;
            if (a.causal != 0 && span.keys != 0) length = position + 1 < static_cast<long long>(span.keys) ? position + 1 : static_cast<long long>(span.keys);
            if (a.window >= 0 && length > 0) {
                // Keys with key + window <= position are hidden: whole pages of them are left out of the row, the rest
                // of the first page is masked by the decode kernel.
                const long long first = position + 1 - static_cast<long long>(a.window);
                if (first >= length) {
                    length = 0;  // (a window of no keys)
                } else if (first > 0) {
                    const long long skipped = first / a.page_size;
                    start += static_cast<unsigned int>(skipped);
                    length -= skipped * a.page_size;
                    begin = static_cast<unsigned int>(first - skipped * a.page_size);
                }
            }
        }
        a.row_starts[index] = start;
        a.lengths[index] = static_cast<int>(length);
        if (a.row_begins != nullptr) a.row_begins[index] = begin;
    }
    if (index < a.page_table) {
        const bool outside = page < 0 || page >= static_cast<long long>(a.cache_pages);
        if (a.pages32 != nullptr) a.pages32[index] = outside ? 0xffffffffu : static_cast<unsigned int>(page);
        if (outside) {
            const SequenceSpan span = span_of(owner_of(a.page_offsets, static_cast<long long>(index)));
            const long long entry = static_cast<long long>(index) - span.page_start;
            // (under a window the pages wholly before the first token's window are read by nobody)
            long long unread = 0;
            if (a.window >= 0) {
                const long long raw = static_cast<long long>(span.keys) - static_cast<long long>(span.queries);
                const long long first = (raw < 0 ? 0 : raw) + 1 - static_cast<long long>(a.window);
                unread = first > 0 ? first / a.page_size : 0;
            }
            if (span.valid && span.queries != 0 && entry >= unread && entry * a.page_size < static_cast<long long>(span.keys)) report_index_error(a.status);
        }
    }
}

}  // namespace cache_ops

extern "C" __global__ __launch_bounds__(256) void singe_rotary_cache_write_f32(RotaryCacheArgs args) {
    cache_ops::rotary_cache_write_body<kElementF32>(args);
}
extern "C" __global__ __launch_bounds__(256) void singe_rotary_cache_write_bf16(RotaryCacheArgs args) {
    cache_ops::rotary_cache_write_body<kElementBf16>(args);
}
extern "C" __global__ __launch_bounds__(256) void singe_rotary_cache_write_f16(RotaryCacheArgs args) {
    cache_ops::rotary_cache_write_body<kElementF16>(args);
}
extern "C" __global__ __launch_bounds__(256) void singe_rotary_cache_write_chunks_f32(RotaryCacheArgs args) {
    cache_ops::rotary_cache_write_chunks_body<kElementF32>(args);
}
extern "C" __global__ __launch_bounds__(256) void singe_rotary_cache_write_chunks_bf16(RotaryCacheArgs args) {
    cache_ops::rotary_cache_write_chunks_body<kElementBf16>(args);
}
extern "C" __global__ __launch_bounds__(256) void singe_rotary_cache_write_chunks_f16(RotaryCacheArgs args) {
    cache_ops::rotary_cache_write_chunks_body<kElementF16>(args);
}
extern "C" __global__ __launch_bounds__(256) void singe_paged_decode_rows_i32(DecodeRowsArgs args) { cache_ops::paged_decode_rows_body<kCsrI32>(args); }
extern "C" __global__ __launch_bounds__(256) void singe_paged_decode_rows_i64(DecodeRowsArgs args) { cache_ops::paged_decode_rows_body<kCsrI64>(args); }
extern "C" __global__ __launch_bounds__(256) void singe_paging_indices_i32(PagingIndicesArgs args) {
    cache_ops::paging_indices_body<false>(args);
}
extern "C" __global__ __launch_bounds__(256) void singe_paging_indices_i64(PagingIndicesArgs args) {
    cache_ops::paging_indices_body<true>(args);
}
