// Host side of the rotate-and-append kernel (singe/src/backend/cuda/kernel_plan/source/rotary_cache.rs:249-427)
// and of the CSR -> block-table paging conversion (kernel_plan/source/paged_attention.rs:325-398).
#include <cmath>
#include <cstdint>

#include "kernel_args.h"
#include "module.h"
#include "singe_hip_attention.h"
#include "validate.h"

using namespace singe_hip;

extern "C" int32_t singe_hip_rotary_cache_write(void* stream, const void* query, const void* key, const void* value,
                                                const void* cos, const void* sin, const void* page_index,
                                                const void* slot_index, const void* query_weight, const void* key_weight,
                                                void* query_out, void* key_cache, void* value_cache, uint32_t* status,
                                                const SingeRotaryCacheProblem* problem) {
    if (problem == nullptr) return fail(SINGE_HIP_NULL_POINTER, "problem");
    const SingeRotaryCacheProblem& p = *problem;
    if (p.tokens < 0 || p.query_heads < 0 || p.cache_heads <= 0 || p.head_dim <= 0 || p.head_dim % 2 != 0 || p.cache_pages <= 0 ||
        p.page_slots <= 0)
        return fail(SINGE_HIP_INVALID_ARGUMENT, "rotary cache shape");
    const int32_t types[] = {p.data_type, p.table_type};
    for (int32_t type : types)
        if (type != SINGE_HIP_F32 && type != SINGE_HIP_BF16 && type != SINGE_HIP_F16) return fail(SINGE_HIP_INVALID_ARGUMENT, "data type");
    if (p.index_type != SINGE_HIP_INDEX_I32 && p.index_type != SINGE_HIP_INDEX_I64) return fail(SINGE_HIP_INVALID_ARGUMENT, "index type");
    if ((p.has_query_norm && !std::isfinite(p.query_eps)) || (p.has_key_norm && !std::isfinite(p.key_eps)))
        return fail(SINGE_HIP_INVALID_ARGUMENT, "eps");
    const int64_t extents[] = {p.tokens, p.query_heads, p.cache_heads, p.head_dim, p.cache_pages, p.page_slots};
    for (int64_t extent : extents)
        if (!fits_i32(static_cast<uint64_t>(extent))) return fail(SINGE_HIP_LENGTH_EXCEEDS_I32, "problem");
    if (p.tokens == 0) return 0;
    const void* pointers[] = {key, value, cos, sin, page_index, slot_index, key_cache, value_cache};
    const char* names[] = {"key", "value", "cos", "sin", "page_index", "slot_index", "key_cache", "value_cache"};
    for (int i = 0; i < 8; ++i)
        if (pointers[i] == nullptr) return fail(SINGE_HIP_NULL_POINTER, names[i]);
    if (p.query_heads > 0 && query == nullptr) return fail(SINGE_HIP_NULL_POINTER, "query");
    if (p.query_heads > 0 && query_out == nullptr) return fail(SINGE_HIP_NULL_POINTER, "query_out");

    RotaryCacheArgs args;
    args.query = query;
    args.key = key;
    args.value = value;
    args.cos = cos;
    args.sin = sin;
    args.pages = page_index;
    args.slots = slot_index;
    args.query_weight = p.has_query_norm ? query_weight : nullptr;
    args.key_weight = p.has_key_norm ? key_weight : nullptr;
    args.query_out = query_out;
    args.key_cache = key_cache;
    args.value_cache = value_cache;
    args.status = status;
    args.tokens = static_cast<uint32_t>(p.tokens);
    args.query_heads = static_cast<uint32_t>(p.query_heads);
    args.cache_heads = static_cast<uint32_t>(p.cache_heads);
    args.head_dim = static_cast<uint32_t>(p.head_dim);
    args.cache_pages = static_cast<uint32_t>(p.cache_pages);
    args.page_slots = static_cast<uint32_t>(p.page_slots);
    args.table_type = static_cast<uint32_t>(p.table_type);
    args.wide_index = p.index_type == SINGE_HIP_INDEX_I64 ? 1u : 0u;
    args.has_query_norm = p.has_query_norm ? 1u : 0u;
    args.has_key_norm = p.has_key_norm ? 1u : 0u;
    args.query_eps = p.query_eps;
    args.key_eps = p.key_eps;
    const uint64_t items = static_cast<uint64_t>(p.tokens) * static_cast<uint64_t>(p.query_heads + 2 * p.cache_heads);
    const int type_index = p.data_type == SINGE_HIP_F32 ? 0 : p.data_type == SINGE_HIP_BF16 ? 1 : 2;
    // Sixteen bytes at a time where a head is a whole number of chunk pairs (its halves are then whole chunks, and so
    // are the angles' rows) and every operand starts on a 16-byte boundary; a lane takes one chunk of each half.
    const uint64_t chunk_elements = p.data_type == SINGE_HIP_F32 ? 4 : 8;
    args.head_lanes = 0;
    args.group_lanes = 0;
    if (static_cast<uint64_t>(p.head_dim) % (2 * chunk_elements) == 0 && static_cast<uint64_t>(p.head_dim) / (2 * chunk_elements) <= 64) {
        bool aligned = true;
        const void* operands[] = {query, key, value, cos, sin, args.query_weight, args.key_weight, query_out, key_cache, value_cache};
        for (const void* operand : operands) aligned = aligned && reinterpret_cast<uintptr_t>(operand) % 16 == 0;
        if (aligned) {
            args.head_lanes = static_cast<uint32_t>(static_cast<uint64_t>(p.head_dim) / (2 * chunk_elements));
            args.group_lanes = 1;
            while (args.group_lanes < args.head_lanes) args.group_lanes *= 2;
        }
    }
    if (args.group_lanes != 0) {
        const uint64_t blocks = (items * args.group_lanes + 255) / 256;
        if (blocks > 0x7fffffffull) return fail(SINGE_HIP_UNSUPPORTED_CONFIGURATION, "too many workgroups");
        return launch(static_cast<KernelId>(kRotaryCacheChunks + type_index), static_cast<unsigned>(blocks), 1, 1, 256, stream, args);
    }
    const uint64_t blocks = (items + 15) / 16;  // sixteen heads of sixteen lanes per workgroup
    if (blocks > 0x7fffffffull) return fail(SINGE_HIP_UNSUPPORTED_CONFIGURATION, "too many workgroups");
    return launch(static_cast<KernelId>(kRotaryCacheF32 + type_index), static_cast<unsigned>(blocks), 1, 1, 256, stream, args);
}

extern "C" int32_t singe_hip_paging_indices(void* stream, const void* query_offsets, const void* page_offsets, const void* pages,
                                            const void* last_page_lengths, int32_t* packed_offsets, int32_t* query_lengths,
                                            int32_t* key_lengths, int32_t* page_table, uint32_t* status,
                                            const SingePagingIndicesProblem* problem) {
    if (problem == nullptr) return fail(SINGE_HIP_NULL_POINTER, "problem");
    const SingePagingIndicesProblem& p = *problem;
    if (p.sequences < 0 || p.tokens < 0 || p.page_count < 0 || p.page_size <= 0 || p.cache_pages < 0 || p.width <= 0 || p.row_elements < 0)
        return fail(SINGE_HIP_INVALID_ARGUMENT, "paging shape");
    if (p.index_type != SINGE_HIP_INDEX_I32 && p.index_type != SINGE_HIP_INDEX_I64) return fail(SINGE_HIP_INVALID_ARGUMENT, "index type");
    const int64_t extents[] = {p.sequences, p.tokens, p.page_count, p.page_size, p.cache_pages, p.width};
    for (int64_t extent : extents)
        if (!fits_i32(static_cast<uint64_t>(extent))) return fail(SINGE_HIP_LENGTH_EXCEEDS_I32, "problem");
    // Packed offsets are written as i32 (paged_attention.rs:379-381).
    uint64_t reach = 0;
    if (__builtin_mul_overflow(static_cast<uint64_t>(p.tokens), static_cast<uint64_t>(p.row_elements), &reach) || !fits_i32(reach))
        return fail(SINGE_HIP_LENGTH_EXCEEDS_I32, "tokens * row_elements");
    if (p.sequences == 0) return 0;
    const void* pointers[] = {query_offsets, page_offsets, last_page_lengths, packed_offsets, query_lengths, key_lengths, page_table};
    const char* names[] = {"query_offsets", "page_offsets", "last_page_lengths", "packed_offsets", "query_lengths", "key_lengths", "page_table"};
    for (int i = 0; i < 7; ++i)
        if (pointers[i] == nullptr) return fail(SINGE_HIP_NULL_POINTER, names[i]);
    if (pages == nullptr && p.page_count > 0) return fail(SINGE_HIP_NULL_POINTER, "pages");
    PagingIndicesArgs args;
    args.query_offsets = query_offsets;
    args.page_offsets = page_offsets;
    args.pages = pages;
    args.last_page_lengths = last_page_lengths;
    args.packed_offsets = packed_offsets;
    args.query_lengths = query_lengths;
    args.key_lengths = key_lengths;
    args.page_table = page_table;
    args.status = status;
    args.sequences = static_cast<uint32_t>(p.sequences);
    args.tokens = static_cast<uint32_t>(p.tokens);
    args.page_count = static_cast<uint32_t>(p.page_count);
    args.page_size = static_cast<uint32_t>(p.page_size);
    args.cache_pages = static_cast<uint32_t>(p.cache_pages);
    args.width = static_cast<uint32_t>(p.width);
    args.row_elements = static_cast<uint64_t>(p.row_elements);
    const uint64_t blocks = (static_cast<uint64_t>(p.sequences) * p.width + 255) / 256;
    if (blocks > 0x7fffffffull) return fail(SINGE_HIP_UNSUPPORTED_CONFIGURATION, "too many workgroups");
    return launch(p.index_type == SINGE_HIP_INDEX_I64 ? kPagingIndicesI64 : kPagingIndicesI32, static_cast<unsigned>(blocks), 1, 1, 256,
                  stream, args);
}
