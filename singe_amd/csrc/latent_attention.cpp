// Host side of latent (MLA) attention over paged caches: the shape rules of spec::paged_mla_attention_problem
// (singe/src/backend/spec/neural/attention.rs:453-497) and the launch, with the kernel's arguments in the order of
// the reference artifact's ABI (singe/src/backend/cuda/kernel_plan/source/mla.rs:219-230, 260).
#include <cmath>

#include "kernel_args.h"
#include "module.h"
#include "singe_hip_attention.h"
#include "validate.h"

using namespace singe_hip;

extern "C" int32_t singe_hip_paged_mla_attention(void* stream, const void* latent_queries, const void* positional_queries,
                                                 const void* latent_cache, const void* positional_cache,
                                                 const void* query_offsets, const void* page_offsets, const void* pages,
                                                 const void* last_page_lengths, void* output, float* lse, uint32_t* status,
                                                 const SingePagedMlaAttentionProblem* problem) {
    if (problem == nullptr) return fail(SINGE_HIP_NULL_POINTER, "problem");
    const SingePagedMlaAttentionProblem& p = *problem;
    // paged_mla_attention_problem: a page holds at least one key and the latent width is positive; the
    // positional width may be zero.
    if (p.tokens < 0 || p.heads < 0 || p.latent_dim <= 0 || p.position_dim < 0 || p.page_size <= 0 || p.sequences < 0 ||
        p.cache_pages < 0 || p.page_table < 0)
        return fail(SINGE_HIP_INVALID_ARGUMENT, "query or cache shapes");
    if (p.index_type != SINGE_HIP_INDEX_I32 && p.index_type != SINGE_HIP_INDEX_I64)
        return fail(SINGE_HIP_INVALID_ARGUMENT, "index type");
    if (p.data_type != SINGE_HIP_F32 && p.data_type != SINGE_HIP_BF16 && p.data_type != SINGE_HIP_F16)
        return fail(SINGE_HIP_INVALID_ARGUMENT, "data type");
    if (p.has_scale && !std::isfinite(p.scale)) return fail(SINGE_HIP_INVALID_ARGUMENT, "scale");
    const int64_t extents[] = {p.tokens, p.heads, p.latent_dim, p.position_dim, p.page_size, p.sequences, p.cache_pages, p.page_table};
    for (int64_t extent : extents)
        if (!fits_i32(static_cast<uint64_t>(extent))) return fail(SINGE_HIP_LENGTH_EXCEEDS_I32, "problem");
    if (p.latent_dim > 512) return fail(SINGE_HIP_UNSUPPORTED_WIDTH, "paged_mla_attention", static_cast<uint64_t>(p.latent_dim));
    if (p.position_dim > 128) return fail(SINGE_HIP_UNSUPPORTED_WIDTH, "paged_mla_attention", static_cast<uint64_t>(p.position_dim));
    if (p.tokens == 0 || p.heads == 0 || p.sequences == 0) return 0;  // nothing to attend
    const void* pointers[] = {latent_queries, latent_cache, query_offsets, page_offsets, last_page_lengths, output};
    const char* names[] = {"latent_queries", "latent_cache", "query_offsets", "page_offsets", "last_page_lengths", "output"};
    for (int i = 0; i < 6; ++i)
        if (pointers[i] == nullptr) return fail(SINGE_HIP_NULL_POINTER, names[i]);
    if (p.position_dim > 0 && (positional_queries == nullptr || positional_cache == nullptr))
        return fail(SINGE_HIP_NULL_POINTER, "positional queries or cache");
    if (pages == nullptr && p.page_table > 0) return fail(SINGE_HIP_NULL_POINTER, "pages");

    LatentAttentionArgs args;
    args.latent_queries = latent_queries;
    args.positional_queries = positional_queries;
    args.latent_cache = latent_cache;
    args.positional_cache = positional_cache;
    args.query_offsets = query_offsets;
    args.page_offsets = page_offsets;
    args.pages = pages;
    args.last_page_lengths = last_page_lengths;
    args.output = output;
    args.lse = lse;
    args.status = status;
    args.tokens = static_cast<uint32_t>(p.tokens);
    args.heads = static_cast<uint32_t>(p.heads);
    args.latent_dim = static_cast<uint32_t>(p.latent_dim);
    args.position_dim = static_cast<uint32_t>(p.position_dim);
    args.page_size = static_cast<uint32_t>(p.page_size);
    args.sequences = static_cast<uint32_t>(p.sequences);
    args.cache_pages = static_cast<uint32_t>(p.cache_pages);
    args.page_table = static_cast<uint32_t>(p.page_table);
    // Latent width 512 with positional width 64 in a 16-bit type runs on the matrix cores, 128 (token, head) rows of
    // a sequence to a workgroup; every other shape on the vector unit, 4 rows to a workgroup.
    const bool tiles = p.data_type != SINGE_HIP_F32 && p.latent_dim == 512 && p.position_dim == 64;
    const uint64_t rows_per_block = tiles ? 128 : 4;
    const uint64_t row_blocks = (static_cast<uint64_t>(p.tokens) * p.heads + rows_per_block - 1) / rows_per_block;
    args.row_blocks = static_cast<uint32_t>(row_blocks);
    args.causal = p.causal ? 1u : 0u;
    args.wide_index = p.index_type == SINGE_HIP_INDEX_I64 ? 1u : 0u;
    // The default scale counts the whole key width (attention.rs:603-606).
    args.scale = p.has_scale ? p.scale : static_cast<float>(1.0 / std::sqrt(static_cast<double>(p.latent_dim + p.position_dim)));
    const uint64_t blocks = row_blocks * static_cast<uint64_t>(p.sequences);
    if (blocks > 0x7fffffffull || row_blocks > 0xffffffffull) return fail(SINGE_HIP_UNSUPPORTED_CONFIGURATION, "too many workgroups");
    if (tiles)
        return launch(p.data_type == SINGE_HIP_BF16 ? kLatentTilesBf16 : kLatentTilesF16, static_cast<unsigned>(blocks), 1, 1, 512, stream, args);
    const int kernel = kLatentGeneral + (p.data_type == SINGE_HIP_F32 ? 0 : p.data_type == SINGE_HIP_BF16 ? 1 : 2);
    return launch(static_cast<KernelId>(kernel), static_cast<unsigned>(blocks), 1, 1, 256, stream, args);
}
