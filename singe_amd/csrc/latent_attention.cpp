// Host side of latent (MLA) attention over paged caches: the shape rules of spec::paged_mla_attention_problem
// (singe/src/backend/spec/neural/attention.rs:453-497) and the launch, with the kernel's arguments in the order of
// the reference artifact's ABI (singe/src/backend/cuda/kernel_plan/source/mla.rs:219-230, 260).
#include <atomic>
#include <cmath>
#include <cstdint>

#include "kernel_args.h"
#include "module.h"
#include "singe_hip_attention.h"
#include "thread_options.h"
#include "validate.h"

using namespace singe_hip;

namespace {

// Whether the problem runs on a matrix-core kernel: a 16-bit type, a latent width that is a multiple of 32 up to 512
// and a positional width that is a multiple of 8 and makes the key width a multiple of 16, the widths the reference's
// tensor-core plan takes (mla.rs:75, 140-146), with a positional part of at most 64 (wider ones, up to the reference's
// 128, stay on the vector unit: the kernel's LDS rows hold 64).
bool on_matrix_cores(const SingePagedMlaAttentionProblem& p) {
    return p.data_type != SINGE_HIP_F32 && p.latent_dim > 0 && p.latent_dim <= 512 && p.latent_dim % 32 == 0 && p.position_dim >= 0 &&
           p.position_dim <= 64 && p.position_dim % 8 == 0 && (p.latent_dim + p.position_dim) % 16 == 0;
}
// The build for exactly latent 512 + positional 64; other widths take the `_any` kernels.
bool built_shape(const SingePagedMlaAttentionProblem& p) { return p.latent_dim == 512 && p.position_dim == 64; }

// Key splits for a problem: the row tiles of a decode step or a short chunk (one workgroup each, one workgroup to a
// compute unit) leave most of the chip idle, so each tile's keys are shared out until there is about one workgroup
// per compute unit: 64 shares at most (the merge keeps a share's weight per lane), and no more than leave a share
// four key tiles of a sequence of average length (the page table bounds the keys from above).  The count of live
// tiles is not known on the host (it depends on the offsets on the device): every sequence has at least one, and
// together they hold at least tokens * heads / 128.
// 0 = chosen by problem size (singe_hip_set_paged_mla_attention_splits).
std::atomic<uint32_t> g_latent_splits{0};

uint32_t latent_splits(const SingePagedMlaAttentionProblem& p) {
    if (!on_matrix_cores(p) || p.tokens <= 0 || p.heads <= 0 || p.sequences <= 0) return 1;
    if (const uint32_t fixed = effective_count(thread_options().paged_mla_attention_splits, g_latent_splits.load(std::memory_order_relaxed)))
        return fixed;
    const uint64_t packed = (static_cast<uint64_t>(p.tokens) * p.heads + 127) / 128;
    const uint64_t workgroups = packed > static_cast<uint64_t>(p.sequences) ? packed : static_cast<uint64_t>(p.sequences);
    const uint64_t wanted = compute_units();
    if (workgroups >= wanted) return 1;
    const uint64_t mean_keys = static_cast<uint64_t>(p.page_table > 0 ? p.page_table : 0) * static_cast<uint64_t>(p.page_size) / static_cast<uint64_t>(p.sequences);
    const uint64_t worth = mean_keys / (4 * 32);
    uint64_t splits = wanted / workgroups;
    if (splits > 64) splits = 64;
    if (splits > worth) splits = worth;
    return static_cast<uint32_t>(splits < 1 ? 1 : splits);
}

size_t latent_scratch_bytes(const SingePagedMlaAttentionProblem& p, uint32_t splits) {
    if (splits <= 1) return 0;
    return static_cast<size_t>(splits) * static_cast<size_t>(p.tokens) * static_cast<size_t>(p.heads) * (512 + 1) * sizeof(float);
}

int32_t paged_mla_attention(void* stream, const void* latent_queries, const void* positional_queries, const void* latent_cache,
                            const void* positional_cache, const void* query_offsets, const void* page_offsets, const void* pages,
                            const void* last_page_lengths, void* output, float* lse, uint32_t* status, void* scratch,
                            size_t scratch_bytes, const SingePagedMlaAttentionProblem* problem) {
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
    // A 16-bit type at the widths on_matrix_cores names runs on the matrix cores, 128 (token, head) rows of a sequence
    // to a workgroup; every other shape on the vector unit, 4 rows to a workgroup.
    const bool tiles = on_matrix_cores(p);
    const uint64_t rows_per_block = tiles ? 128 : 4;
    const uint64_t row_blocks = (static_cast<uint64_t>(p.tokens) * p.heads + rows_per_block - 1) / rows_per_block;
    args.row_blocks = static_cast<uint32_t>(row_blocks);
    args.causal = p.causal ? 1u : 0u;
    args.wide_index = p.index_type == SINGE_HIP_INDEX_I64 ? 1u : 0u;
    // The default scale counts the whole key width (attention.rs:603-606).
    args.scale = p.has_scale ? p.scale : static_cast<float>(1.0 / std::sqrt(static_cast<double>(p.latent_dim + p.position_dim)));
    // Either kernel's units: a sequence owns one per 128 (matrix cores) or 4 (vector unit) of its rows, at least one.
    const uint64_t blocks = row_blocks + static_cast<uint64_t>(p.sequences);
    if (blocks > 0x7fffffffull || row_blocks > 0xffffffffull) return fail(SINGE_HIP_UNSUPPORTED_CONFIGURATION, "too many workgroups");
    args.splits = 1;
    args.page_shift = -1;
    for (int shift = 0; shift < 31; ++shift)
        if (p.page_size == (int64_t{1} << shift)) args.page_shift = shift;
    args.partial_out = nullptr;
    args.partial_lse = nullptr;
    args.unit_band = 1;
    if (tiles) {
        // Key splits, when the caller lent scratch for them: the attention kernel leaves partials, a second kernel
        // merges them.
        uint32_t splits = scratch != nullptr ? latent_splits(p) : 1;
        if (splits > 1 && (scratch_bytes < latent_scratch_bytes(p, splits) || blocks * splits > 0x7fffffffull || blocks * 32 > 0x7fffffffull))
            splits = 1;
        if (splits > 1) {
            if (reinterpret_cast<uintptr_t>(scratch) % 16 != 0) return fail(SINGE_HIP_INVALID_ARGUMENT, "scratch alignment");
            args.splits = splits;
            args.partial_out = static_cast<float*>(scratch);
            args.partial_lse = args.partial_out + static_cast<size_t>(splits) * p.tokens * p.heads * 512;
        }
        // Without splits, units go to the XCDs in bands of neighbours (see the kernel): as wide as leaves every XCD
        // something to do, 32 (an XCD's compute units, each of which holds one workgroup) at most.  The width follows
        // the units that are surely live (the count of blocks is an upper bound: up to one per sequence more), and the
        // grid covers whole rounds of eight bands.  With splits the grid is the units times their shares.
        const uint64_t surely_live = row_blocks > static_cast<uint64_t>(p.sequences) ? row_blocks : static_cast<uint64_t>(p.sequences);
        const uint64_t band = surely_live >= 256 ? 32 : (surely_live + 7) / 8;
        const uint64_t rounds = (blocks + 8 * band - 1) / (8 * band);
        args.unit_band = static_cast<uint32_t>(band);
        const uint64_t grid = splits > 1 ? blocks * splits : rounds * 8 * band;
        if (grid > 0x7fffffffull) return fail(SINGE_HIP_UNSUPPORTED_CONFIGURATION, "too many workgroups");
        const bool bf16 = p.data_type == SINGE_HIP_BF16, built = built_shape(p);
        const KernelId tiles_kernel = built ? (bf16 ? kLatentTilesBf16 : kLatentTilesF16) : (bf16 ? kLatentTilesAnyBf16 : kLatentTilesAnyF16);
        const int32_t launched = launch(tiles_kernel, static_cast<unsigned>(grid), 1, 1, 512, stream, args);
        if (launched != 0 || splits == 1) return launched;
        // The merge: 32 workgroups of four waves to a unit, a wave to a row.
        const KernelId merge = built ? (bf16 ? kLatentCombineBf16 : kLatentCombineF16) : (bf16 ? kLatentCombineAnyBf16 : kLatentCombineAnyF16);
        return launch(merge, static_cast<unsigned>(blocks * 32), 1, 1, 256, stream, args);
    }
    const int kernel = kLatentGeneral + (p.data_type == SINGE_HIP_F32 ? 0 : p.data_type == SINGE_HIP_BF16 ? 1 : 2);
    return launch(static_cast<KernelId>(kernel), static_cast<unsigned>(blocks), 1, 1, 256, stream, args);
}

}  // namespace

extern "C" int32_t singe_hip_paged_mla_attention(void* stream, const void* latent_queries, const void* positional_queries,
                                                 const void* latent_cache, const void* positional_cache,
                                                 const void* query_offsets, const void* page_offsets, const void* pages,
                                                 const void* last_page_lengths, void* output, float* lse, uint32_t* status,
                                                 const SingePagedMlaAttentionProblem* problem) {
    return paged_mla_attention(stream, latent_queries, positional_queries, latent_cache, positional_cache, query_offsets, page_offsets,
                               pages, last_page_lengths, output, lse, status, nullptr, 0, problem);
}

extern "C" void singe_hip_set_paged_mla_attention_splits(uint32_t splits) {
    g_latent_splits.store(splits > 64 ? 64 : splits, std::memory_order_relaxed);
}

extern "C" size_t singe_hip_paged_mla_attention_scratch_bytes(const SingePagedMlaAttentionProblem* problem) {
    if (problem == nullptr) return 0;
    return latent_scratch_bytes(*problem, latent_splits(*problem));
}

extern "C" int32_t singe_hip_paged_mla_attention_scratch(void* stream, const void* latent_queries, const void* positional_queries,
                                                         const void* latent_cache, const void* positional_cache,
                                                         const void* query_offsets, const void* page_offsets, const void* pages,
                                                         const void* last_page_lengths, void* output, float* lse, uint32_t* status,
                                                         void* scratch, size_t scratch_bytes,
                                                         const SingePagedMlaAttentionProblem* problem) {
    return paged_mla_attention(stream, latent_queries, positional_queries, latent_cache, positional_cache, query_offsets, page_offsets,
                               pages, last_page_lengths, output, lse, status, scratch, scratch_bytes, problem);
}
