// Host side of the paged attention op: the shape rules of spec::paged_attention_problem
// (singe/src/backend/spec/neural/attention.rs:337-367, 408-438) and the launch, with the kernel's
// arguments in the order of the reference artifact's ABI
// (singe/src/backend/cuda/kernel_plan/source/paged_attention.rs:687-715).
#include <atomic>
#include <cmath>

#include "kernel_args.h"
#include "module.h"
#include "singe_hip_attention.h"
#include "thread_options.h"
#include "validate.h"

using namespace singe_hip;

namespace singe_hip {
int32_t paged_attention_general(int32_t data_type, void* stream, const void* query_rows, const void* key_cache,
                                const void* value_cache, const void* query_offsets, const void* page_offsets,
                                const void* pages, const void* last_page_lengths, void* output, float* lse, uint32_t* status,
                                const SingePagedAttentionProblem& p, float scale);
}

namespace {

// What rotary_paged_attention adds to the operands: the angle tables, the norm's weight and its attributes.
struct Rotation {
    const void* cos;
    const void* sin;
    const void* weight;
    const SingeQueryRotation* attributes;
};

// Scratch for key splits: what singe_hip_paged_attention_scratch_bytes asked for, or nothing.
struct Scratch {
    void* memory;
    size_t bytes;
};

// How the grid covers the row tiles (see `locate` in paged_attention.hip).  When no sequence can have more than one
// row tile the plain form is used: sequences x kv heads workgroups, a sequence found from the workgroup id alone.
// Otherwise the compact form: every sequence has at least one entry, and the entries of all of them are at most
// floor(tokens * groups / rows) + sequences (rows: the packed rows of a workgroup, 128, or 256 on the two-tile kernel).
struct RowTileGrid {
    uint32_t compact;
    uint32_t longest_first;  // the compact list takes the sequences longest first (see `locate`)
    uint64_t row_tiles;   // the kernel argument
    uint64_t blocks;      // workgroups without key splits
};

RowTileGrid grid_of(uint64_t tokens, uint64_t sequences, uint64_t groups, uint64_t kv_heads = 1, uint64_t rows = 128) {
    RowTileGrid grid;
    const uint64_t longest = (groups * tokens + rows - 1) / rows;
    grid.longest_first = 0;
    if (longest <= 1) {
        grid.compact = 0;
        grid.row_tiles = longest;
        grid.blocks = (sequences * kv_heads + 7) / 8 * 8 * longest;
    } else {
        grid.compact = 1;
        grid.row_tiles = groups * tokens / rows + sequences;
        // Longest sequences first where sequences have row tiles to spare (chunks of a prefill): their workgroups run
        // for hundreds of microseconds and the order decides how full the chip's last round is.
        grid.longest_first = sequences <= 64 && groups * tokens / rows >= 2 * sequences ? 1u : 0u;
        const uint64_t bands = (grid.row_tiles + 31) / 32;
        grid.blocks = (kv_heads * bands + 7) / 8 * 8 * 32;
    }
    return grid;
}

// 0 = chosen by problem size (singe_hip_set_paged_attention_splits).
std::atomic<uint32_t> g_paged_attention_splits{0};
// Packed rows a wave of the bf16 / f16 kernels takes: 0 = chosen by problem size, 32, or 64 where the two-tile kernel
// takes the call (singe_hip_set_paged_attention_rows_per_wave).
std::atomic<uint32_t> g_paged_rows_per_wave{0};

// The count in force on this thread: its own (SingeHipThreadOptions) over the process-wide one.
uint32_t fixed_paged_attention_splits() {
    return effective_count(thread_options().paged_attention_splits, g_paged_attention_splits.load(std::memory_order_relaxed));
}

// Whether a bf16 / f16 call without a fused rotation or key splits runs on the kernel that gives a wave two 32-row
// tiles, and the grid it takes there: a head_dim that is a multiple of 16 up to 128, a page size that is a power of two of at least 16 keys, no cap, no
// window, a positive scale, and (unless the knob says 64) enough 256-row tiles to fill the chip.
bool two_tiles_a_wave(const SingePagedAttentionProblem& p, RowTileGrid* grid) {
    const uint32_t wanted = g_paged_rows_per_wave.load(std::memory_order_relaxed);
    if (wanted == 32 || !has_pair_build(p.head_dim) || p.has_softcap || p.has_window || p.tokens <= 0 || p.sequences <= 0 || p.kv_heads <= 0 ||
        p.heads <= 0 || p.page_size < 16 || (p.page_size & (p.page_size - 1)) != 0)
        return false;
    // (the kernel works out where a page starts from a 32-bit count of a page's bytes)
    if (static_cast<uint64_t>(p.page_size) * static_cast<uint64_t>(p.kv_heads) * (2 * static_cast<uint64_t>(p.head_dim)) > 0xffffffffull) return false;
    const float scale = p.has_scale ? p.scale : 1.0f;
    if (!(scale > 0.0f)) return false;
    const uint64_t groups = static_cast<uint64_t>(p.heads / p.kv_heads);
    *grid = grid_of(static_cast<uint64_t>(p.tokens), static_cast<uint64_t>(p.sequences), groups, static_cast<uint64_t>(p.kv_heads), 256);
    if (grid->blocks > 0x7fffffffull || grid->row_tiles > 0xffffffffull) return false;
    // (workgroups that are sure to have work: the whole 256-row tiles of all sequences together, for every kv head)
    const uint64_t working = static_cast<uint64_t>(p.kv_heads) * (groups * static_cast<uint64_t>(p.tokens) / 256);
    return wanted == 64 || (grid->compact != 0 && working >= compute_units());
}

// Key splits for a problem: enough workgroups to fill the compute units four times over, when the query rows
// alone do not (decoding, short chunks); one (no split) for other element types and head dimensions.
uint32_t paged_attention_splits(const SingePagedAttentionProblem& p) {
    if (!has_matrix_core_build(p.head_dim) || p.tokens <= 0 || p.sequences <= 0 || p.kv_heads <= 0 || p.heads <= 0) return 1;
    if (const uint32_t fixed = fixed_paged_attention_splits()) return fixed;
    const uint64_t groups = static_cast<uint64_t>(p.heads / p.kv_heads);
    // Workgroups of the unsplit grid that can have work: the list of row tiles, or one per sequence, for every kv head.
    const RowTileGrid tiling = grid_of(static_cast<uint64_t>(p.tokens), static_cast<uint64_t>(p.sequences), groups);
    const uint64_t workgroups = static_cast<uint64_t>(p.kv_heads) * (tiling.compact ? tiling.row_tiles : tiling.row_tiles * static_cast<uint64_t>(p.sequences));
    // The sequences' key counts live in device memory: the page table bounds their sum, and shares are sized for
    // a sequence of average length, or for the window when that is shorter (the tiles before it are skipped).
    uint64_t keys = static_cast<uint64_t>(p.page_table > 0 ? p.page_table : 0) * static_cast<uint64_t>(p.page_size) / static_cast<uint64_t>(p.sequences);
    if (p.has_window && static_cast<uint64_t>(p.window) < keys) keys = static_cast<uint64_t>(p.window);
    return attention_key_splits(workgroups, keys);
}

// A decode step (no more tokens than sequences: a token a sequence) through this op takes the block-table decode
// kernels, which cut the keys of all sequences into equal ranges whatever their lengths: a small kernel first turns
// the paging vectors into one row per token (where its page list starts, how many keys it sees) and checks them.
// What the host can tell: a matrix-core decode build for the head dimension, no cap or fused rotation, and
// sizes the decode kernels take.  (The decode kernels read 32-bit page ids: i64 paging is copied on the way.)
constexpr size_t kDecodeRowsMost = 8000;

bool decode_rows_config(const SingePagedAttentionProblem& p, SingePagedKvDecodeAttentionConfig* config) {
    if (fixed_paged_attention_splits() != 0) return false;  // a fixed number of shares asks for the row-tile kernel
    if (!has_decode_build(p.head_dim) || p.has_softcap) return false;
    // Under a short window a token reads few keys, and one workgroup a (sequence, kv head) of the row-tile kernel, which
    // skips the tiles before the window, is done before the route's two extra launches would be (measured: 32 sequences,
    // window 128: 12.6 against 15.2 us; window 1024: level; window 4096: 70 against 57 us).
    if (p.has_window && p.window < 2048) return false;
    // (the decode kernels keep three words a token in LDS, four under a window)
    if (p.tokens <= 0 || p.tokens > p.sequences || static_cast<size_t>(p.tokens) > (p.has_window ? kDecodeRowsMost * 3 / 4 : kDecodeRowsMost) ||
        p.page_table <= 0 || p.cache_pages <= 0)
        return false;
    if (!fits_i32(static_cast<uint64_t>(p.page_table) * static_cast<uint64_t>(p.page_size))) return false;
    config->batch = static_cast<size_t>(p.tokens);
    config->heads = static_cast<size_t>(p.heads);
    config->kv_heads = static_cast<size_t>(p.kv_heads);
    config->head_dim = static_cast<size_t>(p.head_dim);
    config->block_size = static_cast<size_t>(p.page_size);
    config->physical_blocks = static_cast<size_t>(p.cache_pages);
    config->block_table_batch_stride = static_cast<size_t>(p.page_table);  // the count of entries: rows have their own lengths
    config->scale = p.has_scale ? p.scale : 1.0f / std::sqrt(static_cast<float>(p.head_dim));
    return true;
}

size_t align256(size_t bytes) { return (bytes + 255) / 256 * 256; }

size_t decode_rows_page_copy_bytes(const SingePagedAttentionProblem& p) {
    return p.index_type == SINGE_HIP_INDEX_I64 ? align256(static_cast<size_t>(p.page_table) * sizeof(uint32_t)) : 0;
}

// Scratch of that route: the tokens' row starts, their lengths, the 32-bit copy of i64 page ids, the decode kernels' workspace.
size_t decode_rows_bytes(const SingePagedAttentionProblem& p) {
    SingePagedKvDecodeAttentionConfig config;
    if (!decode_rows_config(p, &config)) return 0;
    return (p.has_window ? 3 : 2) * align256(static_cast<size_t>(p.tokens) * sizeof(uint32_t)) + decode_rows_page_copy_bytes(p) +
           paged_decode_workspace_bytes(config);
}

size_t scratch_bytes_for(const SingePagedAttentionProblem& p, uint32_t splits) {
    if (splits <= 1) return 0;
    return static_cast<size_t>(splits) * static_cast<size_t>(p.tokens) * static_cast<size_t>(p.heads) * (static_cast<size_t>(p.head_dim) + 1) * sizeof(float);
}

int32_t paged_attention(int32_t data_type, void* stream, const void* query_rows_any, const void* key_cache_any,
                        const void* value_cache_any, const void* query_offsets, const void* page_offsets, const void* pages,
                        const void* last_page_lengths, void* output_any, float* lse, uint32_t* status,
                        const SingePagedAttentionProblem* problem, const Rotation* rotation = nullptr,
                        const Scratch* scratch = nullptr) {
    if (problem == nullptr) return fail(SINGE_HIP_NULL_POINTER, "problem");
    const SingePagedAttentionProblem& p = *problem;
    if (rotation != nullptr) {
        if (rotation->attributes == nullptr) return fail(SINGE_HIP_NULL_POINTER, "rotation");
        const int32_t table = rotation->attributes->table_type;
        if (table != SINGE_HIP_F32 && table != SINGE_HIP_BF16 && table != SINGE_HIP_F16)
            return fail(SINGE_HIP_INVALID_ARGUMENT, "angle table type");
        if (rotation->attributes->has_norm && !std::isfinite(rotation->attributes->eps)) return fail(SINGE_HIP_INVALID_ARGUMENT, "eps");
        // The fused form exists where the reference fuses (paged_attention.rs:512-531, tensor_core.rs:18-32): f16 or
        // bf16 at a multiple of 16 up to 128, with or without a cap; for the rest the rotation and the attention are
        // planned apart, and so does a caller of this library (singe_hip_rotary_cache_write, then singe_hip_paged_attention_*).
        if ((data_type != SINGE_HIP_BF16 && data_type != SINGE_HIP_F16) || !has_matrix_core_build(p.head_dim))
            return fail(SINGE_HIP_UNSUPPORTED_WIDTH, "rotary_paged_attention", static_cast<uint64_t>(p.head_dim));
    }
    // paged_attention_problem: key_dim == head_dim (one field here), kv_heads > 0 dividing heads, page_size > 0.
    if (p.tokens < 0 || p.heads <= 0 || p.kv_heads <= 0 || p.heads % p.kv_heads != 0 || p.page_size <= 0 || p.head_dim <= 0 ||
        p.sequences < 0 || p.cache_pages < 0 || p.page_table < 0)
        return fail(SINGE_HIP_INVALID_ARGUMENT, "heads, head dimension, or page size");
    if (p.index_type != SINGE_HIP_INDEX_I32 && p.index_type != SINGE_HIP_INDEX_I64)
        return fail(SINGE_HIP_INVALID_ARGUMENT, "index type");
    if (p.has_scale && !std::isfinite(p.scale)) return fail(SINGE_HIP_INVALID_ARGUMENT, "scale");
    if (p.has_softcap && !(std::isfinite(p.softcap) && p.softcap != 0.0f)) return fail(SINGE_HIP_INVALID_ARGUMENT, "softcap");
    if (p.has_window && p.window < 0) return fail(SINGE_HIP_INVALID_ARGUMENT, "window");
    const int64_t extents[] = {p.tokens, p.heads, p.kv_heads, p.page_size, p.sequences, p.cache_pages, p.page_table};
    for (int64_t extent : extents)
        if (!fits_i32(static_cast<uint64_t>(extent))) return fail(SINGE_HIP_LENGTH_EXCEEDS_I32, "problem");
    if (!fits_i32(static_cast<uint64_t>(p.head_dim))) return fail(SINGE_HIP_LENGTH_EXCEEDS_I32, "problem");
    if (static_cast<uint64_t>(p.page_size) * static_cast<uint64_t>(p.kv_heads) * static_cast<uint64_t>(p.head_dim) > 0xffffffffull)
        return fail(SINGE_HIP_UNSUPPORTED_CONFIGURATION, "a cache page beyond 4 Gi elements");
    if (p.tokens == 0 || p.sequences == 0) return 0;  // nothing to attend
    const void* pointers[] = {query_rows_any, key_cache_any, value_cache_any, query_offsets, page_offsets, last_page_lengths, output_any};
    const char* names[] = {"query_rows", "key_cache", "value_cache", "query_offsets", "page_offsets", "last_page_lengths", "output"};
    for (int i = 0; i < 7; ++i)
        if (pointers[i] == nullptr) return fail(SINGE_HIP_NULL_POINTER, names[i]);
    if (pages == nullptr && p.page_table > 0) return fail(SINGE_HIP_NULL_POINTER, "pages");
    if (rotation != nullptr && (rotation->cos == nullptr || rotation->sin == nullptr)) return fail(SINGE_HIP_NULL_POINTER, "cos or sin");
    const float scale = p.has_scale ? p.scale : 1.0f / std::sqrt(static_cast<float>(p.head_dim));
    // The matrix-core kernels cover bf16 and f16 at head dimensions 128 and 64 (the reference's take f16/bf16 at
    // multiples of 16 up to 128: paged_attention.rs:586-592); everything else goes to the general one
    // (paged_general.rs:73-247).
    const bool f16 = data_type == SINGE_HIP_F16;
    const long long head_dim = p.head_dim;  // the build of the kernels for it
    auto built = [head_dim](int kernel) { return at_head_dim(static_cast<KernelId>(kernel), head_dim); };
    if ((data_type != SINGE_HIP_BF16 && !f16) || !has_matrix_core_build(head_dim))
        return paged_attention_general(data_type, stream, query_rows_any, key_cache_any, value_cache_any, query_offsets,
                                       page_offsets, pages, last_page_lengths, output_any, lse, status, p, scale);
    const uint16_t* query_rows = static_cast<const uint16_t*>(query_rows_any);
    const uint16_t* key_cache = static_cast<const uint16_t*>(key_cache_any);
    const uint16_t* value_cache = static_cast<const uint16_t*>(value_cache_any);
    uint16_t* output = static_cast<uint16_t*>(output_any);

    // A decode step with scratch for it: the block-table decode kernels (see decode_rows_config).
    if (rotation == nullptr && scratch != nullptr && scratch->memory != nullptr && reinterpret_cast<uintptr_t>(scratch->memory) % 256 == 0) {
        SingePagedKvDecodeAttentionConfig config;
        const size_t need = decode_rows_bytes(p);
        if (need != 0 && scratch->bytes >= need && decode_rows_config(p, &config)) {
            unsigned char* memory = static_cast<unsigned char*>(scratch->memory);
            const size_t array_bytes = align256(static_cast<size_t>(p.tokens) * sizeof(uint32_t));
            DecodeRowsArgs rows;
            rows.query_offsets = query_offsets;
            rows.page_offsets = page_offsets;
            rows.pages = pages;
            rows.last_page_lengths = last_page_lengths;
            rows.row_starts = reinterpret_cast<uint32_t*>(memory);
            rows.lengths = reinterpret_cast<int32_t*>(memory + array_bytes);
            const size_t copy_bytes = decode_rows_page_copy_bytes(p);
            const size_t arrays = p.has_window ? 3 : 2;
            rows.row_begins = p.has_window ? reinterpret_cast<uint32_t*>(memory + 2 * array_bytes) : nullptr;
            rows.window = !p.has_window ? -1 : p.window > 0x7fffffffll ? 0x7fffffff : static_cast<int32_t>(p.window);  // (positions fit 31 bits)
            rows.pages32 = copy_bytes != 0 ? reinterpret_cast<uint32_t*>(memory + arrays * array_bytes) : nullptr;
            rows.status = status;
            rows.tokens = static_cast<uint32_t>(p.tokens);
            rows.sequences = static_cast<uint32_t>(p.sequences);
            rows.page_table = static_cast<uint32_t>(p.page_table);
            rows.page_size = static_cast<uint32_t>(p.page_size);
            rows.cache_pages = static_cast<uint32_t>(p.cache_pages);
            rows.causal = p.causal ? 1u : 0u;
            const uint64_t most = static_cast<uint64_t>(p.page_table > p.sequences ? p.page_table : p.sequences);
            const KernelId bridge = p.index_type == SINGE_HIP_INDEX_I64 ? kPagedDecodeRowsI64 : kPagedDecodeRows;
            if (int32_t launched = launch(bridge, static_cast<unsigned>((most + 255) / 256), 1, 1, 256, stream, rows)) return launched;
            PagedDecodeLaunch decode;
            decode.stream = stream;
            decode.out = output;
            decode.query = query_rows;
            decode.key_cache = key_cache;
            decode.value_cache = value_cache;
            decode.f16 = f16;
            decode.actual_seq_lens = rows.lengths;
            decode.block_table = rows.pages32 != nullptr ? rows.pages32 : static_cast<const uint32_t*>(pages);
            decode.workspace = memory + arrays * array_bytes + copy_bytes;
            decode.workspace_bytes = scratch->bytes - arrays * array_bytes - copy_bytes;
            decode.row_starts = rows.row_starts;
            decode.row_begins = rows.row_begins;
            decode.lse = lse;
            return launch_paged_decode(config, decode);
        }
    }
    const uint64_t groups = static_cast<uint64_t>(p.heads / p.kv_heads);
    PagedAttentionArgs args;
    args.query_rows = query_rows;
    args.key_cache = key_cache;
    args.value_cache = value_cache;
    args.query_offsets = query_offsets;
    args.page_offsets = page_offsets;
    args.pages = pages;
    args.last_page_lengths = last_page_lengths;
    args.query_lengths = nullptr;
    args.output = output;
    args.lse = lse;
    args.status = status;
    args.window = p.has_window ? p.window : -1;
    args.tokens = static_cast<uint32_t>(p.tokens);
    args.heads = static_cast<uint32_t>(p.heads);
    args.kv_heads = static_cast<uint32_t>(p.kv_heads);
    args.page_size = static_cast<uint32_t>(p.page_size);
    args.sequences = static_cast<uint32_t>(p.sequences);
    args.cache_pages = static_cast<uint32_t>(p.cache_pages);
    args.page_table = static_cast<uint32_t>(p.page_table);
    const RowTileGrid tiling = grid_of(static_cast<uint64_t>(p.tokens), static_cast<uint64_t>(p.sequences), groups,
                                     static_cast<uint64_t>(p.kv_heads));
    if (tiling.row_tiles > 0xffffffffull) return fail(SINGE_HIP_UNSUPPORTED_CONFIGURATION, "too many row tiles");
    args.row_tiles = static_cast<uint32_t>(tiling.row_tiles);
    args.compact = tiling.compact;
    args.longest_first = tiling.longest_first;
    args.causal = p.causal ? 1u : 0u;
    args.page_shift = -1;
    for (int shift = 0; shift < 31; ++shift)
        if ((int64_t{1} << shift) == p.page_size) args.page_shift = shift;
    constexpr float kLog2e = 1.4426950408889634074f;
    args.scale_log2e = scale * kLog2e;
    args.softcap_scale = p.has_softcap ? scale / p.softcap : 0.0f;
    args.softcap_log2e = p.has_softcap ? p.softcap * kLog2e : 0.0f;
    const uint64_t blocks = tiling.blocks;
    if (blocks > 0x7fffffffull) return fail(SINGE_HIP_UNSUPPORTED_CONFIGURATION, "too many workgroups");
    const bool wide = p.index_type == SINGE_HIP_INDEX_I64;
    // Key splits, when the caller lent scratch for them: the attention kernel leaves partials, a second
    // kernel merges them.  Without scratch (or with too little) the keys of a row tile stay in one workgroup.
    uint32_t splits = scratch != nullptr && scratch->memory != nullptr ? paged_attention_splits(p) : 1;
    if (splits > 1 && scratch->bytes < scratch_bytes_for(p, splits)) splits = 1;
    if (splits > 1 && blocks * splits > 0x7fffffffull) splits = 1;
    args.splits = splits;
    if (splits > 1) {
        args.partial_out = static_cast<float*>(scratch->memory);
        args.partial_lse = args.partial_out + static_cast<size_t>(splits) * p.tokens * p.heads * p.head_dim;
    }
    if (rotation != nullptr) {
        args.cos = rotation->cos;
        args.sin = rotation->sin;
        args.query_weight = rotation->attributes->has_norm ? static_cast<const uint16_t*>(rotation->weight) : nullptr;
        args.table_type = static_cast<uint32_t>(rotation->attributes->table_type);
        args.has_query_norm = rotation->attributes->has_norm ? 1u : 0u;
        args.query_eps = rotation->attributes->eps;
    }
    // Prefill-shaped plain calls at the matrix-core head dimensions (with or without the fused query rotation) take the kernel that gives a
    // wave two 32-row tiles (256 packed rows a workgroup, one workgroup a compute unit; paged_attention_pair.hip), when
    // its grid still fills the chip.
    RowTileGrid pair;
    if (splits == 1 && (data_type == SINGE_HIP_BF16 || f16) && two_tiles_a_wave(p, &pair)) {
        args.row_tiles = static_cast<uint32_t>(pair.row_tiles);
        args.compact = pair.compact;
        args.longest_first = pair.longest_first;
        const int kernel = pair_kernels_at(p.head_dim, true) + (wide ? 1 : 0) + (f16 ? 2 : 0) + (rotation != nullptr ? 4 : 0);
        return launch(static_cast<KernelId>(kernel), static_cast<unsigned>(pair.blocks), 1, 1, 256, stream, args);
    }
    const unsigned grid = static_cast<unsigned>(blocks * splits);
    auto finish = [&](int32_t launched) -> int32_t {
        if (launched != 0 || splits == 1) return launched;
        const int combine = (f16 ? kPagedAttentionCombineF16I32 : kPagedAttentionCombineI32) + (wide ? 1 : 0);
        return launch(built(combine), static_cast<unsigned>(blocks), 1, 1, 256, stream, args);
    };
    if (rotation != nullptr) {
        const int rotary = rotary_paged_attention_base(f16, p.has_softcap != 0, head_dim) + (wide ? 1 : 0) + (args.page_shift >= 4 ? 2 : 0);
        return finish(launch(static_cast<KernelId>(rotary), grid, 1, 1, 256, stream, args));
    }
    const int kernel = (f16 ? kPagedAttentionF16 : kPagedAttentionI32) + (p.has_softcap ? 2 : 0) + (wide ? 1 : 0) +
                       (args.page_shift >= 4 ? 4 : 0);
    return finish(launch(built(kernel), grid, 1, 1, 256, stream, args));
}

}  // namespace

extern "C" void singe_hip_set_paged_attention_rows_per_wave(uint32_t rows) { g_paged_rows_per_wave.store(rows, std::memory_order_relaxed); }

extern "C" uint32_t singe_hip_paged_attention_rows_per_wave(const SingePagedAttentionProblem* problem) {
    if (problem == nullptr || !has_matrix_core_build(problem->head_dim)) return 0;
    RowTileGrid grid;
    return paged_attention_splits(*problem) == 1 && two_tiles_a_wave(*problem, &grid) ? 64u : 32u;
}

extern "C" void singe_hip_set_paged_attention_splits(uint32_t splits) {
    g_paged_attention_splits.store(splits > 64 ? 64 : splits, std::memory_order_relaxed);
}

extern "C" size_t singe_hip_paged_attention_scratch_bytes(const SingePagedAttentionProblem* problem) {
    if (problem == nullptr) return 0;
    const size_t shares = scratch_bytes_for(*problem, paged_attention_splits(*problem)), rows = decode_rows_bytes(*problem);
    return shares > rows ? shares : rows;
}

extern "C" int32_t singe_hip_paged_attention_scratch_bf16(void* stream, const uint16_t* query_rows, const uint16_t* key_cache,
                                                          const uint16_t* value_cache, const void* query_offsets,
                                                          const void* page_offsets, const void* pages,
                                                          const void* last_page_lengths, uint16_t* output, float* lse,
                                                          uint32_t* status, void* scratch, size_t scratch_bytes,
                                                          const SingePagedAttentionProblem* problem) {
    const Scratch lent = {scratch, scratch_bytes};
    return paged_attention(SINGE_HIP_BF16, stream, query_rows, key_cache, value_cache, query_offsets, page_offsets, pages,
                           last_page_lengths, output, lse, status, problem, nullptr, &lent);
}

extern "C" int32_t singe_hip_paged_attention_scratch_f16(void* stream, const uint16_t* query_rows, const uint16_t* key_cache,
                                                         const uint16_t* value_cache, const void* query_offsets,
                                                         const void* page_offsets, const void* pages,
                                                         const void* last_page_lengths, uint16_t* output, float* lse,
                                                         uint32_t* status, void* scratch, size_t scratch_bytes,
                                                         const SingePagedAttentionProblem* problem) {
    const Scratch lent = {scratch, scratch_bytes};
    return paged_attention(SINGE_HIP_F16, stream, query_rows, key_cache, value_cache, query_offsets, page_offsets, pages,
                           last_page_lengths, output, lse, status, problem, nullptr, &lent);
}

extern "C" int32_t singe_hip_rotary_paged_attention_bf16(void* stream, const uint16_t* query_rows, const uint16_t* key_cache,
                                                         const uint16_t* value_cache, const void* query_offsets,
                                                         const void* page_offsets, const void* pages,
                                                         const void* last_page_lengths, const void* cos, const void* sin,
                                                         const uint16_t* query_weight, uint16_t* output, float* lse,
                                                         uint32_t* status, const SingePagedAttentionProblem* problem,
                                                         const SingeQueryRotation* rotation) {
    const Rotation operands = {cos, sin, query_weight, rotation};
    return paged_attention(SINGE_HIP_BF16, stream, query_rows, key_cache, value_cache, query_offsets, page_offsets, pages,
                           last_page_lengths, output, lse, status, problem, &operands);
}

extern "C" int32_t singe_hip_rotary_paged_attention_f16(void* stream, const uint16_t* query_rows, const uint16_t* key_cache,
                                                        const uint16_t* value_cache, const void* query_offsets,
                                                        const void* page_offsets, const void* pages,
                                                        const void* last_page_lengths, const void* cos, const void* sin,
                                                        const uint16_t* query_weight, uint16_t* output, float* lse,
                                                        uint32_t* status, const SingePagedAttentionProblem* problem,
                                                        const SingeQueryRotation* rotation) {
    const Rotation operands = {cos, sin, query_weight, rotation};
    return paged_attention(SINGE_HIP_F16, stream, query_rows, key_cache, value_cache, query_offsets, page_offsets, pages,
                           last_page_lengths, output, lse, status, problem, &operands);
}

extern "C" int32_t singe_hip_paged_attention_bf16(void* stream, const uint16_t* query_rows, const uint16_t* key_cache,
                                                  const uint16_t* value_cache, const void* query_offsets,
                                                  const void* page_offsets, const void* pages,
                                                  const void* last_page_lengths, uint16_t* output, float* lse,
                                                  uint32_t* status, const SingePagedAttentionProblem* problem) {
    return paged_attention(SINGE_HIP_BF16, stream, query_rows, key_cache, value_cache, query_offsets, page_offsets, pages,
                           last_page_lengths, output, lse, status, problem);
}

extern "C" int32_t singe_hip_paged_attention_f32(void* stream, const float* query_rows, const float* key_cache,
                                                 const float* value_cache, const void* query_offsets, const void* page_offsets,
                                                 const void* pages, const void* last_page_lengths, float* output, float* lse,
                                                 uint32_t* status, const SingePagedAttentionProblem* problem) {
    return paged_attention(SINGE_HIP_F32, stream, query_rows, key_cache, value_cache, query_offsets, page_offsets, pages,
                           last_page_lengths, output, lse, status, problem);
}

extern "C" int32_t singe_hip_paged_attention_f64(void* stream, const double* query_rows, const double* key_cache,
                                                 const double* value_cache, const void* query_offsets, const void* page_offsets,
                                                 const void* pages, const void* last_page_lengths, double* output, float* lse,
                                                 uint32_t* status, const SingePagedAttentionProblem* problem) {
    return paged_attention(SINGE_HIP_F64, stream, query_rows, key_cache, value_cache, query_offsets, page_offsets, pages,
                           last_page_lengths, output, lse, status, problem);
}

extern "C" int32_t singe_hip_paged_attention_f16(void* stream, const uint16_t* query_rows, const uint16_t* key_cache,
                                                 const uint16_t* value_cache, const void* query_offsets, const void* page_offsets,
                                                 const void* pages, const void* last_page_lengths, uint16_t* output, float* lse,
                                                 uint32_t* status, const SingePagedAttentionProblem* problem) {
    return paged_attention(SINGE_HIP_F16, stream, query_rows, key_cache, value_cache, query_offsets, page_offsets, pages,
                           last_page_lengths, output, lse, status, problem);
}

// validate_paged_kv_prefill_attention_config (singe-kernel/src/cuda/attention/mod.rs:2987-3011).
extern "C" int32_t singe_hip_paged_kv_prefill_attention_config_validate(const SingePagedKvPrefillAttentionConfig* config) {
    if (config == nullptr) return fail(SINGE_HIP_NULL_POINTER, "config");
    const SingePagedKvPrefillAttentionConfig& c = *config;
    if (c.batch == 0 || c.total_query_tokens == 0 || c.heads == 0 || c.kv_heads == 0 || c.head_dim == 0 || c.block_size == 0 ||
        c.physical_blocks == 0 || c.block_table_batch_stride == 0 || c.heads % c.kv_heads != 0 || !std::isfinite(c.scale))
        return fail(SINGE_HIP_INVALID_LENGTH, "config");
    const size_t extents[] = {c.batch, c.total_query_tokens, c.heads, c.kv_heads, c.head_dim, c.block_size, c.physical_blocks,
                              c.block_table_batch_stride};
    for (size_t extent : extents)
        if (!fits_i32(extent)) return fail(SINGE_HIP_LENGTH_EXCEEDS_I32, "config");
    return 0;
}

// paged_kv_prefill_attention_bf16 (singe-kernel/src/cuda/attention/paged.rs:370-420); lengths checked
// in the order of PagedKvPrefillAttentionConfig::validate_lengths (mod.rs:786-818).
namespace {
int32_t paged_kv_prefill(
    bool f16, void* stream, uint16_t* out, size_t out_len, float* lse, size_t lse_len, const uint16_t* query, size_t query_len,
    const uint16_t* key_cache, size_t key_cache_len, const uint16_t* value_cache, size_t value_cache_len,
    const int32_t* actual_seq_lens_q, size_t actual_seq_lens_q_len, const int32_t* actual_seq_lens_kv,
    size_t actual_seq_lens_kv_len, const int32_t* actual_seq_offsets, size_t actual_seq_offsets_len,
    const uint32_t* block_table, size_t block_table_len, const SingePagedKvPrefillAttentionConfig* config);
}  // namespace

extern "C" int32_t singe_hip_paged_kv_prefill_attention_bf16(
    void* stream, uint16_t* out, size_t out_len, float* lse, size_t lse_len, const uint16_t* query, size_t query_len,
    const uint16_t* key_cache, size_t key_cache_len, const uint16_t* value_cache, size_t value_cache_len,
    const int32_t* actual_seq_lens_q, size_t actual_seq_lens_q_len, const int32_t* actual_seq_lens_kv,
    size_t actual_seq_lens_kv_len, const int32_t* actual_seq_offsets, size_t actual_seq_offsets_len,
    const uint32_t* block_table, size_t block_table_len, const SingePagedKvPrefillAttentionConfig* config) {
    return paged_kv_prefill(false, stream, out, out_len, lse, lse_len, query, query_len, key_cache, key_cache_len, value_cache,
                            value_cache_len, actual_seq_lens_q, actual_seq_lens_q_len, actual_seq_lens_kv, actual_seq_lens_kv_len,
                            actual_seq_offsets, actual_seq_offsets_len, block_table, block_table_len, config);
}

// paged_kv_prefill_attention_f16: the same kernel on f16 operands.
extern "C" int32_t singe_hip_paged_kv_prefill_attention_f16(
    void* stream, uint16_t* out, size_t out_len, float* lse, size_t lse_len, const uint16_t* query, size_t query_len,
    const uint16_t* key_cache, size_t key_cache_len, const uint16_t* value_cache, size_t value_cache_len,
    const int32_t* actual_seq_lens_q, size_t actual_seq_lens_q_len, const int32_t* actual_seq_lens_kv,
    size_t actual_seq_lens_kv_len, const int32_t* actual_seq_offsets, size_t actual_seq_offsets_len,
    const uint32_t* block_table, size_t block_table_len, const SingePagedKvPrefillAttentionConfig* config) {
    return paged_kv_prefill(true, stream, out, out_len, lse, lse_len, query, query_len, key_cache, key_cache_len, value_cache,
                            value_cache_len, actual_seq_lens_q, actual_seq_lens_q_len, actual_seq_lens_kv, actual_seq_lens_kv_len,
                            actual_seq_offsets, actual_seq_offsets_len, block_table, block_table_len, config);
}

namespace {
int32_t paged_kv_prefill(
    bool f16, void* stream, uint16_t* out, size_t out_len, float* lse, size_t lse_len, const uint16_t* query, size_t query_len,
    const uint16_t* key_cache, size_t key_cache_len, const uint16_t* value_cache, size_t value_cache_len,
    const int32_t* actual_seq_lens_q, size_t actual_seq_lens_q_len, const int32_t* actual_seq_lens_kv,
    size_t actual_seq_lens_kv_len, const int32_t* actual_seq_offsets, size_t actual_seq_offsets_len,
    const uint32_t* block_table, size_t block_table_len, const SingePagedKvPrefillAttentionConfig* config) {
    if (int32_t status = singe_hip_paged_kv_prefill_attention_config_validate(config)) return status;
    const SingePagedKvPrefillAttentionConfig& c = *config;
    size_t output_len = 0, lse_needed = 0, block_len = 0, cache_len = 0, table_len = 0;
    if (!checked_mul(c.total_query_tokens, c.heads, &lse_needed) || !checked_mul(lse_needed, c.head_dim, &output_len) ||
        !checked_mul(c.block_size, c.kv_heads, &block_len) || !checked_mul(block_len, c.head_dim, &block_len) ||
        !checked_mul(c.physical_blocks, block_len, &cache_len) || !checked_mul(c.batch, c.block_table_batch_stride, &table_len))
        return fail(SINGE_HIP_SIZE_OVERFLOW, "config");
    if (int32_t s = ensure_len_at_least("out", out_len, output_len)) return s;
    if (int32_t s = ensure_len_at_least("lse", lse_len, lse_needed)) return s;
    if (int32_t s = ensure_len_at_least("query", query_len, output_len)) return s;
    if (int32_t s = ensure_len_at_least("key_cache", key_cache_len, cache_len)) return s;
    if (int32_t s = ensure_len_at_least("value_cache", value_cache_len, cache_len)) return s;
    if (int32_t s = ensure_len_at_least("actual_seq_lens_q", actual_seq_lens_q_len, c.batch)) return s;
    if (int32_t s = ensure_len_at_least("actual_seq_lens_kv", actual_seq_lens_kv_len, c.batch)) return s;
    if (int32_t s = ensure_len_at_least("actual_seq_offsets", actual_seq_offsets_len, c.batch)) return s;
    if (int32_t s = ensure_len_at_least("block_table", block_table_len, table_len)) return s;
    if (block_len > 0xffffffffull) return fail(SINGE_HIP_UNSUPPORTED_CONFIGURATION, "a cache block beyond 4 Gi elements");
    const void* pointers[] = {out, lse, query, key_cache, value_cache, actual_seq_lens_q, actual_seq_lens_kv, actual_seq_offsets, block_table};
    const char* names[] = {"out", "lse", "query", "key_cache", "value_cache", "actual_seq_lens_q", "actual_seq_lens_kv",
                           "actual_seq_offsets", "block_table"};
    for (int i = 0; i < 9; ++i)
        if (pointers[i] == nullptr) return fail(SINGE_HIP_NULL_POINTER, names[i]);
    // The matrix-core kernels are built for head dimensions 128 and 64; the others (up to 256) take the
    // one-wave-per-row kernel.
    if (!has_matrix_core_build(static_cast<long long>(c.head_dim)))
        return paged_table_general(f16 ? SINGE_HIP_F16 : SINGE_HIP_BF16, stream,
                                   f16 ? "paged_kv_prefill_attention_f16" : "paged_kv_prefill_attention_bf16", query, key_cache,
                                   value_cache, actual_seq_offsets, actual_seq_lens_q, actual_seq_lens_kv, block_table, out, lse,
                                   c.total_query_tokens, c.batch, c.heads, c.kv_heads, c.head_dim, c.block_size, c.physical_blocks,
                                   c.block_table_batch_stride, c.causal != 0, c.scale);

    const uint64_t groups = c.heads / c.kv_heads;
    PagedAttentionArgs args;
    args.query_rows = query;
    args.key_cache = key_cache;
    args.value_cache = value_cache;
    args.query_offsets = actual_seq_offsets;
    args.page_offsets = nullptr;
    args.pages = block_table;
    args.last_page_lengths = actual_seq_lens_kv;
    args.query_lengths = actual_seq_lens_q;
    args.output = out;
    args.lse = lse;
    args.status = nullptr;
    args.window = -1;
    args.tokens = static_cast<uint32_t>(c.total_query_tokens);
    args.heads = static_cast<uint32_t>(c.heads);
    args.kv_heads = static_cast<uint32_t>(c.kv_heads);
    args.page_size = static_cast<uint32_t>(c.block_size);
    args.sequences = static_cast<uint32_t>(c.batch);
    args.cache_pages = static_cast<uint32_t>(c.physical_blocks);
    args.page_table = static_cast<uint32_t>(c.block_table_batch_stride);
    const RowTileGrid tiling = grid_of(c.total_query_tokens, c.batch, groups, c.kv_heads);
    if (tiling.row_tiles > 0xffffffffull) return fail(SINGE_HIP_UNSUPPORTED_CONFIGURATION, "too many row tiles");
    args.row_tiles = static_cast<uint32_t>(tiling.row_tiles);
    args.compact = tiling.compact;
    args.longest_first = tiling.longest_first;
    args.causal = c.causal ? 1u : 0u;
    args.page_shift = -1;
    for (int shift = 0; shift < 31; ++shift)
        if ((size_t{1} << shift) == c.block_size) args.page_shift = shift;
    args.scale_log2e = c.scale * 1.4426950408889634074f;
    args.softcap_scale = 0.0f;
    args.softcap_log2e = 0.0f;
    const uint64_t blocks = tiling.blocks;
    if (blocks > 0x7fffffffull) return fail(SINGE_HIP_UNSUPPORTED_CONFIGURATION, "too many workgroups");
    const KernelId kernel = static_cast<KernelId>((f16 ? kPagedKvPrefillF16 : kPagedKvPrefill) + (args.page_shift >= 4 ? 1 : 0));
    return launch(at_head_dim(kernel, static_cast<long long>(c.head_dim)), static_cast<unsigned>(blocks), 1, 1, 256, stream, args);
}
}  // namespace
