// Host side of paged decode: the reference's validation (singe-kernel/src/cuda/attention/mod.rs:
// 711-743, 2963-2985), the split-KV scratch layout, and the two launches.
#include <atomic>
#include <cmath>
#include <limits>

#include "kernel_args.h"
#include "module.h"
#include "singe_hip_attention.h"
#include "static_scratch.h"
#include "thread_options.h"
#include "validate.h"

using namespace singe_hip;

namespace {

std::atomic<uint32_t> g_forced_workers{0};
std::atomic<bool> g_relaxed{false};

int32_t decode(void* stream, uint16_t* out, size_t out_len, const uint16_t* query, size_t query_len,
               const void* key_cache, size_t key_cache_len, const void* value_cache, size_t value_cache_len,
               const float* key_scales, size_t key_scales_len, const float* value_scales, size_t value_scales_len,
               bool fp8, const int32_t* actual_seq_lens, size_t actual_seq_lens_len, const uint32_t* block_table,
               size_t block_table_len, void* workspace, size_t workspace_bytes,
               const SingePagedKvDecodeAttentionConfig* config, uint32_t phases, bool f16 = false);

constexpr unsigned kWavesPerWorkgroup = 8;

// How the flat list of 32-key tiles is shared out (see paged_decode.hip).  `span` is the most query heads a wave
// carries: 8 (the one-hot form, and the dense form of fp8 caches), or 16 (the dense form of bf16 / f16 caches).
struct Plan {
    uint32_t head_groups;     // waves per kv head: ceil(group / span)
    uint32_t heads_per_wave;  // min(group, span)
    uint32_t groups;          // 1 or 2 groups of four query heads per wave
    uint32_t work;            // kv_heads * head_groups
    uint32_t work_per_wg;     // min(work, 8)
    uint32_t workers_per_wg;  // 8 / work_per_wg
    uint32_t workers;         // ranges per (kv head, head group)
    uint32_t grid_x, grid_y;
    size_t lse_offset, out_offset, bytes;  // scratch layout, 256-byte aligned regions
};

size_t align256(size_t bytes) { return (bytes + 255) / 256 * 256; }

// One workgroup of eight waves per compute unit, so every wave of the chip gets one equal range and
// the launch finishes in a single round.
Plan make_plan(const SingePagedKvDecodeAttentionConfig& c, size_t span = 8) {
    Plan p;
    const size_t group = c.heads / c.kv_heads;
    p.head_groups = static_cast<uint32_t>((group + span - 1) / span);
    p.heads_per_wave = static_cast<uint32_t>(group < span ? group : span);
    p.groups = p.heads_per_wave <= 4 ? 1 : 2;
    p.work = static_cast<uint32_t>(c.kv_heads) * p.head_groups;
    p.work_per_wg = p.work < kWavesPerWorkgroup ? p.work : kWavesPerWorkgroup;
    p.workers_per_wg = kWavesPerWorkgroup / p.work_per_wg;
    p.grid_y = (p.work + p.work_per_wg - 1) / p.work_per_wg;
    const uint32_t forced = effective_count(thread_options().decode_workers, g_forced_workers.load(std::memory_order_relaxed));
    if (forced != 0) {
        p.grid_x = (forced + p.workers_per_wg - 1) / p.workers_per_wg;
    } else {
        p.grid_x = compute_units() / p.grid_y;
        if (p.grid_x == 0) p.grid_x = 1;
    }
    p.workers = p.grid_x * p.workers_per_wg;
    const size_t rows = static_cast<size_t>(p.work) * (p.workers + c.batch) * p.heads_per_wave;
    p.lse_offset = align256((c.batch + 3) * sizeof(uint32_t));
    p.out_offset = p.lse_offset + align256(rows * sizeof(float));
    p.bytes = p.out_offset + align256(rows * c.head_dim * sizeof(float));
    return p;
}

// What singe_hip_paged_kv_decode_attention_workspace_bytes asks for: the config does not say the cache's type, so
// enough for either form.
size_t workspace_need(const SingePagedKvDecodeAttentionConfig& c) {
    const size_t narrow = make_plan(c, 8).bytes, wide = make_plan(c, 16).bytes;
    return narrow > wide ? narrow : wide;
}

int32_t validate_config(const SingePagedKvDecodeAttentionConfig& c) {
    if (c.batch == 0 || c.heads == 0 || c.kv_heads == 0 || c.head_dim == 0 || c.block_size == 0 ||
        c.physical_blocks == 0 || c.block_table_batch_stride == 0 || c.heads % c.kv_heads != 0 ||
        !std::isfinite(c.scale))
        return fail(SINGE_HIP_INVALID_LENGTH, "config");
    const size_t extents[] = {c.batch, c.heads, c.kv_heads, c.head_dim, c.block_size, c.physical_blocks,
                              c.block_table_batch_stride};
    for (size_t extent : extents)
        if (!fits_i32(extent)) return fail(SINGE_HIP_LENGTH_EXCEEDS_I32, "config");
    return 0;
}

}  // namespace

extern "C" {

void singe_hip_set_decode_workers(uint32_t workers) { g_forced_workers.store(workers, std::memory_order_relaxed); }

uint32_t singe_hip_decode_workers(const SingePagedKvDecodeAttentionConfig* config) {
    if (config == nullptr || validate_config(*config) != 0) return 0;
    return make_plan(*config).workers;
}

int32_t singe_hip_paged_kv_decode_attention_config_validate(const SingePagedKvDecodeAttentionConfig* config) {
    if (config == nullptr) return fail(SINGE_HIP_NULL_POINTER, "config");
    return validate_config(*config);
}

size_t singe_hip_paged_kv_decode_attention_workspace_bytes(const SingePagedKvDecodeAttentionConfig* config) {
    if (config == nullptr || validate_config(*config) != 0) return 0;
    size_t rows = 0, elements = 0;
    if (!checked_mul(config->batch, config->heads, &rows) || !checked_mul(rows, config->head_dim, &elements)) return 0;
    return workspace_need(*config);
}

int32_t singe_hip_paged_kv_decode_attention_bf16(
    void* stream, uint16_t* out, size_t out_len, const uint16_t* query, size_t query_len,
    const uint16_t* key_cache, size_t key_cache_len, const uint16_t* value_cache, size_t value_cache_len,
    const int32_t* actual_seq_lens, size_t actual_seq_lens_len, const uint32_t* block_table,
    size_t block_table_len, void* workspace, size_t workspace_bytes,
    const SingePagedKvDecodeAttentionConfig* config) {
    return singe_hip_paged_kv_decode_attention_phases_bf16(
        stream, out, out_len, query, query_len, key_cache, key_cache_len, value_cache, value_cache_len,
        actual_seq_lens, actual_seq_lens_len, block_table, block_table_len, workspace, workspace_bytes, config,
        SINGE_HIP_DECODE_SPLIT | SINGE_HIP_DECODE_REDUCE);
}

int32_t singe_hip_paged_kv_decode_attention_phases_bf16(
    void* stream, uint16_t* out, size_t out_len, const uint16_t* query, size_t query_len,
    const uint16_t* key_cache, size_t key_cache_len, const uint16_t* value_cache, size_t value_cache_len,
    const int32_t* actual_seq_lens, size_t actual_seq_lens_len, const uint32_t* block_table,
    size_t block_table_len, void* workspace, size_t workspace_bytes,
    const SingePagedKvDecodeAttentionConfig* config, uint32_t phases) {
    return decode(stream, out, out_len, query, query_len, key_cache, key_cache_len, value_cache, value_cache_len,
                  nullptr, 0, nullptr, 0, false, actual_seq_lens, actual_seq_lens_len, block_table, block_table_len,
                  workspace, workspace_bytes, config, phases);
}

// The bf16 decode on the library's fixed device scratch: allocates nothing (no counterpart in the reference).
int32_t singe_hip_paged_kv_decode_attention_no_alloc_bf16(
    void* stream, uint16_t* out, size_t out_len, const uint16_t* query, size_t query_len,
    const uint16_t* key_cache, size_t key_cache_len, const uint16_t* value_cache, size_t value_cache_len,
    const int32_t* actual_seq_lens, size_t actual_seq_lens_len, const uint32_t* block_table,
    size_t block_table_len, const SingePagedKvDecodeAttentionConfig* config) {
    if (config == nullptr) return fail(SINGE_HIP_NULL_POINTER, "config");
    if (int32_t status = validate_config(*config)) return status;
    const size_t need = workspace_need(*config);
    if (need > SINGE_HIP_STATIC_SCRATCH_BYTES)
        return fail(SINGE_HIP_LENGTH_TOO_SHORT, "static scratch", need, SINGE_HIP_STATIC_SCRATCH_BYTES);
    void* scratch = nullptr;
    size_t scratch_bytes = 0;
    if (int status = static_scratch(&scratch, &scratch_bytes)) return fail(status, "hipGetSymbolAddress(static scratch)");
    return decode(stream, out, out_len, query, query_len, key_cache, key_cache_len, value_cache, value_cache_len,
                  nullptr, 0, nullptr, 0, false, actual_seq_lens, actual_seq_lens_len, block_table, block_table_len,
                  scratch, scratch_bytes, config, SINGE_HIP_DECODE_SPLIT | SINGE_HIP_DECODE_REDUCE);
}

// paged_kv_decode_attention_f16 (singe-kernel/src/cuda/attention/paged.rs): the bf16 kernels on f16 operands.
int32_t singe_hip_paged_kv_decode_attention_f16(
    void* stream, uint16_t* out, size_t out_len, const uint16_t* query, size_t query_len,
    const uint16_t* key_cache, size_t key_cache_len, const uint16_t* value_cache, size_t value_cache_len,
    const int32_t* actual_seq_lens, size_t actual_seq_lens_len, const uint32_t* block_table,
    size_t block_table_len, void* workspace, size_t workspace_bytes,
    const SingePagedKvDecodeAttentionConfig* config) {
    return decode(stream, out, out_len, query, query_len, key_cache, key_cache_len, value_cache, value_cache_len,
                  nullptr, 0, nullptr, 0, false, actual_seq_lens, actual_seq_lens_len, block_table, block_table_len,
                  workspace, workspace_bytes, config, SINGE_HIP_DECODE_SPLIT | SINGE_HIP_DECODE_REDUCE, true);
}

int32_t singe_hip_paged_kv_decode_attention_f8e4m3kv_bf16(
    void* stream, uint16_t* out, size_t out_len, const uint16_t* query, size_t query_len,
    const uint8_t* key_cache, size_t key_cache_len, const uint8_t* value_cache, size_t value_cache_len,
    const float* key_scales, size_t key_scales_len, const float* value_scales, size_t value_scales_len,
    const int32_t* actual_seq_lens, size_t actual_seq_lens_len, const uint32_t* block_table,
    size_t block_table_len, void* workspace, size_t workspace_bytes,
    const SingePagedKvDecodeAttentionConfig* config, uint32_t phases) {
    return decode(stream, out, out_len, query, query_len, key_cache, key_cache_len, value_cache, value_cache_len,
                  key_scales, key_scales_len, value_scales, value_scales_len, true, actual_seq_lens,
                  actual_seq_lens_len, block_table, block_table_len, workspace, workspace_bytes, config, phases);
}

}  // extern "C"

namespace {

int32_t decode(
    void* stream, uint16_t* out, size_t out_len, const uint16_t* query, size_t query_len,
    const void* key_cache, size_t key_cache_len, const void* value_cache, size_t value_cache_len,
    const float* key_scales, size_t key_scales_len, const float* value_scales, size_t value_scales_len, bool fp8,
    const int32_t* actual_seq_lens, size_t actual_seq_lens_len, const uint32_t* block_table,
    size_t block_table_len, void* workspace, size_t workspace_bytes,
    const SingePagedKvDecodeAttentionConfig* config, uint32_t phases, bool f16) {
    if (config == nullptr) return fail(SINGE_HIP_NULL_POINTER, "config");
    const SingePagedKvDecodeAttentionConfig& c = *config;
    // PagedKvDecodeAttentionConfig::validate_lengths (mod.rs:711-743), in its order.
    if (int32_t status = validate_config(c)) return status;
    size_t output_len = 0, cache_block_len = 0, cache_len = 0, table_len = 0;
    if (!checked_mul(c.batch, c.heads, &output_len) || !checked_mul(output_len, c.head_dim, &output_len))
        return fail(SINGE_HIP_SIZE_OVERFLOW, "output");
    if (!checked_mul(c.block_size, c.kv_heads, &cache_block_len) || !checked_mul(cache_block_len, c.head_dim, &cache_block_len) ||
        !checked_mul(c.physical_blocks, cache_block_len, &cache_len))
        return fail(SINGE_HIP_SIZE_OVERFLOW, "cache");
    if (int32_t status = ensure_len_at_least("out", out_len, output_len)) return status;
    if (int32_t status = ensure_len_at_least("query", query_len, output_len)) return status;
    if (int32_t status = ensure_len_at_least("key_cache", key_cache_len, cache_len)) return status;
    if (int32_t status = ensure_len_at_least("value_cache", value_cache_len, cache_len)) return status;
    if (int32_t status = ensure_len_at_least("actual_seq_lens", actual_seq_lens_len, c.batch)) return status;
    if (!checked_mul(c.batch, c.block_table_batch_stride, &table_len)) return fail(SINGE_HIP_SIZE_OVERFLOW, "block_table");
    if (int32_t status = ensure_len_at_least("block_table", block_table_len, table_len)) return status;
    if (fp8) {
        size_t scales = 0;
        if (!checked_mul(c.physical_blocks, c.kv_heads, &scales)) return fail(SINGE_HIP_SIZE_OVERFLOW, "scales");
        if (int32_t status = ensure_len_at_least("key_scales", key_scales_len, scales)) return status;
        if (int32_t status = ensure_len_at_least("value_scales", value_scales_len, scales)) return status;
        if (key_scales == nullptr) return fail(SINGE_HIP_NULL_POINTER, "key_scales");
        if (value_scales == nullptr) return fail(SINGE_HIP_NULL_POINTER, "value_scales");
    }
    // A DevicePointer is never null (singe-kernel/src/cuda/interop.rs:5-31).
    const void* pointers[] = {out, query, key_cache, value_cache, actual_seq_lens, block_table};
    const char* names[] = {"out", "query", "key_cache", "value_cache", "actual_seq_lens", "block_table"};
    for (int i = 0; i < 6; ++i)
        if (pointers[i] == nullptr) return fail(SINGE_HIP_NULL_POINTER, names[i]);

    // What the gfx950 kernels take (the reference's cuTile kernels take head_dim 4..64 only and return
    // UnsupportedWidth otherwise: singe-kernel/src/cuda/cutile/attention/paged.rs:799-810).
    if (fp8 && c.head_dim != 128) return fail(SINGE_HIP_UNSUPPORTED_WIDTH, "paged_kv_decode_attention_f8e4m3kv_bf16", c.head_dim, 0);
    // The matrix-core kernels are built for the multiples of 16 up to 128 (fp8 caches: 128); the other head dimensions
    // (the reference's own kernels take 4 to 64 here, this library up to 256) run on the one-wave-per-row kernel and
    // need no workspace.
    if (!has_decode_build(c.head_dim)) {
        if (!(phases & SINGE_HIP_DECODE_REDUCE)) return 0;  // nothing is left in the workspace at these widths
        uint64_t reach_keys = static_cast<uint64_t>(c.block_table_batch_stride) * c.block_size;
        if (!fits_i32(reach_keys)) return fail(SINGE_HIP_LENGTH_EXCEEDS_I32, "block_table_batch_stride * block_size");
        return paged_table_general(f16 ? SINGE_HIP_F16 : SINGE_HIP_BF16, stream,
                                   f16 ? "paged_kv_decode_attention_f16" : "paged_kv_decode_attention_bf16", query, key_cache,
                                   value_cache, nullptr, nullptr, actual_seq_lens, block_table, out, nullptr, c.batch, c.batch,
                                   c.heads, c.kv_heads, c.head_dim, c.block_size, c.physical_blocks, c.block_table_batch_stride,
                                   false, c.scale);
    }
    PagedDecodeLaunch launch_of;
    launch_of.stream = stream, launch_of.out = out, launch_of.query = query, launch_of.key_cache = key_cache, launch_of.value_cache = value_cache;
    launch_of.key_scales = key_scales, launch_of.value_scales = value_scales, launch_of.fp8 = fp8, launch_of.f16 = f16;
    launch_of.actual_seq_lens = actual_seq_lens, launch_of.block_table = block_table, launch_of.workspace = workspace;
    launch_of.workspace_bytes = workspace_bytes, launch_of.phases = phases;
    return launch_paged_decode(c, launch_of);
}

}  // namespace

namespace singe_hip {

size_t paged_decode_workspace_bytes(const SingePagedKvDecodeAttentionConfig& c) { return workspace_need(c); }

// The two launches of the matrix-core decode (a multiple of 16 up to 128), after the entry point's checks.
int32_t launch_paged_decode(const SingePagedKvDecodeAttentionConfig& c, const PagedDecodeLaunch& l) {
    void* const stream = l.stream;
    const bool fp8 = l.fp8, f16 = l.f16;
    const uint32_t phases = l.phases;
    void* const workspace = l.workspace;
    const size_t workspace_bytes = l.workspace_bytes;
    const bool narrow = c.head_dim != 128;  // a narrower build of the same kernels
    uint64_t reach = static_cast<uint64_t>(c.block_table_batch_stride) * c.block_size;
    if (!fits_i32(reach)) return fail(SINGE_HIP_LENGTH_EXCEEDS_I32, "block_table_batch_stride * block_size");

    // bf16 caches take the one-hot form, fp8 caches the dense form (see paged_decode.hip); and so do bf16 / f16
    // caches with more than four query heads per kv head at head_dim 128, where the one-hot form would carry two
    // groups per wave, as long as the batch's prefix sums fit beside that form's 132 KiB of staging in LDS.
    // (the kernel keeps the sequences' tile prefix sums and lengths in LDS, and their rows' starts when rows have their own lengths)
    const unsigned prefix_bytes = static_cast<unsigned>(((l.row_starts == nullptr ? 2 : l.row_begins == nullptr ? 3 : 4) * c.batch + 1) * sizeof(uint32_t));
    constexpr unsigned kWideStagingBytes = 135168, kLdsBytes = 160 * 1024;
    const bool wide = !fp8 && !narrow && c.heads / c.kv_heads > 4 && kWideStagingBytes + prefix_bytes <= kLdsBytes;
    const Plan plan = make_plan(c, wide || fp8 ? 16 : 8);  // (the dense form of fp8 caches has its Q^T in registers and no such limit)
    if (workspace == nullptr) return fail(SINGE_HIP_NULL_POINTER, "workspace");
    if (workspace_bytes < plan.bytes) return fail(SINGE_HIP_LENGTH_TOO_SHORT, "workspace", plan.bytes, workspace_bytes);
    if (c.batch > 8000) return fail(SINGE_HIP_UNSUPPORTED_CONFIGURATION, "more than 8000 sequences per call");
    unsigned char* scratch = static_cast<unsigned char*>(workspace);

    DecodeArgs args;
    args.query = l.query;
    args.key_cache = l.key_cache;
    args.value_cache = l.value_cache;
    args.key_scales = l.key_scales;
    args.value_scales = l.value_scales;
    args.actual_seq_lens = l.actual_seq_lens;
    args.block_table = l.block_table;
    args.row_starts = l.row_starts;
    args.row_begins = l.row_starts != nullptr ? l.row_begins : nullptr;
    args.meta = reinterpret_cast<uint32_t*>(scratch);
    args.partial_lse = reinterpret_cast<float*>(scratch + plan.lse_offset);
    args.partial_out = reinterpret_cast<float*>(scratch + plan.out_offset);
    args.batch = static_cast<uint32_t>(c.batch);
    args.heads = static_cast<uint32_t>(c.heads);
    args.kv_heads = static_cast<uint32_t>(c.kv_heads);
    args.block_size = static_cast<uint32_t>(c.block_size);
    args.block_shift = -1;
    for (int shift = 0; shift < 31; ++shift)
        if ((static_cast<size_t>(1) << shift) == c.block_size) args.block_shift = shift;
    args.physical_blocks = static_cast<uint32_t>(c.physical_blocks);
    args.block_table_batch_stride = static_cast<uint32_t>(c.block_table_batch_stride);
    args.workers = plan.workers;
    args.workers_per_wg = plan.workers_per_wg;
    args.work_per_wg = plan.work_per_wg;
    args.head_groups = plan.head_groups;
    args.heads_per_wave = plan.heads_per_wave;
    args.scale_log2e = c.scale * 1.4426950408889634074f;

    const bool aligned = c.block_size % 16 == 0;
    const KernelId kernel = fp8    ? static_cast<KernelId>(kDecodeF8Wide + (aligned ? 0 : 1) + (effective_relaxed(g_relaxed.load(std::memory_order_relaxed)) ? 2 : 0))
                            : wide ? static_cast<KernelId>(kDecodeWide + (aligned ? 0 : 1) + (f16 ? 2 : 0))
                                   : static_cast<KernelId>((f16 ? kDecodeF16 : kDecodeBf16) + (aligned ? 0 : 2) + (plan.groups == 2 ? 1 : 0));
    if (phases & SINGE_HIP_DECODE_SPLIT)
        if (int32_t status = launch(narrow ? decode_at_head_dim(kernel, c.head_dim) : kernel, plan.grid_x, plan.grid_y, 1, 64 * kWavesPerWorkgroup, stream, args,
                                    prefix_bytes))
            return status;
    if (!(phases & SINGE_HIP_DECODE_REDUCE)) return 0;

    CombineArgs combine;
    combine.out = l.out;
    combine.lse = l.lse;
    combine.row_lengths = l.row_starts != nullptr ? l.actual_seq_lens : nullptr;
    combine.partial_out = args.partial_out;
    combine.partial_lse = args.partial_lse;
    combine.meta = args.meta;
    combine.batch = args.batch;
    combine.heads = args.heads;
    combine.kv_heads = args.kv_heads;
    combine.workers = plan.workers;
    combine.head_groups = plan.head_groups;
    combine.heads_per_wave = plan.heads_per_wave;
    // A row has about workers / batch slots: from 32 on, a workgroup of eight waves folds it instead of one wave.
    if (static_cast<size_t>(plan.workers) >= 32 * c.batch) {
        const KernelId many = static_cast<KernelId>(decode_combine_many_at(c.head_dim) + (f16 ? 1 : 0));
        return launch(many, static_cast<unsigned>(c.batch * c.heads), 1, 1, 512, stream, combine);
    }
    // With no more workers than sequences a row has one or two slots, and the kernel that fetches four rows at a time
    // keeps twice the waves in flight.
    if (static_cast<size_t>(plan.workers) <= c.batch) {
        const KernelId few = static_cast<KernelId>(decode_combine_few_at(c.head_dim) + (f16 ? 1 : 0));
        return launch(few, static_cast<unsigned>((c.batch * c.heads + 3) / 4), 1, 1, 256, stream, combine);
    }
    const KernelId merge = f16 ? kDecodeF16Combine : kDecodeCombine;
    return launch(decode_at_head_dim(merge, c.head_dim), static_cast<unsigned>((c.batch * c.heads + 3) / 4), 1, 1, 256, stream, combine);
}

}  // namespace singe_hip

extern "C" {

void singe_hip_set_relaxed_numerics(int32_t relaxed) { g_relaxed.store(relaxed != 0, std::memory_order_relaxed); }
int32_t singe_hip_relaxed_numerics(void) { return effective_relaxed(g_relaxed.load(std::memory_order_relaxed)) ? 1 : 0; }

}  // extern "C"
