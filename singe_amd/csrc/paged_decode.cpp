// Host side of paged decode: the reference's validation (singe-kernel/src/cuda/attention/mod.rs:
// 711-743, 2963-2985), the split-KV scratch layout, and the two launches.
#include <atomic>
#include <cmath>
#include <limits>

#include "kernel_args.h"
#include "module.h"
#include "singe_hip_attention.h"
#include "validate.h"

using namespace singe_hip;

namespace {

std::atomic<uint32_t> g_keys_per_split{0};

constexpr size_t kHeadDim = 128;

uint32_t round_up_32(uint64_t value) { return static_cast<uint32_t>((value + 31) / 32 * 32); }

// Keys per split: about 4096 work units when every sequence is at full reach, so the ~2048 resident
// waves of the chip see two rounds of equal-sized units; never below 128 keys (64 KiB of KV per unit,
// so the 1 KiB partial row stays in the noise) and never above 4096.
uint32_t choose_keys_per_split(const SingePagedKvDecodeAttentionConfig& c) {
    uint32_t forced = g_keys_per_split.load(std::memory_order_relaxed);
    if (forced != 0) return round_up_32(forced);
    uint64_t reach = static_cast<uint64_t>(c.block_table_batch_stride) * c.block_size;
    uint64_t keys = reach * c.batch * c.kv_heads / 4096;
    if (keys < 128) keys = 128;
    if (keys > 4096) keys = 4096;
    return round_up_32(keys);
}

struct Scratch {
    uint32_t keys_per_split;
    uint32_t splits;
    size_t lse_offset;  // bytes, 256-aligned
    size_t bytes;
};

Scratch scratch_layout(const SingePagedKvDecodeAttentionConfig& c) {
    Scratch s;
    s.keys_per_split = choose_keys_per_split(c);
    uint64_t reach = static_cast<uint64_t>(c.block_table_batch_stride) * c.block_size;
    s.splits = static_cast<uint32_t>((reach + s.keys_per_split - 1) / s.keys_per_split);
    size_t rows = c.batch * c.heads * static_cast<size_t>(s.splits);
    s.lse_offset = (rows * c.head_dim * sizeof(float) + 255) / 256 * 256;
    s.bytes = s.lse_offset + (rows * sizeof(float) + 255) / 256 * 256;
    return s;
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

void singe_hip_set_decode_keys_per_split(uint32_t keys) { g_keys_per_split.store(keys, std::memory_order_relaxed); }

uint32_t singe_hip_decode_keys_per_split(const SingePagedKvDecodeAttentionConfig* config) {
    if (config == nullptr || validate_config(*config) != 0) return 0;
    return choose_keys_per_split(*config);
}

int32_t singe_hip_paged_kv_decode_attention_config_validate(const SingePagedKvDecodeAttentionConfig* config) {
    if (config == nullptr) return fail(SINGE_HIP_NULL_POINTER, "config");
    return validate_config(*config);
}

size_t singe_hip_paged_kv_decode_attention_workspace_bytes(const SingePagedKvDecodeAttentionConfig* config) {
    if (config == nullptr || validate_config(*config) != 0) return 0;
    size_t rows = 0, elements = 0;
    if (!checked_mul(config->batch, config->heads, &rows) || !checked_mul(rows, config->head_dim, &elements)) return 0;
    return scratch_layout(*config).bytes;
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
    // A DevicePointer is never null (singe-kernel/src/cuda/interop.rs:5-31).
    const void* pointers[] = {out, query, key_cache, value_cache, actual_seq_lens, block_table};
    const char* names[] = {"out", "query", "key_cache", "value_cache", "actual_seq_lens", "block_table"};
    for (int i = 0; i < 6; ++i)
        if (pointers[i] == nullptr) return fail(SINGE_HIP_NULL_POINTER, names[i]);

    // What the gfx950 kernels take (the reference's cuTile kernels take head_dim 4..64 only and return
    // UnsupportedWidth otherwise: singe-kernel/src/cuda/cutile/attention/paged.rs:799-810).
    if (c.head_dim != kHeadDim) return fail(SINGE_HIP_UNSUPPORTED_WIDTH, "paged_kv_decode_attention_bf16", c.head_dim, 0);
    const size_t group = c.heads / c.kv_heads;
    if (group > 16) return fail(SINGE_HIP_UNSUPPORTED_CONFIGURATION, "more than 16 query heads per kv head");
    uint64_t reach = static_cast<uint64_t>(c.block_table_batch_stride) * c.block_size;
    if (!fits_i32(reach)) return fail(SINGE_HIP_LENGTH_EXCEEDS_I32, "block_table_batch_stride * block_size");

    const Scratch scratch = scratch_layout(c);
    if (workspace == nullptr) return fail(SINGE_HIP_NULL_POINTER, "workspace");
    if (workspace_bytes < scratch.bytes) return fail(SINGE_HIP_LENGTH_TOO_SHORT, "workspace", scratch.bytes, workspace_bytes);
    if (scratch.splits > 65535 || c.kv_heads > 65535 || c.batch > 65535)
        return fail(SINGE_HIP_UNSUPPORTED_CONFIGURATION, "grid extent above 65535");

    DecodeArgs args;
    args.query = query;
    args.key_cache = key_cache;
    args.value_cache = value_cache;
    args.actual_seq_lens = actual_seq_lens;
    args.block_table = block_table;
    args.partial_out = static_cast<float*>(workspace);
    args.partial_lse = reinterpret_cast<float*>(static_cast<unsigned char*>(workspace) + scratch.lse_offset);
    args.heads = static_cast<uint32_t>(c.heads);
    args.kv_heads = static_cast<uint32_t>(c.kv_heads);
    args.block_size = static_cast<uint32_t>(c.block_size);
    args.block_shift = -1;
    for (int shift = 0; shift < 31; ++shift)
        if ((static_cast<size_t>(1) << shift) == c.block_size) args.block_shift = shift;
    args.physical_blocks = static_cast<uint32_t>(c.physical_blocks);
    args.block_table_batch_stride = static_cast<uint32_t>(c.block_table_batch_stride);
    args.splits = scratch.splits;
    args.keys_per_split = scratch.keys_per_split;
    args.scale_log2e = c.scale * 1.4426950408889634074f;

    int padded = 1;
    while (static_cast<size_t>(padded) < group) padded *= 2;
    int column = padded == 1 ? 0 : padded == 2 ? 1 : padded == 4 ? 2 : padded == 8 ? 3 : 4;
    const bool aligned = c.block_size % 16 == 0;
    KernelId kernel = static_cast<KernelId>((aligned ? kDecodeG1B16 : kDecodeG1Any) + column);
    if (phases & SINGE_HIP_DECODE_SPLIT)
        if (int32_t status = launch(kernel, scratch.splits, static_cast<unsigned>(c.kv_heads),
                                    static_cast<unsigned>(c.batch), 64, stream, args))
            return status;
    if (!(phases & SINGE_HIP_DECODE_REDUCE)) return 0;

    CombineArgs combine;
    combine.out = out;
    combine.partial_out = args.partial_out;
    combine.partial_lse = args.partial_lse;
    combine.actual_seq_lens = actual_seq_lens;
    combine.heads = args.heads;
    combine.dim = static_cast<uint32_t>(c.head_dim);
    combine.splits = scratch.splits;
    combine.keys_per_split = scratch.keys_per_split;
    combine.reach = static_cast<uint32_t>(reach);
    return launch(kDecodeCombine, static_cast<unsigned>(c.batch * c.heads), 1, 1, 128, stream, combine);
}

}  // extern "C"
