// Host side of the f32 forms of the two block-table ops: paged_kv_decode_attention_f32 and
// paged_kv_prefill_attention_f32 (singe-kernel/src/cuda/attention/paged.rs; CPU forms
// singe-kernel/src/cpu/attention.rs:1172-1341), validated as the bf16 entry points are
// (PagedKvDecodeAttentionConfig::validate_lengths, mod.rs:711-743; PagedKvPrefillAttentionConfig::validate_lengths,
// mod.rs:786-818) and run on the vector-unit row kernels of attention_rows_f32.hip.
#include <algorithm>
#include <cmath>

#include "kernel_args.h"
#include "module.h"
#include "singe_hip_attention.h"
#include "validate.h"

using namespace singe_hip;

namespace {

// Index of the row kernel for a head dimension (4, 8, ..., 256), or -1.
int width_index(size_t head_dim) {
    const size_t widths[] = {4, 8, 16, 32, 64, 128, 256};
    for (int i = 0; i < 7; ++i)
        if (head_dim == widths[i]) return i;
    return -1;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Key splits of a decode call: enough workgroups for about four per compute unit, at most 64 (the reduce kernel
// walks them serially) and never more than the table can hold keys for.
size_t decode_splits(const SingePagedKvDecodeAttentionConfig& c) {
    const size_t units = c.batch * c.kv_heads;
    const size_t wanted = (4 * static_cast<size_t>(compute_units()) + units - 1) / units;
    const size_t longest = c.block_table_batch_stride * c.block_size;
    return std::max<size_t>(1, std::min<size_t>({wanted, 64, longest}));
}

}  // namespace

extern "C" {

size_t singe_hip_paged_kv_decode_attention_f32_workspace_bytes(const SingePagedKvDecodeAttentionConfig* config) {
    if (config == nullptr || singe_hip_paged_kv_decode_attention_config_validate(config) != 0) return 0;
    size_t rows = 0, values = 0;
    if (!checked_mul(config->batch, config->heads, &rows) || !checked_mul(rows, 64, &rows) ||
        !checked_mul(rows, config->head_dim + 1, &values) || !checked_mul(values, sizeof(float), &values))
        return 0;
    return values;
}

int32_t singe_hip_paged_kv_decode_attention_f32(void* stream, float* out, size_t out_len, const float* query, size_t query_len,
                                                const float* key_cache, size_t key_cache_len, const float* value_cache,
                                                size_t value_cache_len, const int32_t* actual_seq_lens,
                                                size_t actual_seq_lens_len, const uint32_t* block_table, size_t block_table_len,
                                                void* workspace, size_t workspace_bytes,
                                                const SingePagedKvDecodeAttentionConfig* config) {
    if (int32_t status = singe_hip_paged_kv_decode_attention_config_validate(config)) return status;
    const SingePagedKvDecodeAttentionConfig& c = *config;
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
    const void* pointers[] = {out, query, key_cache, value_cache, actual_seq_lens, block_table};
    const char* names[] = {"out", "query", "key_cache", "value_cache", "actual_seq_lens", "block_table"};
    for (int i = 0; i < 6; ++i)
        if (pointers[i] == nullptr) return fail(SINGE_HIP_NULL_POINTER, names[i]);
    const int index = width_index(c.head_dim);
    if (index < 0) return fail(SINGE_HIP_UNSUPPORTED_WIDTH, "paged_kv_decode_attention_f32", c.head_dim, 0);
    if (!fits_i32(static_cast<uint64_t>(c.block_table_batch_stride) * c.block_size))
        return fail(SINGE_HIP_LENGTH_EXCEEDS_I32, "block_table_batch_stride * block_size");
    const size_t needed = singe_hip_paged_kv_decode_attention_f32_workspace_bytes(config);
    if (workspace == nullptr) return fail(SINGE_HIP_NULL_POINTER, "workspace");
    if (needed == 0) return fail(SINGE_HIP_SIZE_OVERFLOW, "workspace");
    if (workspace_bytes < needed) return fail(SINGE_HIP_LENGTH_TOO_SHORT, "workspace", needed, workspace_bytes);

    const size_t splits = decode_splits(c);
    const size_t rows = c.batch * c.heads;
    float* partial_lse = static_cast<float*>(workspace);
    float* partial_out = partial_lse + rows * 64;  // the LSEs first, so the rows that follow stay 16-byte aligned
    PagedRowsF32Args args = {};
    args.out = partial_out;
    args.lse = partial_lse;
    args.query = query;
    args.key_cache = key_cache;
    args.value_cache = value_cache;
    args.seq_lens_kv = actual_seq_lens;
    args.block_table = block_table;
    args.batch = static_cast<uint32_t>(c.batch);
    args.heads = static_cast<uint32_t>(c.heads);
    args.kv_heads = static_cast<uint32_t>(c.kv_heads);
    args.block_size = static_cast<uint32_t>(c.block_size);
    args.block_table_batch_stride = static_cast<uint32_t>(c.block_table_batch_stride);
    args.physical_blocks = static_cast<uint32_t>(c.physical_blocks);
    args.splits = static_cast<uint32_t>(splits);
    args.aligned = aligned16(query) && aligned16(key_cache) && aligned16(value_cache) ? 1u : 0u;
    args.scale = c.scale;
    const uint64_t groups = static_cast<uint64_t>(c.batch) * c.kv_heads * splits;
    if (groups > 0x7fffffffull) return fail(SINGE_HIP_UNSUPPORTED_CONFIGURATION, "too many workgroups");
    if (int32_t status = launch(static_cast<KernelId>(kPagedKvDecodeSplitKF32 + index), static_cast<unsigned>(groups), 1, 1, 256,
                                stream, args))
        return status;
    SingeSplitKReduceConfig reduce;
    reduce.batch = c.batch;
    reduce.heads = c.heads;
    reduce.splits = splits;
    reduce.head_dim = c.head_dim;
    reduce.attn_batch_stride = c.heads * splits * c.head_dim;
    reduce.attn_head_stride = splits * c.head_dim;
    reduce.attn_split_stride = c.head_dim;
    reduce.lse_batch_stride = c.heads * splits;
    reduce.lse_head_stride = splits;
    reduce.output_batch_stride = c.heads * c.head_dim;
    reduce.output_head_stride = c.head_dim;
    return singe_hip_splitk_reduce_f32(stream, out, out_len, partial_out, rows * splits * c.head_dim, partial_lse, rows * splits,
                                       &reduce);
}

int32_t singe_hip_paged_kv_prefill_attention_f32(
    void* stream, float* out, size_t out_len, float* lse, size_t lse_len, const float* query, size_t query_len,
    const float* key_cache, size_t key_cache_len, const float* value_cache, size_t value_cache_len,
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
    const int index = width_index(c.head_dim);
    if (index < 0) return fail(SINGE_HIP_UNSUPPORTED_WIDTH, "paged_kv_prefill_attention_f32", c.head_dim, 0);
    const void* pointers[] = {out, lse, query, key_cache, value_cache, actual_seq_lens_q, actual_seq_lens_kv, actual_seq_offsets, block_table};
    const char* names[] = {"out", "lse", "query", "key_cache", "value_cache", "actual_seq_lens_q", "actual_seq_lens_kv",
                           "actual_seq_offsets", "block_table"};
    for (int i = 0; i < 9; ++i)
        if (pointers[i] == nullptr) return fail(SINGE_HIP_NULL_POINTER, names[i]);
    PagedRowsF32Args args = {};
    args.out = out;
    args.lse = lse;
    args.query = query;
    args.key_cache = key_cache;
    args.value_cache = value_cache;
    args.seq_lens_q = actual_seq_lens_q;
    args.seq_lens_kv = actual_seq_lens_kv;
    args.seq_offsets = actual_seq_offsets;
    args.block_table = block_table;
    args.batch = static_cast<uint32_t>(c.batch);
    args.heads = static_cast<uint32_t>(c.heads);
    args.kv_heads = static_cast<uint32_t>(c.kv_heads);
    args.block_size = static_cast<uint32_t>(c.block_size);
    args.block_table_batch_stride = static_cast<uint32_t>(c.block_table_batch_stride);
    args.physical_blocks = static_cast<uint32_t>(c.physical_blocks);
    args.splits = 1;
    args.causal = c.causal ? 1u : 0u;
    args.aligned = aligned16(query) && aligned16(key_cache) && aligned16(value_cache) ? 1u : 0u;
    args.scale = c.scale;
    const uint64_t groups = static_cast<uint64_t>(c.total_query_tokens) * c.kv_heads;
    if (groups > 0x7fffffffull) return fail(SINGE_HIP_UNSUPPORTED_CONFIGURATION, "too many workgroups");
    return launch(static_cast<KernelId>(kPagedKvPrefillF32 + index), static_cast<unsigned>(groups), 1, 1, 256, stream, args);
}

}  // extern "C"
