// Host side of the kernels that take any element type and head dimension: the dense
// scaled-dot-product attention of the singe crate (shape rules of spec::attention_problem,
// singe/src/backend/spec/neural/attention.rs:209-290), the general paged attention
// (singe/src/backend/cuda/kernel_plan/source/paged_general.rs:73-247) and splitk_reduce_f32
// (singe-kernel/src/cuda/attention/fmha.rs:1038-1067).
#include <cmath>

#include "kernel_args.h"
#include "module.h"
#include "singe_hip_attention.h"
#include "validate.h"

using namespace singe_hip;

namespace {

// Kernel of a family for (element, widest dimension): families are laid out element-major with
// the 64 / 128 / 256 variants consecutive.
int32_t pick(KernelId base, int32_t data_type, uint64_t widest, const char* op, KernelId* kernel) {
    if (data_type != SINGE_HIP_F32 && data_type != SINGE_HIP_BF16 && data_type != SINGE_HIP_F16 && data_type != SINGE_HIP_F64)
        return fail(SINGE_HIP_INVALID_ARGUMENT, "data type");
    if (widest > 256) return fail(SINGE_HIP_UNSUPPORTED_WIDTH, op, widest, 0);
    const int width = widest <= 64 ? 0 : widest <= 128 ? 1 : 2;
    if (data_type == SINGE_HIP_F64)  // the f64 kernels sit after the others: dense, then paged
        *kernel = static_cast<KernelId>((base == kDenseGeneral ? kDenseGeneralF64 : kPagedGeneralF64) + width);
    else
        *kernel = static_cast<KernelId>(base + 3 * data_type + width);
    return 0;
}

bool span_reach(size_t count, size_t stride, size_t* total) {  // *total += (count - 1) * stride
    size_t span = 0;
    return count > 0 && checked_mul(count - 1, stride, &span) && checked_add(*total, span, total);
}

}  // namespace

namespace singe_hip {

// Shared with the bf16 entry point, which hands head dimensions other than 128 to this kernel.
int32_t paged_attention_general(int32_t data_type, void* stream, const void* query_rows, const void* key_cache,
                                const void* value_cache, const void* query_offsets, const void* page_offsets,
                                const void* pages, const void* last_page_lengths, void* output, float* lse, uint32_t* status,
                                const SingePagedAttentionProblem& p, float scale) {
    KernelId kernel;
    if (int32_t s = pick(kPagedGeneral, data_type, static_cast<uint64_t>(p.head_dim), "paged_attention", &kernel)) return s;
    GeneralPagedArgs args;
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
    args.head_dim = static_cast<uint32_t>(p.head_dim);
    args.page_size = static_cast<uint32_t>(p.page_size);
    args.sequences = static_cast<uint32_t>(p.sequences);
    args.cache_pages = static_cast<uint32_t>(p.cache_pages);
    args.page_table = static_cast<uint32_t>(p.page_table);
    const uint64_t row_blocks = (static_cast<uint64_t>(p.tokens) * p.heads + 3) / 4;
    args.row_blocks = static_cast<uint32_t>(row_blocks);
    args.causal = p.causal ? 1u : 0u;
    args.has_softcap = p.has_softcap ? 1u : 0u;
    args.form = p.index_type == SINGE_HIP_INDEX_I64 ? 1u : 0u;
    args.scale = scale;
    args.scale_wide = p.has_scale ? static_cast<double>(p.scale) : 1.0 / std::sqrt(static_cast<double>(p.head_dim));
    args.softcap = p.has_softcap ? p.softcap : 0.0f;
    // Four rows to a workgroup, at least one workgroup to a sequence: a bound on the list the kernel walks.
    const uint64_t blocks = static_cast<uint64_t>(p.tokens) * p.heads / 4 + static_cast<uint64_t>(p.sequences);
    if (blocks > 0x7fffffffull || row_blocks > 0xffffffffull) return fail(SINGE_HIP_UNSUPPORTED_CONFIGURATION, "too many workgroups");
    return launch(kernel, static_cast<unsigned>(blocks), 1, 1, 256, stream, args);
}

// The block-table ops of the singe-kernel surface at head dimensions the matrix-core kernels are not built for
// (the reference's own kernels take 4 to 64 there: singe-kernel/src/cuda/cutile/attention/paged.rs:799-810), on the
// same one-wave-per-row kernel.  Prefill: `query_offsets`, `query_lengths`, `key_lengths` [sequences] i32; decode:
// query_lengths null, one query per sequence at row `sequence`.
int32_t paged_table_general(int32_t data_type, void* stream, const char* op, const void* query_rows, const void* key_cache,
                            const void* value_cache, const int32_t* query_offsets, const int32_t* query_lengths,
                            const int32_t* key_lengths, const uint32_t* block_table, void* output, float* lse, uint64_t tokens,
                            uint64_t sequences, uint64_t heads, uint64_t kv_heads, uint64_t head_dim, uint64_t block_size,
                            uint64_t physical_blocks, uint64_t table_stride, bool causal, float scale) {
    KernelId kernel;
    if (int32_t s = pick(kPagedGeneral, data_type, head_dim, op, &kernel)) return s;
    const bool decode = query_lengths == nullptr;
    GeneralPagedArgs args;
    args.query_rows = query_rows;
    args.key_cache = key_cache;
    args.value_cache = value_cache;
    args.query_offsets = query_offsets;
    args.page_offsets = nullptr;
    args.pages = block_table;
    args.last_page_lengths = key_lengths;
    args.query_lengths = query_lengths;
    args.output = output;
    args.lse = lse;
    args.status = nullptr;
    args.window = -1;
    args.tokens = static_cast<uint32_t>(tokens);
    args.heads = static_cast<uint32_t>(heads);
    args.kv_heads = static_cast<uint32_t>(kv_heads);
    args.head_dim = static_cast<uint32_t>(head_dim);
    args.page_size = static_cast<uint32_t>(block_size);
    args.sequences = static_cast<uint32_t>(sequences);
    args.cache_pages = static_cast<uint32_t>(physical_blocks);
    args.page_table = static_cast<uint32_t>(table_stride);
    // A sequence holds at most every token (prefill) or one (decode).
    const uint64_t row_blocks = ((decode ? 1 : tokens) * heads + 3) / 4;
    args.row_blocks = static_cast<uint32_t>(row_blocks);
    args.causal = causal ? 1u : 0u;
    args.has_softcap = 0;
    args.form = decode ? 3u : 2u;
    args.scale = scale;
    args.scale_wide = scale;
    args.softcap = 0.0f;
    // Decoding: ceil(heads / 4) workgroups to a sequence.  Prefill: four rows to a workgroup, at least one workgroup
    // to a sequence, a bound on the list the kernel walks.
    const uint64_t blocks = decode ? row_blocks * sequences : tokens * heads / 4 + sequences;
    if (blocks > 0x7fffffffull || row_blocks > 0xffffffffull) return fail(SINGE_HIP_UNSUPPORTED_CONFIGURATION, "too many workgroups");
    return launch(kernel, static_cast<unsigned>(blocks), 1, 1, 256, stream, args);
}

// Dense attention through element strides on the one-wave-per-row kernel: the scaled-dot-product op below, and
// fmha_prefill[_lse] of the singe-kernel surface at head dimensions the matrix-core kernels are not built for.
int32_t dense_general(int32_t data_type, void* stream, const char* op, const DenseGeneralOperands& o) {
    KernelId kernel;
    const uint64_t widest = o.head_dim > o.value_dim ? o.head_dim : o.value_dim;
    if (int32_t s = pick(kDenseGeneral, data_type, widest, op, &kernel)) return s;
    GeneralAttentionArgs args;
    args.query = o.query;
    args.key = o.key;
    args.value = o.value;
    args.mask = o.mask;
    args.sinks = o.sinks;
    args.key_lengths = o.key_lengths;
    args.out = o.out;
    args.lse = o.lse;
    for (int i = 0; i < 3; ++i) {
        args.query_strides[i] = o.query_strides[i];
        args.key_strides[i] = o.key_strides[i];
        args.value_strides[i] = o.value_strides[i];
        args.out_strides[i] = o.out_strides[i];
    }
    for (int i = 0; i < 4; ++i) args.mask_strides[i] = o.mask_strides[i];
    args.window = o.window;
    args.batch = static_cast<uint32_t>(o.batch);
    args.heads = static_cast<uint32_t>(o.heads);
    args.kv_heads = static_cast<uint32_t>(o.kv_heads);
    args.query_len = static_cast<uint32_t>(o.query_len);
    args.key_len = static_cast<uint32_t>(o.key_len);
    args.head_dim = static_cast<uint32_t>(o.head_dim);
    args.value_dim = static_cast<uint32_t>(o.value_dim);
    args.causal = o.causal ? 1u : 0u;
    args.has_softcap = o.has_softcap ? 1u : 0u;
    args.scale = o.scale;
    args.scale_wide = o.scale_wide;
    args.softcap = o.softcap;
    args.query_start = o.query_start;
    args.key_start = o.key_start;
    args.lookahead = o.lookahead;
    args.output_scale = o.output_scale;
    args.empty_lse = o.empty_lse;
    args.block_table = o.block_table;
    args.block_size = static_cast<uint32_t>(o.block_size);
    args.physical_blocks = static_cast<uint32_t>(o.physical_blocks);
    args.table_stride = static_cast<uint32_t>(o.table_stride);
    args.key_block_stride = o.key_block_stride;
    args.value_block_stride = o.value_block_stride;
    args.ragged = o.ragged ? 1u : 0u;
    args.total_kv_tokens = static_cast<uint32_t>(o.total_kv_tokens);
    args.query_lengths = o.query_lengths;
    args.kv_lengths = o.kv_lengths;
    args.sequence_offsets = o.sequence_offsets;
    const uint64_t rows = (o.ragged ? 1 : o.batch) * o.heads * o.query_len;
    const uint64_t blocks = (rows + 3) / 4;
    if (blocks > 0x7fffffffull) return fail(SINGE_HIP_UNSUPPORTED_CONFIGURATION, "too many workgroups");
    return launch(kernel, static_cast<unsigned>(blocks), 1, 1, 256, stream, args);
}

}  // namespace singe_hip

namespace {

// The config the matrix-core dense kernels read a [batch, heads, len, dim] problem through.
SingeFmhaPrefillConfig matrix_core_config(const SingeAttentionProblem& p, float scale) {
    const size_t dim = static_cast<size_t>(p.head_dim);
    SingeFmhaPrefillConfig c;
    c.batch = p.batch, c.query_len = p.query_len, c.key_len = p.key_len, c.heads = p.heads, c.kv_heads = p.kv_heads, c.head_dim = dim;
    c.query_batch_stride = c.output_batch_stride = static_cast<size_t>(p.heads) * p.query_len * dim;
    c.key_batch_stride = c.value_batch_stride = static_cast<size_t>(p.kv_heads) * p.key_len * dim;
    c.query_sequence_stride = c.key_sequence_stride = c.value_sequence_stride = c.output_sequence_stride = dim;
    c.query_head_stride = c.output_head_stride = static_cast<size_t>(p.query_len) * dim;
    c.key_head_stride = c.value_head_stride = static_cast<size_t>(p.key_len) * dim;
    c.scale = scale, c.causal = p.causal ? 1 : 0;
    return c;
}

bool takes_matrix_cores(const SingeAttentionProblem& p) {
    return (p.data_type == SINGE_HIP_BF16 || p.data_type == SINGE_HIP_F16) && has_matrix_core_build(p.head_dim) &&
           p.value_dim == p.head_dim;
}

int32_t scaled_dot_product_attention(void* stream, const void* query, const void* key, const void* value, const void* mask,
                                     const void* sinks, const int32_t* key_lengths, void* output, void* scratch, size_t scratch_bytes,
                                     const SingeAttentionProblem* problem) {
    if (problem == nullptr) return fail(SINGE_HIP_NULL_POINTER, "problem");
    const SingeAttentionProblem& p = *problem;
    // attention_problem: batch, heads, query length and value dimension may be zero; head dimension and
    // key length may not; the key heads divide the query heads.
    if (p.batch < 0 || p.heads < 0 || p.query_len < 0 || p.value_dim < 0 || p.head_dim <= 0 || p.key_len <= 0 || p.kv_heads <= 0 ||
        p.heads % p.kv_heads != 0)
        return fail(SINGE_HIP_INVALID_ARGUMENT, "attention shape");
    if (p.has_scale && !std::isfinite(p.scale)) return fail(SINGE_HIP_INVALID_ARGUMENT, "scale");
    if (p.has_softcap && !(std::isfinite(p.softcap) && p.softcap != 0.0f)) return fail(SINGE_HIP_INVALID_ARGUMENT, "softcap");
    if (p.has_window && p.window < 0) return fail(SINGE_HIP_INVALID_ARGUMENT, "window");
    const int64_t extents[] = {p.batch, p.heads, p.kv_heads, p.query_len, p.key_len, p.head_dim, p.value_dim};
    for (int64_t extent : extents)
        if (!fits_i32(static_cast<uint64_t>(extent))) return fail(SINGE_HIP_LENGTH_EXCEEDS_I32, "problem");
    for (int64_t stride : p.mask_strides)
        if (stride < 0) return fail(SINGE_HIP_INVALID_ARGUMENT, "mask stride");
    const uint64_t rows = static_cast<uint64_t>(p.batch) * p.heads * p.query_len;
    if (rows == 0 || p.value_dim == 0) return 0;
    if (query == nullptr) return fail(SINGE_HIP_NULL_POINTER, "query");
    if (key == nullptr) return fail(SINGE_HIP_NULL_POINTER, "key");
    if (value == nullptr) return fail(SINGE_HIP_NULL_POINTER, "value");
    if (output == nullptr) return fail(SINGE_HIP_NULL_POINTER, "output");
    const float scale = p.has_scale ? p.scale : 1.0f / std::sqrt(static_cast<float>(p.head_dim));

    // bf16 and f16 at head dimensions 128 and 64 are what the MFMA flash kernels compute, every option included,
    // reading [batch, heads, len, dim] through their strides.
    if (takes_matrix_cores(p)) {
        const size_t dim = static_cast<size_t>(p.head_dim);
        SingeFmhaPrefillConfig c = matrix_core_config(p, scale);
        const size_t q_len = static_cast<size_t>(rows) * dim, kv_len = static_cast<size_t>(p.batch) * p.kv_heads * p.key_len * dim;
        DenseOptions options;
        options.scratch = scratch;
        options.scratch_bytes = scratch_bytes;
        options.sinks = static_cast<const uint16_t*>(sinks);
        options.key_lengths = key_lengths;
        options.mask = static_cast<const uint16_t*>(mask);
        for (int i = 0; i < 4; ++i) options.mask_strides[i] = static_cast<uint64_t>(p.mask_strides[i]);
        options.window = p.has_window ? p.window : -1;
        options.softcap = p.has_softcap ? p.softcap : 0.0f;
        return dense_prefill_with_options(stream, p.data_type == SINGE_HIP_F16, static_cast<uint16_t*>(output), q_len,
                                          static_cast<const uint16_t*>(query), q_len, static_cast<const uint16_t*>(key), kv_len,
                                          static_cast<const uint16_t*>(value), kv_len, &c, options);
    }

    DenseGeneralOperands o;
    o.query = query, o.key = key, o.value = value, o.mask = mask, o.sinks = sinks, o.key_lengths = key_lengths, o.out = output;
    const uint64_t dim = static_cast<uint64_t>(p.head_dim), value_dim = static_cast<uint64_t>(p.value_dim);
    const uint64_t query_len = static_cast<uint64_t>(p.query_len), key_len = static_cast<uint64_t>(p.key_len);
    o.query_strides[0] = p.heads * query_len * dim, o.query_strides[1] = query_len * dim, o.query_strides[2] = dim;
    o.key_strides[0] = p.kv_heads * key_len * dim, o.key_strides[1] = key_len * dim, o.key_strides[2] = dim;
    o.value_strides[0] = p.kv_heads * key_len * value_dim, o.value_strides[1] = key_len * value_dim, o.value_strides[2] = value_dim;
    o.out_strides[0] = p.heads * query_len * value_dim, o.out_strides[1] = query_len * value_dim, o.out_strides[2] = value_dim;
    for (int i = 0; i < 4; ++i) o.mask_strides[i] = static_cast<uint64_t>(p.mask_strides[i]);
    o.window = p.has_window ? p.window : -1;
    o.batch = p.batch, o.heads = p.heads, o.kv_heads = p.kv_heads, o.query_len = query_len, o.key_len = key_len;
    o.head_dim = dim, o.value_dim = value_dim;
    o.causal = p.causal != 0, o.has_softcap = p.has_softcap != 0;
    o.scale = scale, o.softcap = p.has_softcap ? p.softcap : 0.0f;
    o.scale_wide = p.has_scale ? static_cast<double>(p.scale) : 1.0 / std::sqrt(static_cast<double>(p.head_dim));
    return dense_general(p.data_type, stream, "scaled_dot_product_attention", o);
}

}  // namespace

extern "C" int32_t singe_hip_scaled_dot_product_attention(void* stream, const void* query, const void* key, const void* value,
                                                          const void* mask, const void* sinks, const int32_t* key_lengths,
                                                          void* output, const SingeAttentionProblem* problem) {
    return scaled_dot_product_attention(stream, query, key, value, mask, sinks, key_lengths, output, nullptr, 0, problem);
}

extern "C" int32_t singe_hip_scaled_dot_product_attention_scratch(void* stream, const void* query, const void* key, const void* value,
                                                                  const void* mask, const void* sinks, const int32_t* key_lengths,
                                                                  void* output, void* scratch, size_t scratch_bytes,
                                                                  const SingeAttentionProblem* problem) {
    return scaled_dot_product_attention(stream, query, key, value, mask, sinks, key_lengths, output, scratch, scratch_bytes, problem);
}

extern "C" size_t singe_hip_scaled_dot_product_attention_scratch_bytes(const SingeAttentionProblem* problem) {
    if (problem == nullptr || !takes_matrix_cores(*problem) || problem->batch <= 0 || problem->heads <= 0 || problem->query_len <= 0 ||
        problem->key_len <= 0 || problem->kv_heads <= 0)
        return 0;
    const SingeFmhaPrefillConfig c = matrix_core_config(*problem, 1.0f);
    return dense_prefill_scratch_bytes(c, dense_prefill_splits(c));
}

// validate_splitk_reduce_config (singe-kernel/src/cuda/attention/mod.rs:3557-3573) and
// SplitKReduceConfig::validate_lengths (mod.rs:2330-2361).
extern "C" int32_t singe_hip_splitk_reduce_f32(void* stream, float* out, size_t out_len, const float* attn_splitk,
                                               size_t attn_splitk_len, const float* lse_splitk, size_t lse_splitk_len,
                                               const SingeSplitKReduceConfig* config) {
    if (config == nullptr) return fail(SINGE_HIP_NULL_POINTER, "config");
    const SingeSplitKReduceConfig& c = *config;
    if (c.batch == 0 || c.heads == 0 || c.splits == 0 || c.head_dim == 0 || c.attn_batch_stride == 0 || c.attn_head_stride == 0 ||
        c.attn_split_stride == 0 || c.lse_batch_stride == 0 || c.lse_head_stride == 0 || c.output_batch_stride == 0 ||
        c.output_head_stride == 0)
        return fail(SINGE_HIP_INVALID_LENGTH, "config");
    size_t attn_reach = c.head_dim, lse_reach = c.splits, out_reach = c.head_dim;
    if (!span_reach(c.heads, c.attn_head_stride, &attn_reach) || !span_reach(c.splits, c.attn_split_stride, &attn_reach) ||
        !span_reach(c.batch, c.attn_batch_stride, &attn_reach) || !span_reach(c.heads, c.lse_head_stride, &lse_reach) ||
        !span_reach(c.batch, c.lse_batch_stride, &lse_reach) || !span_reach(c.heads, c.output_head_stride, &out_reach) ||
        !span_reach(c.batch, c.output_batch_stride, &out_reach))
        return fail(SINGE_HIP_SIZE_OVERFLOW, "config");
    if (int32_t s = ensure_len_at_least("attn_splitk", attn_splitk_len, attn_reach)) return s;
    if (int32_t s = ensure_len_at_least("lse_splitk", lse_splitk_len, lse_reach)) return s;
    if (int32_t s = ensure_len_at_least("out", out_len, out_reach)) return s;
    const size_t extents[] = {c.batch, c.heads, c.splits, c.head_dim};
    for (size_t extent : extents)
        if (!fits_i32(extent)) return fail(SINGE_HIP_LENGTH_EXCEEDS_I32, "config");
    if (out == nullptr) return fail(SINGE_HIP_NULL_POINTER, "out");
    if (attn_splitk == nullptr) return fail(SINGE_HIP_NULL_POINTER, "attn_splitk");
    if (lse_splitk == nullptr) return fail(SINGE_HIP_NULL_POINTER, "lse_splitk");
    SplitKReduceArgs args;
    args.out = out;
    args.attn = attn_splitk;
    args.lse = lse_splitk;
    args.attn_batch_stride = c.attn_batch_stride;
    args.attn_head_stride = c.attn_head_stride;
    args.attn_split_stride = c.attn_split_stride;
    args.lse_batch_stride = c.lse_batch_stride;
    args.lse_head_stride = c.lse_head_stride;
    args.output_batch_stride = c.output_batch_stride;
    args.output_head_stride = c.output_head_stride;
    args.batch = static_cast<uint32_t>(c.batch);
    args.heads = static_cast<uint32_t>(c.heads);
    args.splits = static_cast<uint32_t>(c.splits);
    args.head_dim = static_cast<uint32_t>(c.head_dim);
    const uint64_t blocks = (static_cast<uint64_t>(c.batch) * c.heads + 3) / 4;
    if (blocks > 0x7fffffffull) return fail(SINGE_HIP_UNSUPPORTED_CONFIGURATION, "too many workgroups");
    return launch(kSplitKReduce, static_cast<unsigned>(blocks), 1, 1, 256, stream, args);
}
