// The rest of the singe-kernel dense attention family (singe-kernel/src/cuda/attention/fmha.rs:193-1036,
// paged.rs:36-116, 427-576): windowed attention with a score cap on 16-bit tensors, attention with sink logits,
// single-query decode with a log-sum-exp, windowed decode, ragged packed prefill and sliding-window attention over
// dense, packed and block-table keys.  Each entry point checks its config and lengths in the reference's order
// (mod.rs: the `validate_lengths` of the config it mirrors) and then runs on a kernel the library already has: the
// matrix-core prefill kernels where a call is one of their shapes, otherwise the one-wave-per-row kernel that reads
// every operand through element strides (general_attention.hip).
#include <cmath>

#include "module.h"
#include "singe_hip_attention.h"
#include "validate.h"

using namespace singe_hip;

namespace {

// projected_layout_reach (mod.rs:3647-3668) and batched_reach (mod.rs:3670-3677).
bool layout_reach(size_t sequence_len, size_t heads, size_t head_dim, size_t sequence_stride, size_t head_stride, size_t* out) {
    size_t sequence_span, head_span;
    if (sequence_len == 0 || heads == 0) return false;
    return checked_mul(sequence_len - 1, sequence_stride, &sequence_span) && checked_mul(heads - 1, head_stride, &head_span) &&
           checked_add(sequence_span, head_span, out) && checked_add(*out, head_dim, out);
}

int32_t ensure_reach(const char* name, size_t actual, size_t batch, size_t sequence_len, size_t heads, size_t head_dim,
                     size_t batch_stride, size_t sequence_stride, size_t head_stride) {
    size_t item = 0, span = 0, need = 0;
    if (!layout_reach(sequence_len, heads, head_dim, sequence_stride, head_stride, &item) || batch == 0 ||
        !checked_mul(batch - 1, batch_stride, &span) || !checked_add(span, item, &need))
        return fail(SINGE_HIP_SIZE_OVERFLOW, name);
    return ensure_len_at_least(name, actual, need);
}

int32_t data_type_of(bool f16, bool wide) { return wide ? SINGE_HIP_F32 : f16 ? SINGE_HIP_F16 : SINGE_HIP_BF16; }

int32_t null_check(const void* const* pointers, const char* const* names, int count) {
    for (int i = 0; i < count; ++i)
        if (pointers[i] == nullptr) return fail(SINGE_HIP_NULL_POINTER, names[i]);
    return 0;
}

// validate_fmha_prefill_config (mod.rs:3369-3398).
int32_t validate_prefill_config(const SingeFmhaPrefillConfig& c) {
    const size_t extents[] = {c.batch, c.query_len, c.key_len, c.heads, c.kv_heads, c.head_dim,
                              c.query_batch_stride, c.key_batch_stride, c.value_batch_stride, c.output_batch_stride,
                              c.query_sequence_stride, c.key_sequence_stride, c.value_sequence_stride,
                              c.output_sequence_stride, c.query_head_stride, c.key_head_stride,
                              c.value_head_stride, c.output_head_stride};
    for (size_t extent : extents)
        if (extent == 0) return fail(SINGE_HIP_INVALID_LENGTH, "config");
    if (!std::isfinite(c.scale) || c.heads % c.kv_heads != 0) return fail(SINGE_HIP_INVALID_LENGTH, "config");
    return 0;
}

// FmhaPrefillConfig::validate_output_lengths (mod.rs:1704-1756): query, key, value, out in that order.
int32_t validate_prefill_lengths(const SingeFmhaPrefillConfig& c, size_t out_len, size_t query_len, size_t key_len, size_t value_len) {
    if (int32_t s = validate_prefill_config(c)) return s;
    if (int32_t s = ensure_reach("query", query_len, c.batch, c.query_len, c.heads, c.head_dim, c.query_batch_stride,
                                 c.query_sequence_stride, c.query_head_stride)) return s;
    if (int32_t s = ensure_reach("key", key_len, c.batch, c.key_len, c.kv_heads, c.head_dim, c.key_batch_stride,
                                 c.key_sequence_stride, c.key_head_stride)) return s;
    if (int32_t s = ensure_reach("value", value_len, c.batch, c.key_len, c.kv_heads, c.head_dim, c.value_batch_stride,
                                 c.value_sequence_stride, c.value_head_stride)) return s;
    return ensure_reach("out", out_len, c.batch, c.query_len, c.heads, c.head_dim, c.output_batch_stride,
                        c.output_sequence_stride, c.output_head_stride);
}

// The strides of a FmhaPrefillConfig as the row kernel takes them: over (batch, head, position).
void prefill_operands(DenseGeneralOperands& o, const SingeFmhaPrefillConfig& c) {
    o.batch = c.batch, o.heads = c.heads, o.kv_heads = c.kv_heads, o.query_len = c.query_len, o.key_len = c.key_len;
    o.head_dim = o.value_dim = c.head_dim;
    o.query_strides[0] = c.query_batch_stride, o.query_strides[1] = c.query_head_stride, o.query_strides[2] = c.query_sequence_stride;
    o.key_strides[0] = c.key_batch_stride, o.key_strides[1] = c.key_head_stride, o.key_strides[2] = c.key_sequence_stride;
    o.value_strides[0] = c.value_batch_stride, o.value_strides[1] = c.value_head_stride, o.value_strides[2] = c.value_sequence_stride;
    o.out_strides[0] = c.output_batch_stride, o.out_strides[1] = c.output_head_stride, o.out_strides[2] = c.output_sequence_stride;
    o.scale = c.scale, o.scale_wide = c.scale, o.causal = c.causal != 0;
}

// A single-query FmhaDecodeConfig read as a prefill of one query row per batch item.
SingeFmhaPrefillConfig decode_as_prefill(const SingeFmhaDecodeConfig& c) {
    SingeFmhaPrefillConfig p;
    p.batch = c.batch, p.query_len = 1, p.key_len = c.key_len, p.heads = c.heads, p.kv_heads = c.kv_heads, p.head_dim = c.head_dim;
    p.query_batch_stride = c.query_batch_stride, p.key_batch_stride = c.key_batch_stride, p.value_batch_stride = c.value_batch_stride;
    p.output_batch_stride = c.output_batch_stride;
    p.query_sequence_stride = 1, p.output_sequence_stride = 1;  // one query: never stepped over
    p.key_sequence_stride = c.key_sequence_stride, p.value_sequence_stride = c.value_sequence_stride;
    p.query_head_stride = c.query_head_stride, p.key_head_stride = c.key_head_stride, p.value_head_stride = c.value_head_stride;
    p.output_head_stride = c.output_head_stride;
    p.scale = c.scale, p.causal = 0;
    return p;
}

// validate_fmha_decode_config (mod.rs:3530-3555) and FmhaDecodeConfig::validate_lengths (mod.rs:2262-2308).
int32_t validate_decode_lengths(const SingeFmhaDecodeConfig& c, size_t out_len, size_t lse_len, size_t query_len, size_t key_len,
                                size_t value_len) {
    const size_t extents[] = {c.batch, c.key_len, c.heads, c.kv_heads, c.head_dim, c.query_batch_stride, c.key_batch_stride,
                              c.value_batch_stride, c.output_batch_stride, c.query_head_stride, c.key_sequence_stride,
                              c.value_sequence_stride, c.output_head_stride, c.key_head_stride, c.value_head_stride};
    for (size_t extent : extents)
        if (extent == 0) return fail(SINGE_HIP_INVALID_LENGTH, "config");
    if (!std::isfinite(c.scale) || c.heads % c.kv_heads != 0) return fail(SINGE_HIP_INVALID_LENGTH, "config");
    if (int32_t s = ensure_reach("query", query_len, c.batch, 1, c.heads, c.head_dim, c.query_batch_stride, 1, c.query_head_stride)) return s;
    if (int32_t s = ensure_reach("key", key_len, c.batch, c.key_len, c.kv_heads, c.head_dim, c.key_batch_stride,
                                 c.key_sequence_stride, c.key_head_stride)) return s;
    if (int32_t s = ensure_reach("value", value_len, c.batch, c.key_len, c.kv_heads, c.head_dim, c.value_batch_stride,
                                 c.value_sequence_stride, c.value_head_stride)) return s;
    if (int32_t s = ensure_reach("out", out_len, c.batch, 1, c.heads, c.head_dim, c.output_batch_stride, 1, c.output_head_stride)) return s;
    size_t rows = 0;
    if (!checked_mul(c.batch, c.heads, &rows)) return fail(SINGE_HIP_SIZE_OVERFLOW, "lse");
    return ensure_len_at_least("lse", lse_len, rows);
}

int32_t extents_fit(const size_t* extents, int count) {
    for (int i = 0; i < count; ++i)
        if (!fits_i32(extents[i])) return fail(SINGE_HIP_LENGTH_EXCEEDS_I32, "config");
    return 0;
}

// Option<f32> soft caps must be finite and positive (mod.rs:3418-3443).
int32_t validate_cap(uint8_t has_soft_cap, float soft_cap) {
    if (has_soft_cap && !(std::isfinite(soft_cap) && soft_cap > 0.0f)) return fail(SINGE_HIP_INVALID_LENGTH, "soft_cap");
    return 0;
}

// ---- softcapped_window_attention_{f16,bf16} (fmha.rs:295-393; CPU form cpu/attention.rs:1835-1925) ----
int32_t softcapped_window_attention(void* stream, bool f16, uint16_t* out, size_t out_len, const uint16_t* query, size_t query_len,
                                    const uint16_t* key, size_t key_len, const uint16_t* value, size_t value_len,
                                    const SingeSoftcappedWindowAttentionConfig* config, const char* op) {
    if (config == nullptr) return fail(SINGE_HIP_NULL_POINTER, "config");
    const SingeFmhaPrefillConfig& c = config->attention;
    if (int32_t s = validate_prefill_lengths(c, out_len, query_len, key_len, value_len)) return s;
    if (int32_t s = validate_cap(config->has_soft_cap, config->soft_cap)) return s;
    if (!fits_i32(config->window_size)) return fail(SINGE_HIP_LENGTH_EXCEEDS_I32, "window_size");
    const void* pointers[] = {out, query, key, value};
    const char* names[] = {"out", "query", "key", "value"};
    if (int32_t s = null_check(pointers, names, 4)) return s;
    const size_t extents[] = {c.batch, c.query_len, c.key_len, c.heads, c.kv_heads, c.head_dim};
    if (int32_t s = extents_fit(extents, 6)) return s;
    if (c.head_dim > 256) return fail(SINGE_HIP_UNSUPPORTED_WIDTH, op, c.head_dim, 0);
    const size_t window = config->window_size;
    // A window hides keys more than `window` positions from the query on either side.  Under the causal mask only the
    // side before the query is left, which is the matrix-core kernels' window of window + 1 keys; without a window
    // they take the call as it is.  A two-sided window without the causal mask runs on the row kernel.
    if (dense_prefill_takes(c, out, query, key, value) && (window == 0 || c.causal)) {
        DenseOptions options;
        options.window = window == 0 ? -1 : static_cast<long long>(window) + 1;
        options.softcap = config->has_soft_cap ? config->soft_cap : 0.0f;
        return dense_prefill_with_options(stream, f16, out, out_len, query, query_len, key, key_len, value, value_len, &c, options);
    }
    DenseGeneralOperands o;
    prefill_operands(o, c);
    o.query = query, o.key = key, o.value = value, o.out = out;
    if (window > 0) o.window = static_cast<long long>(window) + 1, o.lookahead = static_cast<long long>(window);
    o.has_softcap = config->has_soft_cap != 0, o.softcap = config->soft_cap;
    return dense_general(data_type_of(f16, false), stream, op, o);
}

// ---- attention_sink_prefill_{f32,f16,bf16} (fmha.rs:193-243, 796-898; CPU form cpu/attention.rs:2073-2155) ----
int32_t attention_sink_prefill(void* stream, int32_t data_type, void* out, size_t out_len, const void* query, size_t query_len,
                               const void* key, size_t key_len, const void* value, size_t value_len, const void* sinks,
                               size_t sinks_len, const SingeAttentionSinkPrefillConfig* config, const char* op) {
    if (config == nullptr) return fail(SINGE_HIP_NULL_POINTER, "config");
    const SingeFmhaPrefillConfig& c = config->attention;
    if (int32_t s = validate_prefill_lengths(c, out_len, query_len, key_len, value_len)) return s;
    if (int32_t s = ensure_len_at_least("sinks", sinks_len, c.heads)) return s;
    if (!fits_i32(config->start_q)) return fail(SINGE_HIP_LENGTH_EXCEEDS_I32, "start_q");
    if (!fits_i32(config->window)) return fail(SINGE_HIP_LENGTH_EXCEEDS_I32, "window");
    const void* pointers[] = {out, query, key, value, sinks};
    const char* names[] = {"out", "query", "key", "value", "sinks"};
    if (int32_t s = null_check(pointers, names, 5)) return s;
    const size_t extents[] = {c.batch, c.query_len, c.key_len, c.heads, c.kv_heads, c.head_dim};
    if (int32_t s = extents_fit(extents, 6)) return s;
    if (c.head_dim > 256) return fail(SINGE_HIP_UNSUPPORTED_WIDTH, op, c.head_dim, 0);
    // Query q sits at position start_q + q; the causal mask hides later keys, a window of w keys those before
    // position - (w - 1); every row's softmax also holds its head's sink, which weighs no value.
    if (data_type != SINGE_HIP_F32 && config->start_q == 0 && dense_prefill_takes(c, out, query, key, value)) {
        DenseOptions options;
        options.sinks = static_cast<const uint16_t*>(sinks);
        options.window = config->window == 0 ? -1 : static_cast<long long>(config->window);
        return dense_prefill_with_options(stream, data_type == SINGE_HIP_F16, static_cast<uint16_t*>(out), out_len,
                                          static_cast<const uint16_t*>(query), query_len, static_cast<const uint16_t*>(key), key_len,
                                          static_cast<const uint16_t*>(value), value_len, &c, options);
    }
    DenseGeneralOperands o;
    prefill_operands(o, c);
    o.query = query, o.key = key, o.value = value, o.out = out, o.sinks = sinks;
    o.query_start = static_cast<long long>(config->start_q);
    if (config->window > 0) o.window = static_cast<long long>(config->window);
    return dense_general(data_type, stream, op, o);
}

// ---- fmha_decode_lse_* (fmha.rs:395-438, 900-1036) and softcapped_window_decode_lse_* (fmha.rs:440-582; CPU form
// cpu/attention.rs:1927-1998): one query per batch item at position key_len - 1, natural-log lse [batch, heads] ----
int32_t decode_lse(void* stream, int32_t data_type, void* out, size_t out_len, float* lse, size_t lse_len, const void* query,
                   size_t query_len, const void* key, size_t key_len, const void* value, size_t value_len,
                   const SingeFmhaDecodeConfig* decode, size_t window_size, uint8_t has_soft_cap, float soft_cap, bool windowed_op,
                   const char* op) {
    if (decode == nullptr) return fail(SINGE_HIP_NULL_POINTER, "config");
    const SingeFmhaDecodeConfig& c = *decode;
    if (windowed_op) {
        // validate_softcapped_window_decode_config comes first (mod.rs:2609-2612): the decode config, the cap, the window.
        const size_t extents[] = {c.batch, c.key_len, c.heads, c.kv_heads, c.head_dim, c.query_batch_stride, c.key_batch_stride,
                                  c.value_batch_stride, c.output_batch_stride, c.query_head_stride, c.key_sequence_stride,
                                  c.value_sequence_stride, c.output_head_stride, c.key_head_stride, c.value_head_stride};
        for (size_t extent : extents)
            if (extent == 0) return fail(SINGE_HIP_INVALID_LENGTH, "config");
        if (!std::isfinite(c.scale) || c.heads % c.kv_heads != 0) return fail(SINGE_HIP_INVALID_LENGTH, "config");
        if (int32_t s = validate_cap(has_soft_cap, soft_cap)) return s;
        if (!fits_i32(window_size)) return fail(SINGE_HIP_LENGTH_EXCEEDS_I32, "window_size");
    }
    if (int32_t s = validate_decode_lengths(c, out_len, lse_len, query_len, key_len, value_len)) return s;
    const void* pointers[] = {out, lse, query, key, value};
    const char* names[] = {"out", "lse", "query", "key", "value"};
    if (int32_t s = null_check(pointers, names, 5)) return s;
    const size_t extents[] = {c.batch, c.key_len, c.heads, c.kv_heads, c.head_dim};
    if (int32_t s = extents_fit(extents, 5)) return s;
    if (c.head_dim > 256) return fail(SINGE_HIP_UNSUPPORTED_WIDTH, op, c.head_dim, 0);
    const SingeFmhaPrefillConfig as_prefill = decode_as_prefill(c);
    DenseGeneralOperands o;
    prefill_operands(o, as_prefill);
    o.query = query, o.key = key, o.value = value, o.out = out, o.lse = lse;
    // The query's position is the last key's; a window keeps the keys with key + window_size >= position.
    o.query_start = static_cast<long long>(c.key_len) - 1;
    if (window_size > 0) o.window = static_cast<long long>(window_size) + 1;
    o.has_softcap = has_soft_cap != 0, o.softcap = soft_cap;
    return dense_general(data_type, stream, op, o);
}

// ---- ragged_kv_prefill_attention_* (paged.rs:427-576; CPU form cpu/attention.rs:1343-1420) ----
int32_t ragged_kv_prefill(void* stream, int32_t data_type, void* out, size_t out_len, float* lse, size_t lse_len, const void* query,
                          size_t query_len, const void* key, size_t key_len, const void* value, size_t value_len,
                          const int32_t* lens_q, size_t lens_q_len, const int32_t* lens_kv, size_t lens_kv_len,
                          const int32_t* offsets, size_t offsets_len, const SingeRaggedKvPrefillAttentionConfig* config, const char* op) {
    if (config == nullptr) return fail(SINGE_HIP_NULL_POINTER, "config");
    const SingeRaggedKvPrefillAttentionConfig& c = *config;
    // validate_ragged_kv_prefill_attention_config (mod.rs:3013-3035).
    if (c.batch == 0 || c.total_query_tokens == 0 || c.total_kv_tokens == 0 || c.heads == 0 || c.kv_heads == 0 || c.head_dim == 0 ||
        c.heads % c.kv_heads != 0 || !std::isfinite(c.scale))
        return fail(SINGE_HIP_INVALID_LENGTH, "config");
    const size_t extents[] = {c.batch, c.total_query_tokens, c.total_kv_tokens, c.heads, c.kv_heads, c.head_dim};
    if (int32_t s = extents_fit(extents, 6)) return s;
    // RaggedKvPrefillAttentionConfig::validate_lengths (mod.rs:858-882).
    size_t output_len = 0, kv_len = 0, rows = 0;
    if (!checked_mul(c.total_query_tokens, c.heads, &rows) || !checked_mul(rows, c.head_dim, &output_len) ||
        !checked_mul(c.total_kv_tokens, c.kv_heads, &kv_len) || !checked_mul(kv_len, c.head_dim, &kv_len))
        return fail(SINGE_HIP_SIZE_OVERFLOW, "config");
    if (int32_t s = ensure_len_at_least("out", out_len, output_len)) return s;
    if (int32_t s = ensure_len_at_least("lse", lse_len, rows)) return s;
    if (int32_t s = ensure_len_at_least("query", query_len, output_len)) return s;
    if (int32_t s = ensure_len_at_least("key", key_len, kv_len)) return s;
    if (int32_t s = ensure_len_at_least("value", value_len, kv_len)) return s;
    if (int32_t s = ensure_len_at_least("actual_seq_lens_q", lens_q_len, c.batch)) return s;
    if (int32_t s = ensure_len_at_least("actual_seq_lens_kv", lens_kv_len, c.batch)) return s;
    if (int32_t s = ensure_len_at_least("actual_seq_offsets", offsets_len, c.batch)) return s;
    const void* pointers[] = {out, lse, query, key, value, lens_q, lens_kv, offsets};
    const char* names[] = {"out", "lse", "query", "key", "value", "actual_seq_lens_q", "actual_seq_lens_kv", "actual_seq_offsets"};
    if (int32_t s = null_check(pointers, names, 8)) return s;
    if (c.head_dim > 256) return fail(SINGE_HIP_UNSUPPORTED_WIDTH, op, c.head_dim, 0);
    DenseGeneralOperands o;
    o.query = query, o.key = key, o.value = value, o.out = out, o.lse = lse;
    o.batch = c.batch, o.heads = c.heads, o.kv_heads = c.kv_heads, o.query_len = c.total_query_tokens, o.key_len = 0;
    o.head_dim = o.value_dim = c.head_dim;
    o.query_strides[1] = o.out_strides[1] = o.key_strides[1] = o.value_strides[1] = c.head_dim;
    o.query_strides[2] = o.out_strides[2] = c.heads * c.head_dim;
    o.key_strides[2] = o.value_strides[2] = c.kv_heads * c.head_dim;
    o.scale = c.scale, o.scale_wide = c.scale, o.causal = c.causal != 0;
    o.ragged = true, o.total_kv_tokens = c.total_kv_tokens;
    o.query_lengths = lens_q, o.kv_lengths = lens_kv, o.sequence_offsets = offsets;
    o.empty_lse = -1.0e20f;  // what a token that sees no key reports (cpu/attention.rs:1389-1392)
    return dense_general(data_type, stream, op, o);
}

// validate_sliding_window_attention_config (mod.rs:3037-3075).
int32_t validate_sliding_config(const SingeSlidingWindowAttentionConfig& c) {
    const size_t extents[] = {c.batch, c.query_len, c.key_len, c.heads, c.kv_heads, c.head_dim, c.window, c.query_batch_stride,
                              c.key_batch_stride, c.value_batch_stride, c.output_batch_stride, c.query_sequence_stride,
                              c.key_sequence_stride, c.value_sequence_stride, c.output_sequence_stride, c.query_head_stride,
                              c.key_head_stride, c.value_head_stride, c.output_head_stride};
    for (size_t extent : extents)
        if (extent == 0) return fail(SINGE_HIP_INVALID_LENGTH, "config");
    if (!std::isfinite(c.scale) || !std::isfinite(c.output_scale) || c.heads % c.kv_heads != 0) return fail(SINGE_HIP_INVALID_LENGTH, "config");
    size_t reach;
    if (!checked_add(c.query_start, c.query_len, &reach) || !checked_add(c.key_start, c.key_len, &reach))
        return fail(SINGE_HIP_SIZE_OVERFLOW, "config");
    return 0;
}

void sliding_operands(DenseGeneralOperands& o, const SingeSlidingWindowAttentionConfig& c) {
    o.batch = c.batch, o.heads = c.heads, o.kv_heads = c.kv_heads, o.query_len = c.query_len, o.key_len = c.key_len;
    o.head_dim = o.value_dim = c.head_dim;
    o.query_strides[0] = c.query_batch_stride, o.query_strides[1] = c.query_head_stride, o.query_strides[2] = c.query_sequence_stride;
    o.key_strides[0] = c.key_batch_stride, o.key_strides[1] = c.key_head_stride, o.key_strides[2] = c.key_sequence_stride;
    o.value_strides[0] = c.value_batch_stride, o.value_strides[1] = c.value_head_stride, o.value_strides[2] = c.value_sequence_stride;
    o.out_strides[0] = c.output_batch_stride, o.out_strides[1] = c.output_head_stride, o.out_strides[2] = c.output_sequence_stride;
    o.scale = c.scale, o.scale_wide = c.scale, o.output_scale = c.output_scale;
    // A key is kept when key_abs <= query_abs and key_abs + window > query_abs (cpu/attention.rs:1116-1119).
    o.causal = true;
    o.query_start = static_cast<long long>(c.query_start), o.key_start = static_cast<long long>(c.key_start);
    o.window = c.window > 0x7fffffffffffffffull ? 0x7fffffffffffffffll : static_cast<long long>(c.window);
}

int32_t sliding_extents_fit(const SingeSlidingWindowAttentionConfig& c) {
    const size_t extents[] = {c.batch, c.query_len, c.key_len, c.heads, c.kv_heads, c.head_dim};
    if (int32_t s = extents_fit(extents, 6)) return s;
    size_t last_query = 0, last_key = 0;
    checked_add(c.query_start, c.query_len, &last_query);
    checked_add(c.key_start, c.key_len, &last_key);
    if (last_query > 0x3fffffffffffffffull || last_key > 0x3fffffffffffffffull) return fail(SINGE_HIP_LENGTH_EXCEEDS_I32, "positions");
    return 0;
}

// SlidingWindowAttentionConfig::validate_lengths (mod.rs:570-628): query, key, value, out.
int32_t sliding_window_attention(void* stream, float* out, size_t out_len, const float* query, size_t query_len, const float* key,
                                 size_t key_len, const float* value, size_t value_len, const SingeSlidingWindowAttentionConfig& c,
                                 const char* op) {
    if (int32_t s = validate_sliding_config(c)) return s;
    if (int32_t s = ensure_reach("query", query_len, c.batch, c.query_len, c.heads, c.head_dim, c.query_batch_stride,
                                 c.query_sequence_stride, c.query_head_stride)) return s;
    if (int32_t s = ensure_reach("key", key_len, c.batch, c.key_len, c.kv_heads, c.head_dim, c.key_batch_stride,
                                 c.key_sequence_stride, c.key_head_stride)) return s;
    if (int32_t s = ensure_reach("value", value_len, c.batch, c.key_len, c.kv_heads, c.head_dim, c.value_batch_stride,
                                 c.value_sequence_stride, c.value_head_stride)) return s;
    if (int32_t s = ensure_reach("out", out_len, c.batch, c.query_len, c.heads, c.head_dim,
                                 c.output_batch_stride, c.output_sequence_stride, c.output_head_stride)) return s;
    const void* pointers[] = {out, query, key, value};
    const char* names[] = {"out", "query", "key", "value"};
    if (int32_t s = null_check(pointers, names, 4)) return s;
    if (int32_t s = sliding_extents_fit(c)) return s;
    if (c.head_dim > 256) return fail(SINGE_HIP_UNSUPPORTED_WIDTH, op, c.head_dim, 0);
    DenseGeneralOperands o;
    sliding_operands(o, c);
    o.query = query, o.key = key, o.value = value, o.out = out;
    return dense_general(SINGE_HIP_F32, stream, op, o);
}

}  // namespace

extern "C" {

int32_t singe_hip_softcapped_window_attention_bf16(void* stream, uint16_t* out, size_t out_len, const uint16_t* query, size_t query_len,
                                                   const uint16_t* key, size_t key_len, const uint16_t* value, size_t value_len,
                                                   const SingeSoftcappedWindowAttentionConfig* config) {
    return softcapped_window_attention(stream, false, out, out_len, query, query_len, key, key_len, value, value_len, config,
                                       "softcapped_window_attention_bf16");
}

int32_t singe_hip_softcapped_window_attention_f16(void* stream, uint16_t* out, size_t out_len, const uint16_t* query, size_t query_len,
                                                  const uint16_t* key, size_t key_len, const uint16_t* value, size_t value_len,
                                                  const SingeSoftcappedWindowAttentionConfig* config) {
    return softcapped_window_attention(stream, true, out, out_len, query, query_len, key, key_len, value, value_len, config,
                                       "softcapped_window_attention_f16");
}

int32_t singe_hip_attention_sink_prefill_f32(void* stream, float* out, size_t out_len, const float* query, size_t query_len,
                                             const float* key, size_t key_len, const float* value, size_t value_len, const float* sinks,
                                             size_t sinks_len, const SingeAttentionSinkPrefillConfig* config) {
    return attention_sink_prefill(stream, SINGE_HIP_F32, out, out_len, query, query_len, key, key_len, value, value_len, sinks, sinks_len,
                                  config, "attention_sink_prefill_f32");
}

int32_t singe_hip_attention_sink_prefill_bf16(void* stream, uint16_t* out, size_t out_len, const uint16_t* query, size_t query_len,
                                              const uint16_t* key, size_t key_len, const uint16_t* value, size_t value_len,
                                              const uint16_t* sinks, size_t sinks_len, const SingeAttentionSinkPrefillConfig* config) {
    return attention_sink_prefill(stream, SINGE_HIP_BF16, out, out_len, query, query_len, key, key_len, value, value_len, sinks, sinks_len,
                                  config, "attention_sink_prefill_bf16");
}

int32_t singe_hip_attention_sink_prefill_f16(void* stream, uint16_t* out, size_t out_len, const uint16_t* query, size_t query_len,
                                             const uint16_t* key, size_t key_len, const uint16_t* value, size_t value_len,
                                             const uint16_t* sinks, size_t sinks_len, const SingeAttentionSinkPrefillConfig* config) {
    return attention_sink_prefill(stream, SINGE_HIP_F16, out, out_len, query, query_len, key, key_len, value, value_len, sinks, sinks_len,
                                  config, "attention_sink_prefill_f16");
}

int32_t singe_hip_fmha_decode_lse_f32(void* stream, float* out, size_t out_len, float* lse, size_t lse_len, const float* query,
                                      size_t query_len, const float* key, size_t key_len, const float* value, size_t value_len,
                                      const SingeFmhaDecodeConfig* config) {
    return decode_lse(stream, SINGE_HIP_F32, out, out_len, lse, lse_len, query, query_len, key, key_len, value, value_len, config, 0, 0,
                      0.0f, false, "fmha_decode_lse_f32");
}

int32_t singe_hip_fmha_decode_lse_bf16(void* stream, uint16_t* out, size_t out_len, float* lse, size_t lse_len, const uint16_t* query,
                                       size_t query_len, const uint16_t* key, size_t key_len, const uint16_t* value, size_t value_len,
                                       const SingeFmhaDecodeConfig* config) {
    return decode_lse(stream, SINGE_HIP_BF16, out, out_len, lse, lse_len, query, query_len, key, key_len, value, value_len, config, 0, 0,
                      0.0f, false, "fmha_decode_lse_bf16");
}

int32_t singe_hip_fmha_decode_lse_f16(void* stream, uint16_t* out, size_t out_len, float* lse, size_t lse_len, const uint16_t* query,
                                      size_t query_len, const uint16_t* key, size_t key_len, const uint16_t* value, size_t value_len,
                                      const SingeFmhaDecodeConfig* config) {
    return decode_lse(stream, SINGE_HIP_F16, out, out_len, lse, lse_len, query, query_len, key, key_len, value, value_len, config, 0, 0,
                      0.0f, false, "fmha_decode_lse_f16");
}

int32_t singe_hip_softcapped_window_decode_lse_f32(void* stream, float* out, size_t out_len, float* lse, size_t lse_len,
                                                   const float* query, size_t query_len, const float* key, size_t key_len,
                                                   const float* value, size_t value_len, const SingeSoftcappedWindowDecodeConfig* config) {
    if (config == nullptr) return fail(SINGE_HIP_NULL_POINTER, "config");
    return decode_lse(stream, SINGE_HIP_F32, out, out_len, lse, lse_len, query, query_len, key, key_len, value, value_len,
                      &config->decode, config->window_size, config->has_soft_cap, config->soft_cap, true, "softcapped_window_decode_lse_f32");
}

int32_t singe_hip_softcapped_window_decode_lse_bf16(void* stream, uint16_t* out, size_t out_len, float* lse, size_t lse_len,
                                                    const uint16_t* query, size_t query_len, const uint16_t* key, size_t key_len,
                                                    const uint16_t* value, size_t value_len, const SingeSoftcappedWindowDecodeConfig* config) {
    if (config == nullptr) return fail(SINGE_HIP_NULL_POINTER, "config");
    return decode_lse(stream, SINGE_HIP_BF16, out, out_len, lse, lse_len, query, query_len, key, key_len, value, value_len,
                      &config->decode, config->window_size, config->has_soft_cap, config->soft_cap, true, "softcapped_window_decode_lse_bf16");
}

int32_t singe_hip_softcapped_window_decode_lse_f16(void* stream, uint16_t* out, size_t out_len, float* lse, size_t lse_len,
                                                   const uint16_t* query, size_t query_len, const uint16_t* key, size_t key_len,
                                                   const uint16_t* value, size_t value_len, const SingeSoftcappedWindowDecodeConfig* config) {
    if (config == nullptr) return fail(SINGE_HIP_NULL_POINTER, "config");
    return decode_lse(stream, SINGE_HIP_F16, out, out_len, lse, lse_len, query, query_len, key, key_len, value, value_len,
                      &config->decode, config->window_size, config->has_soft_cap, config->soft_cap, true, "softcapped_window_decode_lse_f16");
}

int32_t singe_hip_ragged_kv_prefill_attention_f32(void* stream, float* out, size_t out_len, float* lse, size_t lse_len, const float* query,
                                                  size_t query_len, const float* key, size_t key_len, const float* value, size_t value_len,
                                                  const int32_t* actual_seq_lens_q, size_t actual_seq_lens_q_len,
                                                  const int32_t* actual_seq_lens_kv, size_t actual_seq_lens_kv_len,
                                                  const int32_t* actual_seq_offsets, size_t actual_seq_offsets_len,
                                                  const SingeRaggedKvPrefillAttentionConfig* config) {
    return ragged_kv_prefill(stream, SINGE_HIP_F32, out, out_len, lse, lse_len, query, query_len, key, key_len, value, value_len,
                             actual_seq_lens_q, actual_seq_lens_q_len, actual_seq_lens_kv, actual_seq_lens_kv_len, actual_seq_offsets,
                             actual_seq_offsets_len, config, "ragged_kv_prefill_attention_f32");
}

int32_t singe_hip_ragged_kv_prefill_attention_bf16(void* stream, uint16_t* out, size_t out_len, float* lse, size_t lse_len,
                                                   const uint16_t* query, size_t query_len, const uint16_t* key, size_t key_len,
                                                   const uint16_t* value, size_t value_len, const int32_t* actual_seq_lens_q,
                                                   size_t actual_seq_lens_q_len, const int32_t* actual_seq_lens_kv,
                                                   size_t actual_seq_lens_kv_len, const int32_t* actual_seq_offsets,
                                                   size_t actual_seq_offsets_len, const SingeRaggedKvPrefillAttentionConfig* config) {
    return ragged_kv_prefill(stream, SINGE_HIP_BF16, out, out_len, lse, lse_len, query, query_len, key, key_len, value, value_len,
                             actual_seq_lens_q, actual_seq_lens_q_len, actual_seq_lens_kv, actual_seq_lens_kv_len, actual_seq_offsets,
                             actual_seq_offsets_len, config, "ragged_kv_prefill_attention_bf16");
}

int32_t singe_hip_ragged_kv_prefill_attention_f16(void* stream, uint16_t* out, size_t out_len, float* lse, size_t lse_len,
                                                  const uint16_t* query, size_t query_len, const uint16_t* key, size_t key_len,
                                                  const uint16_t* value, size_t value_len, const int32_t* actual_seq_lens_q,
                                                  size_t actual_seq_lens_q_len, const int32_t* actual_seq_lens_kv,
                                                  size_t actual_seq_lens_kv_len, const int32_t* actual_seq_offsets,
                                                  size_t actual_seq_offsets_len, const SingeRaggedKvPrefillAttentionConfig* config) {
    return ragged_kv_prefill(stream, SINGE_HIP_F16, out, out_len, lse, lse_len, query, query_len, key, key_len, value, value_len,
                             actual_seq_lens_q, actual_seq_lens_q_len, actual_seq_lens_kv, actual_seq_lens_kv_len, actual_seq_offsets,
                             actual_seq_offsets_len, config, "ragged_kv_prefill_attention_f16");
}

int32_t singe_hip_sliding_window_attention_f32(void* stream, float* out, size_t out_len, const float* query, size_t query_len,
                                               const float* key, size_t key_len, const float* value, size_t value_len,
                                               const SingeSlidingWindowAttentionConfig* config) {
    if (config == nullptr) return fail(SINGE_HIP_NULL_POINTER, "config");
    return sliding_window_attention(stream, out, out_len, query, query_len, key, key_len, value, value_len, *config,
                                    "sliding_window_attention_f32");
}

// sliding_window_attention_packed_qkv_f32 (paged.rs:36-50): query, key and value are views of one buffer from their
// offsets on (validate_packed_qkv_attention_config, mod.rs:2857-2871).
int32_t singe_hip_sliding_window_attention_packed_qkv_f32(void* stream, float* out, size_t out_len, const float* qkv, size_t qkv_len,
                                                          const SingePackedQkvAttentionConfig* config) {
    if (config == nullptr) return fail(SINGE_HIP_NULL_POINTER, "config");
    const SingePackedQkvAttentionConfig& c = *config;
    if (c.query_offset > qkv_len || c.key_offset > qkv_len || c.value_offset > qkv_len)
        return fail(SINGE_HIP_LENGTH_TOO_SHORT, "qkv", c.query_offset > c.key_offset ? (c.query_offset > c.value_offset ? c.query_offset : c.value_offset)
                                                                                      : (c.key_offset > c.value_offset ? c.key_offset : c.value_offset), qkv_len);
    if (qkv == nullptr) return fail(SINGE_HIP_NULL_POINTER, "qkv");
    // The packed form checks the three views against the one buffer and then the output (paged.rs:42-49: the inner
    // launch's own validate_lengths sees the output's real length).
    return sliding_window_attention(stream, out, out_len, qkv + c.query_offset, qkv_len - c.query_offset, qkv + c.key_offset,
                                    qkv_len - c.key_offset, qkv + c.value_offset, qkv_len - c.value_offset, c.attention,
                                    "sliding_window_attention_packed_qkv_f32");
}

// sliding_window_attention_paged_kv_f32 (paged.rs:56-116; kernel arithmetic cutile/kernel/attention/local.rs:9150-9330):
// keys and values behind a block table, a block id outside the cache hides its keys.
int32_t singe_hip_sliding_window_attention_paged_kv_f32(void* stream, float* out, size_t out_len, const float* query, size_t query_len,
                                                        const float* key_cache, size_t key_cache_len, const float* value_cache,
                                                        size_t value_cache_len, const uint32_t* block_table, size_t block_table_len,
                                                        const SingePagedKvAttentionConfig* config) {
    if (config == nullptr) return fail(SINGE_HIP_NULL_POINTER, "config");
    const SingePagedKvAttentionConfig& p = *config;
    const SingeSlidingWindowAttentionConfig& c = p.attention;
    // validate_paged_kv_attention_config (mod.rs:2873-2961).
    if (int32_t s = validate_sliding_config(c)) return s;
    if (p.block_size == 0 || p.physical_blocks == 0 || p.block_table_batch_stride == 0 || p.key_cache_block_stride == 0 ||
        p.value_cache_block_stride == 0)
        return fail(SINGE_HIP_INVALID_LENGTH, "config");
    size_t key_blocks = 0, span = 0, need = 0;
    if (!checked_add(c.key_len, p.block_size - 1, &key_blocks)) return fail(SINGE_HIP_SIZE_OVERFLOW, "block_table");
    key_blocks /= p.block_size;
    if (!checked_mul(c.batch - 1, p.block_table_batch_stride, &span) || !checked_add(span, key_blocks, &need))
        return fail(SINGE_HIP_SIZE_OVERFLOW, "block_table");
    if (int32_t s = ensure_len_at_least("block_table", block_table_len, need)) return s;
    if (int32_t s = ensure_reach("query", query_len, c.batch, c.query_len, c.heads, c.head_dim, c.query_batch_stride,
                                 c.query_sequence_stride, c.query_head_stride)) return s;
    if (int32_t s = ensure_reach("out", out_len, c.batch, c.query_len, c.heads, c.head_dim, c.output_batch_stride,
                                 c.output_sequence_stride, c.output_head_stride)) return s;
    if (int32_t s = ensure_reach("key_cache", key_cache_len, p.physical_blocks, p.block_size, c.kv_heads, c.head_dim,
                                 p.key_cache_block_stride, c.key_sequence_stride, c.key_head_stride)) return s;
    if (int32_t s = ensure_reach("value_cache", value_cache_len, p.physical_blocks, p.block_size, c.kv_heads, c.head_dim,
                                 p.value_cache_block_stride, c.value_sequence_stride, c.value_head_stride)) return s;
    const void* pointers[] = {out, query, key_cache, value_cache, block_table};
    const char* names[] = {"out", "query", "key_cache", "value_cache", "block_table"};
    if (int32_t s = null_check(pointers, names, 5)) return s;
    if (int32_t s = sliding_extents_fit(c)) return s;
    if (!fits_i32(p.block_size) || !fits_i32(p.physical_blocks) || !fits_i32(p.block_table_batch_stride))
        return fail(SINGE_HIP_LENGTH_EXCEEDS_I32, "config");
    if (c.head_dim > 256) return fail(SINGE_HIP_UNSUPPORTED_WIDTH, "sliding_window_attention_paged_kv_f32", c.head_dim, 0);
    DenseGeneralOperands o;
    sliding_operands(o, c);
    o.query = query, o.key = key_cache, o.value = value_cache, o.out = out;
    o.block_table = block_table, o.block_size = p.block_size, o.physical_blocks = p.physical_blocks;
    o.table_stride = p.block_table_batch_stride, o.key_block_stride = p.key_cache_block_stride, o.value_block_stride = p.value_cache_block_stride;
    return dense_general(SINGE_HIP_F32, stream, "sliding_window_attention_paged_kv_f32", o);
}

}  // extern "C"
