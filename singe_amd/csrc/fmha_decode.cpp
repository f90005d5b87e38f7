// Host side of the dense f32 split-KV decode: FmhaDecodeSplitKConfig / FmhaDecodeSplitKReduceConfig validation as
// the reference does it (singe-kernel/src/cuda/attention/mod.rs:2263-2308, 2364-2380, 2456-2560, 2661-2760,
// 3530-3555, 3575-3604), the two launches of fmha_decode_splitk_reduce_f32 (fmha.rs:1120-1250) and its choice of
// a split count (singe-kernel/src/cuda/autotune.rs:77-89, 586-733).
#include <algorithm>
#include <cmath>
#include <limits>
#include <map>
#include <mutex>
#include <array>
#include <vector>

#include "kernel_args.h"
#include "module.h"
#include "singe_hip_attention.h"
#include "validate.h"

using namespace singe_hip;

namespace {

// projected_layout_reach (mod.rs:3647-3668) and the two split-layout forms (mod.rs:3612-3645): the elements one
// batch item can address; batched_reach (mod.rs:3670-3677) on top.
bool item_reach(size_t outer, size_t outer_stride, size_t inner, size_t inner_stride, size_t tail, size_t* out) {
    size_t outer_span, inner_span;
    if (outer == 0 || inner == 0) return false;
    return checked_mul(outer - 1, outer_stride, &outer_span) && checked_mul(inner - 1, inner_stride, &inner_span) &&
           checked_add(outer_span, inner_span, out) && checked_add(*out, tail, out);
}

int32_t ensure_batched(const char* name, size_t actual, size_t batch, size_t item, size_t batch_stride) {
    size_t span, need;
    if (batch == 0 || !checked_mul(batch - 1, batch_stride, &span) || !checked_add(span, item, &need))
        return fail(SINGE_HIP_SIZE_OVERFLOW, name);
    return ensure_len_at_least(name, actual, need);
}

// validate_fmha_decode_config (mod.rs:3530-3555).
int32_t validate_decode(const SingeFmhaDecodeConfig& c) {
    const size_t extents[] = {c.batch, c.key_len, c.heads, c.kv_heads, c.head_dim, c.query_batch_stride, c.key_batch_stride,
                              c.value_batch_stride, c.output_batch_stride, c.query_head_stride, c.key_sequence_stride,
                              c.value_sequence_stride, c.output_head_stride, c.key_head_stride, c.value_head_stride};
    for (size_t extent : extents)
        if (extent == 0) return fail(SINGE_HIP_INVALID_LENGTH, "config");
    if (!std::isfinite(c.scale) || c.heads % c.kv_heads != 0) return fail(SINGE_HIP_INVALID_LENGTH, "config");
    return 0;
}

// validate_fmha_decode_splitk_config (mod.rs:3575-3604).
int32_t validate_split(const SingeFmhaDecodeSplitKConfig& c) {
    const size_t extents[] = {c.batch, c.key_len, c.heads, c.kv_heads, c.splits, c.kv_len_per_split, c.head_dim,
                              c.query_batch_stride, c.key_batch_stride, c.value_batch_stride, c.output_batch_stride,
                              c.query_head_stride, c.key_sequence_stride, c.value_sequence_stride, c.output_head_stride,
                              c.output_split_stride, c.key_head_stride, c.value_head_stride, c.lse_batch_stride,
                              c.lse_head_stride};
    for (size_t extent : extents)
        if (extent == 0) return fail(SINGE_HIP_INVALID_LENGTH, "config");
    if (!std::isfinite(c.scale) || c.heads % c.kv_heads != 0) return fail(SINGE_HIP_INVALID_LENGTH, "config");
    return 0;
}

// The query / key / value checks FmhaDecodeConfig::validate_lengths and FmhaDecodeSplitKConfig::validate_lengths
// share (mod.rs:2272-2301, 2709-2741).
template <class Config>
int32_t ensure_inputs(const Config& c, size_t query_len, size_t key_len, size_t value_len) {
    size_t item;
    if (!item_reach(1, 1, c.heads, c.query_head_stride, c.head_dim, &item)) return fail(SINGE_HIP_SIZE_OVERFLOW, "query");
    if (int32_t s = ensure_batched("query", query_len, c.batch, item, c.query_batch_stride)) return s;
    if (!item_reach(c.key_len, c.key_sequence_stride, c.kv_heads, c.key_head_stride, c.head_dim, &item))
        return fail(SINGE_HIP_SIZE_OVERFLOW, "key");
    if (int32_t s = ensure_batched("key", key_len, c.batch, item, c.key_batch_stride)) return s;
    if (!item_reach(c.key_len, c.value_sequence_stride, c.kv_heads, c.value_head_stride, c.head_dim, &item))
        return fail(SINGE_HIP_SIZE_OVERFLOW, "value");
    return ensure_batched("value", value_len, c.batch, item, c.value_batch_stride);
}

// FmhaDecodeSplitKConfig::validate_lengths (mod.rs:2699-2760).
int32_t validate_split_lengths(const SingeFmhaDecodeSplitKConfig& c, size_t out_len, size_t lse_len, size_t query_len,
                               size_t key_len, size_t value_len) {
    if (int32_t s = validate_split(c)) return s;
    if (int32_t s = ensure_inputs(c, query_len, key_len, value_len)) return s;
    size_t item;
    if (!item_reach(c.heads, c.output_head_stride, c.splits, c.output_split_stride, c.head_dim, &item))
        return fail(SINGE_HIP_SIZE_OVERFLOW, "out");
    if (int32_t s = ensure_batched("out", out_len, c.batch, item, c.output_batch_stride)) return s;
    if (!item_reach(c.heads, c.lse_head_stride, 1, 1, c.splits, &item)) return fail(SINGE_HIP_SIZE_OVERFLOW, "lse");
    return ensure_batched("lse", lse_len, c.batch, item, c.lse_batch_stride);
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

int32_t launch_split(void* stream, float* out, float* lse, const float* query, const float* key, const float* value,
                     const SingeFmhaDecodeSplitKConfig& c) {
    // Every extent travels as a 32-bit value, as in the reference's launch (checked_i32_value on each, cutile/attention/splitk.rs).
    const size_t extents[] = {c.batch, c.key_len, c.heads, c.kv_heads, c.splits, c.kv_len_per_split, c.head_dim,
                              c.query_batch_stride, c.key_batch_stride, c.value_batch_stride, c.output_batch_stride,
                              c.query_head_stride, c.key_sequence_stride, c.value_sequence_stride, c.output_head_stride,
                              c.output_split_stride, c.key_head_stride, c.value_head_stride, c.lse_batch_stride,
                              c.lse_head_stride};
    for (size_t extent : extents)
        if (!fits_i32(extent)) return fail(SINGE_HIP_LENGTH_EXCEEDS_I32, "config");
    int index = -1;
    const size_t widths[] = {4, 8, 16, 32, 64, 128, 256};
    for (int i = 0; i < 7; ++i)
        if (c.head_dim == widths[i]) index = i;
    if (index < 0) return fail(SINGE_HIP_UNSUPPORTED_WIDTH, "fmha_decode_splitk_f32", c.head_dim, 0);
    if (out == nullptr) return fail(SINGE_HIP_NULL_POINTER, "out");
    if (lse == nullptr) return fail(SINGE_HIP_NULL_POINTER, "lse");
    if (query == nullptr) return fail(SINGE_HIP_NULL_POINTER, "query");
    if (key == nullptr) return fail(SINGE_HIP_NULL_POINTER, "key");
    if (value == nullptr) return fail(SINGE_HIP_NULL_POINTER, "value");
    FmhaDecodeSplitKArgs args;
    args.out = out;
    args.lse = lse;
    args.query = query;
    args.key = key;
    args.value = value;
    args.query_batch_stride = c.query_batch_stride;
    args.key_batch_stride = c.key_batch_stride;
    args.value_batch_stride = c.value_batch_stride;
    args.output_batch_stride = c.output_batch_stride;
    args.query_head_stride = c.query_head_stride;
    args.key_sequence_stride = c.key_sequence_stride;
    args.value_sequence_stride = c.value_sequence_stride;
    args.output_head_stride = c.output_head_stride;
    args.output_split_stride = c.output_split_stride;
    args.key_head_stride = c.key_head_stride;
    args.value_head_stride = c.value_head_stride;
    args.lse_batch_stride = c.lse_batch_stride;
    args.lse_head_stride = c.lse_head_stride;
    args.batch = static_cast<uint32_t>(c.batch);
    args.key_len = static_cast<uint32_t>(c.key_len);
    args.heads = static_cast<uint32_t>(c.heads);
    args.kv_heads = static_cast<uint32_t>(c.kv_heads);
    args.splits = static_cast<uint32_t>(c.splits);
    args.kv_len_per_split = static_cast<uint32_t>(c.kv_len_per_split);
    args.scale = c.scale;
    // 16-byte loads need every row start on a 16-byte boundary.
    const size_t strides[] = {c.query_batch_stride, c.key_batch_stride, c.value_batch_stride, c.query_head_stride,
                              c.key_sequence_stride, c.value_sequence_stride, c.key_head_stride, c.value_head_stride};
    bool aligned = aligned16(query) && aligned16(key) && aligned16(value);
    for (size_t stride : strides) aligned = aligned && stride % 4 == 0;
    args.aligned = aligned ? 1u : 0u;
    const uint64_t groups = static_cast<uint64_t>(c.batch) * c.kv_heads * c.splits;
    if (groups > 0x7fffffffull) return fail(SINGE_HIP_UNSUPPORTED_CONFIGURATION, "too many workgroups");
    return launch(static_cast<KernelId>(kFmhaDecodeSplitK + index), static_cast<unsigned>(groups), 1, 1, 256, stream, args);
}

// fmha_splitk_decode_config and fmha_splitk_reduce_config (mod.rs:2456-2509): scratch laid out
// attn [batch, heads, splits, dim], lse [batch, heads, splits].
SingeFmhaDecodeSplitKConfig split_config(const SingeFmhaDecodeConfig& d, size_t splits) {
    SingeFmhaDecodeSplitKConfig c;
    c.batch = d.batch;
    c.key_len = d.key_len;
    c.heads = d.heads;
    c.kv_heads = d.kv_heads;
    c.splits = splits;
    c.kv_len_per_split = (d.key_len + splits - 1) / splits;
    c.head_dim = d.head_dim;
    c.query_batch_stride = d.query_batch_stride;
    c.key_batch_stride = d.key_batch_stride;
    c.value_batch_stride = d.value_batch_stride;
    c.output_batch_stride = d.heads * splits * d.head_dim;
    c.query_head_stride = d.query_head_stride;
    c.key_sequence_stride = d.key_sequence_stride;
    c.value_sequence_stride = d.value_sequence_stride;
    c.output_head_stride = splits * d.head_dim;
    c.output_split_stride = d.head_dim;
    c.key_head_stride = d.key_head_stride;
    c.value_head_stride = d.value_head_stride;
    c.lse_batch_stride = d.heads * splits;
    c.lse_head_stride = splits;
    c.scale = d.scale;
    return c;
}

SingeSplitKReduceConfig reduce_config(const SingeFmhaDecodeConfig& d, size_t splits) {
    SingeSplitKReduceConfig c;
    c.batch = d.batch;
    c.heads = d.heads;
    c.splits = splits;
    c.head_dim = d.head_dim;
    c.attn_batch_stride = d.heads * splits * d.head_dim;
    c.attn_head_stride = splits * d.head_dim;
    c.attn_split_stride = d.head_dim;
    c.lse_batch_stride = d.heads * splits;
    c.lse_head_stride = splits;
    c.output_batch_stride = d.output_batch_stride;
    c.output_head_stride = d.output_head_stride;
    return c;
}

// validate_fmha_decode_splitk_reduce_lengths (mod.rs:2511-2539).
int32_t validate_reduce_lengths(const SingeFmhaDecodeSplitKReduceConfig& c, size_t out_len, size_t attn_scratch_len,
                                size_t lse_scratch_len, size_t query_len, size_t key_len, size_t value_len) {
    const SingeFmhaDecodeConfig& d = c.decode;
    if (int32_t s = validate_decode(d)) return s;
    if (c.max_splits == 0) return fail(SINGE_HIP_INVALID_LENGTH, "max_splits");
    if (int32_t s = ensure_inputs(d, query_len, key_len, value_len)) return s;
    size_t item;
    if (!item_reach(1, 1, d.heads, d.output_head_stride, d.head_dim, &item)) return fail(SINGE_HIP_SIZE_OVERFLOW, "out");
    if (int32_t s = ensure_batched("out", out_len, d.batch, item, d.output_batch_stride)) return s;
    size_t rows, scratch_values, attn_values;
    const size_t effective = std::min(c.max_splits, d.key_len);
    if (!checked_mul(d.batch, d.heads, &rows) || !checked_mul(rows, effective, &scratch_values) ||
        !checked_mul(scratch_values, d.head_dim, &attn_values))
        return fail(SINGE_HIP_SIZE_OVERFLOW, "attn_scratch");
    if (int32_t s = ensure_len_at_least("attn_scratch", attn_scratch_len, attn_values)) return s;
    return ensure_len_at_least("lse_scratch", lse_scratch_len, scratch_values);
}

// attention_splitk_candidates (mod.rs:2364-2380).
std::vector<size_t> candidates(const SingeFmhaDecodeSplitKReduceConfig& c) {
    const size_t limit = std::min(c.max_splits, c.decode.key_len);
    std::vector<size_t> splits;
    for (size_t ladder : {1, 2, 4, 8, 16, 32, 64})
        if (ladder <= limit) splits.push_back(ladder);
    if (limit > 0 && (splits.empty() || splits.back() != limit)) splits.push_back(limit);
    std::sort(splits.begin(), splits.end());
    splits.erase(std::unique(splits.begin(), splits.end()), splits.end());
    return splits;
}

// The tune cache: the device and what TuneProblemKey::AttentionSplitK holds (mod.rs:2382-2415): the extents,
// max_splits and the ten strides.
using TuneKey = std::array<size_t, 17>;
std::mutex g_tune_mutex;
std::map<TuneKey, size_t> g_tuned;

bool tune_key(const SingeFmhaDecodeSplitKReduceConfig& c, TuneKey* key) {
    const HipRuntime* hip = hip_runtime();
    int device = 0;
    if (hip == nullptr || hip->hipGetDevice(&device) != hipSuccess) return false;
    const SingeFmhaDecodeConfig& d = c.decode;
    *key = TuneKey{static_cast<size_t>(device), d.batch, d.key_len, d.heads, d.kv_heads, d.head_dim, c.max_splits,
                   d.query_batch_stride, d.key_batch_stride, d.value_batch_stride, d.output_batch_stride, d.query_head_stride,
                   d.key_sequence_stride, d.value_sequence_stride, d.output_head_stride, d.key_head_stride, d.value_head_stride};
    return true;
}

// validate_attention_splitk_tuning (mod.rs:2541-2552).
int32_t validate_tuning(const SingeFmhaDecodeSplitKReduceConfig& c, size_t splits) {
    if (splits == 0 || splits > c.max_splits || splits > c.decode.key_len) return fail(SINGE_HIP_INVALID_LENGTH, "splits");
    return 0;
}

// launch_fmha_decode_splitk_reduce_f32 (fmha.rs:1120-1148).
int32_t launch_pair(void* stream, float* out, size_t out_len, float* attn_scratch, size_t attn_scratch_len, float* lse_scratch,
                    size_t lse_scratch_len, const float* query, const float* key, const float* value,
                    const SingeFmhaDecodeSplitKReduceConfig& c, size_t splits) {
    if (int32_t s = validate_tuning(c, splits)) return s;
    const SingeFmhaDecodeSplitKConfig split = split_config(c.decode, splits);
    if (int32_t s = launch_split(stream, attn_scratch, lse_scratch, query, key, value, split)) return s;
    const SingeSplitKReduceConfig reduce = reduce_config(c.decode, splits);
    return singe_hip_splitk_reduce_f32(stream, out, out_len, attn_scratch, attn_scratch_len, lse_scratch, lse_scratch_len, &reduce);
}

constexpr int kStreamCaptureStatusNone = 0;

// The stream's capture status, or a status on failure.
int32_t capturing(void* stream, bool* active) {
    const HipRuntime* hip = hip_runtime();
    if (hip == nullptr) return fail(SINGE_HIP_RUNTIME_UNAVAILABLE, "libamdhip64");
    int status = kStreamCaptureStatusNone;
    if (hipError_t error = hip->hipStreamIsCapturing(stream, &status)) return fail_hip(error, "hipStreamIsCapturing");
    *active = status != kStreamCaptureStatusNone;
    return 0;
}

}  // namespace

extern "C" {

int32_t singe_hip_fmha_decode_splitk_f32(void* stream, float* out, size_t out_len, float* lse, size_t lse_len, const float* query,
                                         size_t query_len, const float* key, size_t key_len, const float* value,
                                         size_t value_len, const SingeFmhaDecodeSplitKConfig* config) {
    if (config == nullptr) return fail(SINGE_HIP_NULL_POINTER, "config");
    if (int32_t s = validate_split_lengths(*config, out_len, lse_len, query_len, key_len, value_len)) return s;
    return launch_split(stream, out, lse, query, key, value, *config);
}

int32_t singe_hip_attention_splitk_candidates(const SingeFmhaDecodeSplitKReduceConfig* config, size_t* splits, size_t capacity,
                                              size_t* count) {
    if (config == nullptr) return fail(SINGE_HIP_NULL_POINTER, "config");
    if (count == nullptr) return fail(SINGE_HIP_NULL_POINTER, "count");
    const std::vector<size_t> found = candidates(*config);
    *count = found.size();
    if (splits != nullptr)
        for (size_t i = 0; i < found.size() && i < capacity; ++i) splits[i] = found[i];
    return 0;
}

int32_t singe_hip_fmha_decode_splitk_reduce_tuned_splits(const SingeFmhaDecodeSplitKReduceConfig* config, size_t* splits) {
    if (config == nullptr) return fail(SINGE_HIP_NULL_POINTER, "config");
    if (splits == nullptr) return fail(SINGE_HIP_NULL_POINTER, "splits");
    TuneKey key;
    if (!tune_key(*config, &key)) return fail(SINGE_HIP_RUNTIME_UNAVAILABLE, "libamdhip64");
    std::lock_guard<std::mutex> lock(g_tune_mutex);
    auto found = g_tuned.find(key);
    *splits = found == g_tuned.end() ? 0 : found->second;
    return 0;
}

void singe_hip_clear_tune_cache(void) {
    std::lock_guard<std::mutex> lock(g_tune_mutex);
    g_tuned.clear();
}

int32_t singe_hip_fmha_decode_splitk_reduce_f32(void* stream, float* out, size_t out_len, float* attn_scratch,
                                                size_t attn_scratch_len, float* lse_scratch, size_t lse_scratch_len,
                                                const float* query, size_t query_len, const float* key, size_t key_len,
                                                const float* value, size_t value_len,
                                                const SingeFmhaDecodeSplitKReduceConfig* config) {
    if (config == nullptr) return fail(SINGE_HIP_NULL_POINTER, "config");
    const SingeFmhaDecodeSplitKReduceConfig& c = *config;
    if (int32_t s = validate_reduce_lengths(c, out_len, attn_scratch_len, lse_scratch_len, query_len, key_len, value_len)) return s;
    const size_t fallback = std::min(c.max_splits, c.decode.key_len);
    auto run = [&](size_t splits) {
        return launch_pair(stream, out, out_len, attn_scratch, attn_scratch_len, lse_scratch, lse_scratch_len, query, key, value, c,
                           splits);
    };
    switch (c.tuning) {
        case SINGE_HIP_TUNING_DEFAULT: return run(fallback);
        case SINGE_HIP_TUNING_EXPLICIT: return run(c.explicit_splits);
        case SINGE_HIP_TUNING_CACHED: break;
        case SINGE_HIP_TUNING_TUNE:
        case SINGE_HIP_TUNING_RETUNE: {
            // autotune::ensure_not_capturing (autotune.rs:586-592), before anything is looked up or timed.
            bool active = false;
            if (int32_t s = capturing(stream, &active)) return s;
            if (active) return fail(SINGE_HIP_AUTOTUNE_DURING_CAPTURE, "fmha_decode_splitk_reduce_f32");
            break;
        }
        default: return fail(SINGE_HIP_INVALID_ARGUMENT, "tuning");
    }
    TuneKey problem;
    if (!tune_key(c, &problem)) return fail(SINGE_HIP_RUNTIME_UNAVAILABLE, "libamdhip64");
    size_t chosen = 0;
    {
        std::lock_guard<std::mutex> lock(g_tune_mutex);
        auto found = g_tuned.find(problem);
        if (found != g_tuned.end()) chosen = found->second;
    }
    if (c.tuning == SINGE_HIP_TUNING_CACHED) {
        if (chosen == 0) {
            // cache_miss_error (autotune.rs:596-602).
            bool active = false;
            if (int32_t s = capturing(stream, &active)) return s;
            return fail(active ? SINGE_HIP_AUTOTUNE_DURING_CAPTURE : SINGE_HIP_TUNE_CACHE_MISS, "fmha_decode_splitk_reduce_f32");
        }
        return run(chosen);
    }
    if (c.tuning == SINGE_HIP_TUNING_RETUNE || chosen == 0) {
        // tune_candidates (autotune.rs:618-733): per candidate `warmup` launches, then `repeats` timed ones, each
        // between two events; a candidate whose launch fails is skipped; the lowest average wins.
        const HipRuntime* hip = hip_runtime();
        std::vector<size_t> tried = candidates(c);
        if (tried.size() > c.options.max_candidates) tried.resize(c.options.max_candidates);
        if (tried.empty()) return fail(SINGE_HIP_NO_TUNE_CANDIDATES, "fmha_decode_splitk_reduce_f32");
        const size_t repeats = std::max<size_t>(c.options.repeats, 1);
        void *start = nullptr, *stop = nullptr;
        if (hipError_t error = hip->hipEventCreate(&start)) return fail_hip(error, "hipEventCreate");
        if (hipError_t error = hip->hipEventCreate(&stop)) {
            hip->hipEventDestroy(start);
            return fail_hip(error, "hipEventCreate");
        }
        float best_ms = std::numeric_limits<float>::infinity();
        size_t best = 0;
        for (size_t splits : tried) {
            bool failed = false;
            for (size_t i = 0; i < c.options.warmup && !failed; ++i) failed = run(splits) != 0;
            float total = 0.0f;
            for (size_t i = 0; i < repeats && !failed; ++i) {
                float ms = 0.0f;
                failed = hip->hipEventRecord(start, stream) != hipSuccess || run(splits) != 0 ||
                         hip->hipEventRecord(stop, stream) != hipSuccess || hip->hipEventSynchronize(stop) != hipSuccess ||
                         hip->hipEventElapsedTime(&ms, start, stop) != hipSuccess;
                total += ms;
            }
            if (failed) continue;
            const float average = total / static_cast<float>(repeats);
            if (average < best_ms) {
                best_ms = average;
                best = splits;
            }
        }
        hip->hipEventDestroy(start);
        hip->hipEventDestroy(stop);
        if (best == 0) return fail(SINGE_HIP_NO_SUCCESSFUL_TUNE_CANDIDATES, "fmha_decode_splitk_reduce_f32");
        chosen = best;
        std::lock_guard<std::mutex> lock(g_tune_mutex);
        g_tuned[problem] = chosen;
    }
    // The winner is launched once more so the output holds its result (fmha.rs:1238-1249).
    return run(chosen);
}

}  // extern "C"
