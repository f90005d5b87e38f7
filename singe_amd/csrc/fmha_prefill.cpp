// Host side of dense prefill: FmhaPrefillConfig validation as the reference does it
// (singe-kernel/src/cuda/attention/mod.rs:1602-1756, 3369-3398, 3647-3677) and the launch.
#include <atomic>
#include <cmath>

#include "kernel_args.h"
#include "module.h"
#include "singe_hip_attention.h"
#include "validate.h"

using namespace singe_hip;

namespace {

// Query rows a wave of the dense bf16 / f16 prefill takes: 0 = chosen by problem size, 32, or 64 where the two-tile
// kernel takes the call (singe_hip_set_dense_prefill_rows_per_wave).
std::atomic<uint32_t> g_rows_per_wave{0};

int32_t validate_config(const SingeFmhaPrefillConfig& c) {
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

// projected_layout_reach (mod.rs:3647-3668): elements one batch item can address.
bool layout_reach(size_t sequence_len, size_t heads, size_t head_dim, size_t sequence_stride, size_t head_stride, size_t* out) {
    size_t sequence_span, head_span;
    if (sequence_len == 0 || heads == 0) return false;
    return checked_mul(sequence_len - 1, sequence_stride, &sequence_span) && checked_mul(heads - 1, head_stride, &head_span) &&
           checked_add(sequence_span, head_span, out) && checked_add(*out, head_dim, out);
}

// batched_reach (mod.rs:3670-3677).
bool batched_reach(size_t batch, size_t item_len, size_t batch_stride, size_t* out) {
    size_t span;
    if (batch == 0) return false;
    return checked_mul(batch - 1, batch_stride, &span) && checked_add(span, item_len, out);
}

int32_t ensure_reach(const char* name, size_t actual, size_t batch, size_t sequence_len, size_t heads, size_t head_dim,
                     size_t batch_stride, size_t sequence_stride, size_t head_stride) {
    size_t item = 0, need = 0;
    if (!layout_reach(sequence_len, heads, head_dim, sequence_stride, head_stride, &item) ||
        !batched_reach(batch, item, batch_stride, &need))
        return fail(SINGE_HIP_SIZE_OVERFLOW, name);
    return ensure_len_at_least(name, actual, need);
}

// FmhaPrefillConfig::validate_lengths / validate_output_lengths (mod.rs:1634-1756), in their order,
// then the null checks every DevicePointer implies.
int32_t validate_call(const SingeFmhaPrefillConfig& c, const void* out, size_t out_len, const void* lse, size_t lse_len,
                      bool with_lse, const void* query, size_t query_len, const void* key, size_t key_len,
                      const void* value, size_t value_len) {
    if (int32_t status = validate_config(c)) return status;
    if (int32_t status = ensure_reach("query", query_len, c.batch, c.query_len, c.heads, c.head_dim, c.query_batch_stride,
                                      c.query_sequence_stride, c.query_head_stride)) return status;
    if (int32_t status = ensure_reach("key", key_len, c.batch, c.key_len, c.kv_heads, c.head_dim, c.key_batch_stride,
                                      c.key_sequence_stride, c.key_head_stride)) return status;
    if (int32_t status = ensure_reach("value", value_len, c.batch, c.key_len, c.kv_heads, c.head_dim, c.value_batch_stride,
                                      c.value_sequence_stride, c.value_head_stride)) return status;
    if (int32_t status = ensure_reach("out", out_len, c.batch, c.query_len, c.heads, c.head_dim, c.output_batch_stride,
                                      c.output_sequence_stride, c.output_head_stride)) return status;
    if (with_lse) {
        size_t rows = 0;
        if (!checked_mul(c.batch, c.heads, &rows) || !checked_mul(rows, c.query_len, &rows)) return fail(SINGE_HIP_SIZE_OVERFLOW, "lse");
        if (int32_t status = ensure_len_at_least("lse", lse_len, rows)) return status;
        if (lse == nullptr) return fail(SINGE_HIP_NULL_POINTER, "lse");
    }
    const void* pointers[] = {out, query, key, value};
    const char* names[] = {"out", "query", "key", "value"};
    for (int i = 0; i < 4; ++i)
        if (pointers[i] == nullptr) return fail(SINGE_HIP_NULL_POINTER, names[i]);
    if (!fits_i32(c.query_len) || !fits_i32(c.key_len) || !fits_i32(c.batch) || !fits_i32(c.heads))
        return fail(SINGE_HIP_LENGTH_EXCEEDS_I32, "config");
    return 0;
}

int32_t prefill_f32(void* stream, float* out, size_t out_len, float* lse, size_t lse_len, bool with_lse, const float* query,
                    size_t query_len, const float* key, size_t key_len, const float* value, size_t value_len,
                    const SingeFmhaPrefillConfig* config, size_t window_size, bool has_soft_cap, float soft_cap,
                    const char* op) {
    if (config == nullptr) return fail(SINGE_HIP_NULL_POINTER, "config");
    const SingeFmhaPrefillConfig& c = *config;
    if (int32_t status = validate_call(c, out, out_len, lse, lse_len, with_lse, query, query_len, key, key_len, value, value_len))
        return status;
    if (c.head_dim > 256) return fail(SINGE_HIP_UNSUPPORTED_WIDTH, op, c.head_dim, 0);
    // (the cap first, then the window: validate_softcapped_window_attention_config, singe-kernel/src/cuda/attention/mod.rs:3418-3430)
    if (has_soft_cap && !(std::isfinite(soft_cap) && soft_cap > 0.0f)) return fail(SINGE_HIP_INVALID_LENGTH, "soft_cap");
    if (!fits_i32(window_size)) return fail(SINGE_HIP_LENGTH_EXCEEDS_I32, "window_size");
    PrefillF32Args args;
    args.query = query;
    args.key = key;
    args.value = value;
    args.out = out;
    args.lse = with_lse ? lse : nullptr;
    args.query_batch_stride = c.query_batch_stride;
    args.query_sequence_stride = c.query_sequence_stride;
    args.query_head_stride = c.query_head_stride;
    args.key_batch_stride = c.key_batch_stride;
    args.key_sequence_stride = c.key_sequence_stride;
    args.key_head_stride = c.key_head_stride;
    args.value_batch_stride = c.value_batch_stride;
    args.value_sequence_stride = c.value_sequence_stride;
    args.value_head_stride = c.value_head_stride;
    args.output_batch_stride = c.output_batch_stride;
    args.output_sequence_stride = c.output_sequence_stride;
    args.output_head_stride = c.output_head_stride;
    args.batch = static_cast<uint32_t>(c.batch);
    args.query_len = static_cast<uint32_t>(c.query_len);
    args.key_len = static_cast<uint32_t>(c.key_len);
    args.heads = static_cast<uint32_t>(c.heads);
    args.kv_heads = static_cast<uint32_t>(c.kv_heads);
    args.head_dim = static_cast<uint32_t>(c.head_dim);
    args.causal = c.causal ? 1u : 0u;
    args.window_size = static_cast<uint32_t>(window_size);
    args.has_soft_cap = has_soft_cap ? 1u : 0u;
    args.soft_cap = soft_cap;
    args.scale = c.scale;
    // Head dimensions that are powers of two from 4 to 256 take the row kernel (a workgroup per (batch, query, kv
    // head), several keys per wave step); the rest the one-wave-per-row kernel below.
    const size_t widths[] = {4, 8, 16, 32, 64, 128, 256};
    for (int index = 0; index < 7; ++index) {
        if (c.head_dim != widths[index]) continue;
        const size_t strides[] = {c.query_batch_stride, c.query_sequence_stride, c.query_head_stride, c.key_batch_stride,
                                  c.key_sequence_stride, c.key_head_stride, c.value_batch_stride, c.value_sequence_stride,
                                  c.value_head_stride};
        bool aligned = ((reinterpret_cast<uintptr_t>(query) | reinterpret_cast<uintptr_t>(key) | reinterpret_cast<uintptr_t>(value)) & 15u) == 0;
        for (size_t stride : strides) aligned = aligned && stride % 4 == 0;
        args.aligned = aligned ? 1u : 0u;
        const uint64_t units = static_cast<uint64_t>(c.batch) * c.query_len * c.kv_heads;
        if (units > 0x7fffffffull) return fail(SINGE_HIP_UNSUPPORTED_CONFIGURATION, "too many workgroups");
        return launch(static_cast<KernelId>(kPrefillRowsF32 + index), static_cast<unsigned>(units), 1, 1, 256, stream, args);
    }
    const uint64_t rows = static_cast<uint64_t>(c.batch) * c.heads * c.query_len;
    const uint64_t groups = (rows + 3) / 4;
    if (groups > 0x7fffffffull) return fail(SINGE_HIP_UNSUPPORTED_CONFIGURATION, "too many workgroups");
    const KernelId kernel = c.head_dim <= 32 ? kPrefillF32D32 : c.head_dim <= 64 ? kPrefillF32D64
                            : c.head_dim <= 128 ? kPrefillF32D128 : kPrefillF32D256;
    return launch(kernel, static_cast<unsigned>(groups), 1, 1, 256, stream, args);
}

// Whether a call without options runs on the kernel that gives a wave two 32-row tiles: a head_dim that is a multiple of 16 up to 128, a positive
// scale, no heads packed into one tile, and (unless the knob says 64) 256-row tiles that still fill the chip.
bool two_tiles_a_wave(const SingeFmhaPrefillConfig& c) {
    const uint32_t wanted = g_rows_per_wave.load(std::memory_order_relaxed);
    if (wanted == 32 || !has_pair_build(static_cast<long long>(c.head_dim)) || c.key_len == 0 || !(c.scale > 0.0f) || dense_prefill_packs_heads(c))
        return false;
    const uint64_t rows = (static_cast<uint64_t>(c.batch) * c.heads + 7) / 8 * 8, pair_tiles = (c.query_len + 255) / 256;
    if (wanted == 64) return true;
    // Measured against the 32-row kernel at batch 4 x 32 heads x 4096: faster from head_dim 64 up (1.02 - 1.14 x), at 48
    // without the causal mask only (1.09 x; 0.97 x with it), slower at 32 and 16 under the mask, where the softmax's vector
    // instructions bound both kernels and two waves a SIMD share them out better than one.
    if (c.head_dim < 48 || (c.head_dim == 48 && c.causal)) return false;
    return rows * ((pair_tiles + 1) / 2) >= compute_units();
}

int32_t prefill(void* stream, uint16_t* out, size_t out_len, float* lse, size_t lse_len, bool with_lse,
                const uint16_t* query, size_t query_len, const uint16_t* key, size_t key_len, const uint16_t* value,
                size_t value_len, const SingeFmhaPrefillConfig* config, bool f16 = false, const DenseOptions& options = DenseOptions()) {
    if (config == nullptr) return fail(SINGE_HIP_NULL_POINTER, "config");
    const SingeFmhaPrefillConfig& c = *config;
    if (int32_t status = validate_call(c, out, out_len, lse, lse_len, with_lse, query, query_len, key, key_len, value, value_len))
        return status;

    // What the gfx950 kernel takes: head_dim 128 and rows it can fetch 16 bytes at a time.
    if (!has_matrix_core_build(static_cast<long long>(c.head_dim))) {
        // Other head dimensions (the reference's matrix path takes 16 and 32 too: fmha.rs:752-755) run on the
        // one-wave-per-row kernel, up to 256; without the dense op's options, which only reach here at 64 and 128.
        DenseGeneralOperands o;
        o.query = query, o.key = key, o.value = value, o.out = out, o.lse = with_lse ? lse : nullptr;
        o.query_strides[0] = c.query_batch_stride, o.query_strides[1] = c.query_head_stride, o.query_strides[2] = c.query_sequence_stride;
        o.key_strides[0] = c.key_batch_stride, o.key_strides[1] = c.key_head_stride, o.key_strides[2] = c.key_sequence_stride;
        o.value_strides[0] = c.value_batch_stride, o.value_strides[1] = c.value_head_stride, o.value_strides[2] = c.value_sequence_stride;
        o.out_strides[0] = c.output_batch_stride, o.out_strides[1] = c.output_head_stride, o.out_strides[2] = c.output_sequence_stride;
        o.batch = c.batch, o.heads = c.heads, o.kv_heads = c.kv_heads, o.query_len = c.query_len, o.key_len = c.key_len;
        o.head_dim = o.value_dim = c.head_dim;
        o.causal = c.causal != 0, o.scale = c.scale, o.scale_wide = c.scale;
        return dense_general(f16 ? SINGE_HIP_F16 : SINGE_HIP_BF16, stream, f16 ? "fmha_prefill_f16" : "fmha_prefill_bf16", o);
    }
    const size_t strides[] = {c.query_batch_stride, c.key_batch_stride, c.value_batch_stride, c.output_batch_stride,
                              c.query_sequence_stride, c.key_sequence_stride, c.value_sequence_stride,
                              c.output_sequence_stride, c.query_head_stride, c.key_head_stride,
                              c.value_head_stride, c.output_head_stride};
    for (size_t stride : strides)
        if (stride % 8 != 0) return fail(SINGE_HIP_UNSUPPORTED_CONFIGURATION, "strides must be multiples of 8 elements");
    const uintptr_t addresses[] = {reinterpret_cast<uintptr_t>(out), reinterpret_cast<uintptr_t>(query),
                                   reinterpret_cast<uintptr_t>(key), reinterpret_cast<uintptr_t>(value)};
    for (uintptr_t address : addresses)
        if (address % 16 != 0) return fail(SINGE_HIP_UNSUPPORTED_CONFIGURATION, "buffers must be 16-byte aligned");
    // The kernel addresses the keys of one (batch, head) slice with 32-bit byte offsets.
    const size_t widest = c.key_sequence_stride > c.value_sequence_stride ? c.key_sequence_stride : c.value_sequence_stride;
    size_t slice_bytes = 0;
    if (!checked_mul(c.key_len, widest, &slice_bytes) || !checked_mul(slice_bytes, 2, &slice_bytes) || slice_bytes > 0xffffffffull)
        return fail(SINGE_HIP_UNSUPPORTED_CONFIGURATION, "key_len * sequence stride beyond 4 GiB");
    PrefillArgs args;
    args.query = query;
    args.key = key;
    args.value = value;
    args.out = out;
    args.lse = with_lse ? lse : nullptr;
    args.query_batch_stride = c.query_batch_stride;
    args.query_sequence_stride = c.query_sequence_stride;
    args.query_head_stride = c.query_head_stride;
    args.key_batch_stride = c.key_batch_stride;
    args.key_sequence_stride = c.key_sequence_stride;
    args.key_head_stride = c.key_head_stride;
    args.value_batch_stride = c.value_batch_stride;
    args.value_sequence_stride = c.value_sequence_stride;
    args.value_head_stride = c.value_head_stride;
    args.output_batch_stride = c.output_batch_stride;
    args.output_sequence_stride = c.output_sequence_stride;
    args.output_head_stride = c.output_head_stride;
    args.batch = static_cast<uint32_t>(c.batch);
    args.query_len = static_cast<uint32_t>(c.query_len);
    args.key_len = static_cast<uint32_t>(c.key_len);
    args.heads = static_cast<uint32_t>(c.heads);
    args.kv_heads = static_cast<uint32_t>(c.kv_heads);
    constexpr size_t kTileRows = 32 * kDensePrefillWaves;
    args.query_tiles = static_cast<uint32_t>((c.query_len + kTileRows - 1) / kTileRows);
    args.scale_log2e = c.scale * 1.4426950408889634074f;
    args.sinks = options.sinks;
    args.key_lengths = options.key_lengths;
    const bool with_options = options.mask != nullptr || options.window >= 0 || options.softcap != 0.0f;
    args.mask = options.mask;
    for (int i = 0; i < 4; ++i) args.mask_strides[i] = options.mask_strides[i];
    args.mask_packed = options.mask != nullptr && options.mask_strides[3] == 1 && options.mask_strides[0] % 4 == 0 &&
                               options.mask_strides[1] % 4 == 0 && options.mask_strides[2] % 4 == 0 &&
                               (reinterpret_cast<uintptr_t>(options.mask) & 7u) == 0
                           ? 1u : 0u;
    args.window = options.window;
    if (options.softcap != 0.0f) {
        args.cap_scale = std::fabs(c.scale / options.softcap);
        args.cap_log2e = std::fabs(options.softcap) * 1.4426950408889634074f;
    }
    // A decode step through the dense op (few query rows, grouped heads, no causal mask): the query heads of a kv head
    // share one tile, so its keys and values are fetched once.
    args.packed_heads = dense_prefill_packs_heads(c) ? 1u : 0u;
    const uint64_t rows = (static_cast<uint64_t>(c.batch) * (args.packed_heads ? c.kv_heads : c.heads) + 7) / 8 * 8;
    uint64_t groups = rows * ((args.query_tiles + 1) / 2);  // a workgroup takes a pair of query tiles
    if (groups > 0x7fffffffull) return fail(SINGE_HIP_UNSUPPORTED_CONFIGURATION, "too many workgroups");
    // Key splits, when the caller lent scratch for them and the launch is too small to fill the chip.
    uint32_t splits = options.scratch != nullptr ? dense_prefill_splits(c) : 1;
    if (splits > 1 && (options.scratch_bytes < dense_prefill_scratch_bytes(c, splits) || groups * splits > 0x7fffffffull)) splits = 1;
    args.splits = splits;
    if (splits > 1) {
        const size_t row_count = static_cast<size_t>(c.batch) * c.heads * c.query_len;
        args.partial_out = static_cast<float*>(options.scratch);
        args.partial_lse = args.partial_out + static_cast<size_t>(splits) * row_count * c.head_dim;
        groups *= splits;
    }
    const long long head_dim = static_cast<long long>(c.head_dim);
    // Long rows without options: the kernel that gives a wave two 32-row tiles (256 query rows a
    // workgroup, one workgroup a compute unit), when its launch still fills the chip; a build of its own where the last
    // key tile is not whole.
    if (!with_options && splits == 1 && two_tiles_a_wave(c)) {
        const uint32_t pair_tiles = static_cast<uint32_t>((c.query_len + 255) / 256);
        const uint64_t pair_groups = rows * ((pair_tiles + 1) / 2);
        args.query_tiles = pair_tiles;
        // (the builds that take a last tile that is not whole also take a key count of their own for every batch entry)
        const bool ragged = c.key_len % 64 != 0 || options.key_lengths != nullptr;
        const KernelId pair = static_cast<KernelId>(pair_kernels_at(static_cast<long long>(c.head_dim), false) + (c.causal ? 0 : 1) + (f16 ? 2 : 0) + (ragged ? 4 : 0));
        return launch(pair, static_cast<unsigned>(pair_groups), 1, 1, 256, stream, args);
    }
    const KernelId kernel = static_cast<KernelId>((f16 ? kPrefillCausalF16 : kPrefillCausal) + (c.causal ? 0 : 1) + (with_options ? 4 : 0));
    if (int32_t status = launch(at_head_dim(kernel, head_dim), static_cast<unsigned>(groups), 1, 1, 64 * kDensePrefillWaves, stream, args))
        return status;
    if (splits == 1) return 0;
    const uint64_t merge_groups = (static_cast<uint64_t>(c.batch) * c.heads * c.query_len + 3) / 4;
    if (merge_groups > 0x7fffffffull) return fail(SINGE_HIP_UNSUPPORTED_CONFIGURATION, "too many workgroups");
    const KernelId merge = static_cast<KernelId>(prefill_combine_at(head_dim) + (f16 ? 1 : 0));
    return launch(merge, static_cast<unsigned>(merge_groups), 1, 1, 256, stream, args);
}

}  // namespace

namespace singe_hip {

bool dense_prefill_packs_heads(const SingeFmhaPrefillConfig& c) {
    constexpr size_t kTileRows = 32 * kDensePrefillWaves;
    return !c.causal && c.kv_heads > 0 && c.heads > c.kv_heads && c.heads % c.kv_heads == 0 && c.query_len * (c.heads / c.kv_heads) <= kTileRows;
}

uint32_t dense_prefill_splits(const SingeFmhaPrefillConfig& c) {
    if (!has_matrix_core_build(static_cast<long long>(c.head_dim)) || c.batch == 0 || c.heads == 0 || c.query_len == 0) return 1;
    constexpr size_t kTileRows = 32 * kDensePrefillWaves;
    const uint64_t query_tiles = (c.query_len + kTileRows - 1) / kTileRows;
    const uint64_t workgroups = static_cast<uint64_t>(c.batch) * (dense_prefill_packs_heads(c) ? c.kv_heads : c.heads) * ((query_tiles + 1) / 2);
    return attention_key_splits(workgroups, c.key_len);
}

size_t dense_prefill_scratch_bytes(const SingeFmhaPrefillConfig& c, uint32_t splits) {
    if (splits <= 1) return 0;
    return static_cast<size_t>(splits) * c.batch * c.heads * c.query_len * (c.head_dim + 1) * sizeof(float);
}

// The dense op's way into the matrix-core kernel: the public entry points' checks and launch, plus the op's options
// (general_attention.cpp).
bool dense_prefill_takes(const SingeFmhaPrefillConfig& c, const void* out, const void* query, const void* key, const void* value) {
    if (!has_matrix_core_build(static_cast<long long>(c.head_dim))) return false;
    const size_t strides[] = {c.query_batch_stride, c.key_batch_stride, c.value_batch_stride, c.output_batch_stride,
                              c.query_sequence_stride, c.key_sequence_stride, c.value_sequence_stride,
                              c.output_sequence_stride, c.query_head_stride, c.key_head_stride,
                              c.value_head_stride, c.output_head_stride};
    for (size_t stride : strides)
        if (stride % 8 != 0) return false;
    const uintptr_t addresses[] = {reinterpret_cast<uintptr_t>(out), reinterpret_cast<uintptr_t>(query),
                                   reinterpret_cast<uintptr_t>(key), reinterpret_cast<uintptr_t>(value)};
    for (uintptr_t address : addresses)
        if (address % 16 != 0) return false;
    const size_t widest = c.key_sequence_stride > c.value_sequence_stride ? c.key_sequence_stride : c.value_sequence_stride;
    size_t slice_bytes = 0;
    return checked_mul(c.key_len, widest, &slice_bytes) && checked_mul(slice_bytes, 2, &slice_bytes) && slice_bytes <= 0xffffffffull;
}

int32_t dense_prefill_with_options(void* stream, bool f16, uint16_t* out, size_t out_len, const uint16_t* query, size_t query_len,
                                   const uint16_t* key, size_t key_len, const uint16_t* value, size_t value_len,
                                   const SingeFmhaPrefillConfig* config, const DenseOptions& options) {
    return prefill(stream, out, out_len, nullptr, 0, false, query, query_len, key, key_len, value, value_len, config, f16, options);
}

}  // namespace singe_hip

extern "C" {

int32_t singe_hip_fmha_prefill_config_validate(const SingeFmhaPrefillConfig* config) {
    if (config == nullptr) return fail(SINGE_HIP_NULL_POINTER, "config");
    return validate_config(*config);
}

int32_t singe_hip_fmha_prefill_f32(void* stream, float* out, size_t out_len, const float* query, size_t query_len,
                                   const float* key, size_t key_len, const float* value, size_t value_len,
                                   const SingeFmhaPrefillConfig* config) {
    return prefill_f32(stream, out, out_len, nullptr, 0, false, query, query_len, key, key_len, value, value_len, config, 0,
                       false, 0.0f, "fmha_prefill_f32");
}

int32_t singe_hip_fmha_prefill_lse_f32(void* stream, float* out, size_t out_len, float* lse, size_t lse_len,
                                       const float* query, size_t query_len, const float* key, size_t key_len,
                                       const float* value, size_t value_len, const SingeFmhaPrefillConfig* config) {
    return prefill_f32(stream, out, out_len, lse, lse_len, true, query, query_len, key, key_len, value, value_len, config, 0,
                       false, 0.0f, "fmha_prefill_lse_f32");
}

int32_t singe_hip_softcapped_window_attention_f32(void* stream, float* out, size_t out_len, const float* query,
                                                  size_t query_len, const float* key, size_t key_len, const float* value,
                                                  size_t value_len, const SingeSoftcappedWindowAttentionConfig* config) {
    if (config == nullptr) return fail(SINGE_HIP_NULL_POINTER, "config");
    return prefill_f32(stream, out, out_len, nullptr, 0, false, query, query_len, key, key_len, value, value_len,
                       &config->attention, config->window_size, config->has_soft_cap != 0, config->soft_cap,
                       "softcapped_window_attention_f32");
}

int32_t singe_hip_fmha_prefill_bf16(void* stream, uint16_t* out, size_t out_len, const uint16_t* query, size_t query_len,
                                    const uint16_t* key, size_t key_len, const uint16_t* value, size_t value_len,
                                    const SingeFmhaPrefillConfig* config) {
    return prefill(stream, out, out_len, nullptr, 0, false, query, query_len, key, key_len, value, value_len, config);
}

int32_t singe_hip_fmha_prefill_lse_bf16(void* stream, uint16_t* out, size_t out_len, float* lse, size_t lse_len,
                                        const uint16_t* query, size_t query_len, const uint16_t* key, size_t key_len,
                                        const uint16_t* value, size_t value_len, const SingeFmhaPrefillConfig* config) {
    return prefill(stream, out, out_len, lse, lse_len, true, query, query_len, key, key_len, value, value_len, config);
}

// fmha_prefill_f16 / fmha_prefill_lse_f16 (fmha.rs): the same kernels on f16 operands.
int32_t singe_hip_fmha_prefill_f16(void* stream, uint16_t* out, size_t out_len, const uint16_t* query, size_t query_len,
                                   const uint16_t* key, size_t key_len, const uint16_t* value, size_t value_len,
                                   const SingeFmhaPrefillConfig* config) {
    return prefill(stream, out, out_len, nullptr, 0, false, query, query_len, key, key_len, value, value_len, config, true);
}

int32_t singe_hip_fmha_prefill_lse_f16(void* stream, uint16_t* out, size_t out_len, float* lse, size_t lse_len,
                                       const uint16_t* query, size_t query_len, const uint16_t* key, size_t key_len,
                                       const uint16_t* value, size_t value_len, const SingeFmhaPrefillConfig* config) {
    return prefill(stream, out, out_len, lse, lse_len, true, query, query_len, key, key_len, value, value_len, config, true);
}

}  // extern "C"

extern "C" void singe_hip_set_dense_prefill_rows_per_wave(uint32_t rows) { g_rows_per_wave.store(rows, std::memory_order_relaxed); }

extern "C" uint32_t singe_hip_dense_prefill_rows_per_wave(const SingeFmhaPrefillConfig* config) {
    if (config == nullptr) return 0;
    return has_matrix_core_build(static_cast<long long>(config->head_dim)) ? (two_tiles_a_wave(*config) ? 64u : 32u) : 0u;
}
