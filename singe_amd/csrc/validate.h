// Checked arithmetic and length checks shared by the entry points; the counterparts of
// singe-kernel/src/utility.rs:4-11 (checked_i32_value, checked_element_count) and :245-266
// (ensure_len_at_least).
#pragma once

#include <stddef.h>
#include <stdint.h>

#include "module.h"
#include "singe_hip_attention.h"

namespace singe_hip {

inline bool fits_i32(uint64_t value) { return value <= 0x7fffffffull; }

inline bool checked_mul(size_t a, size_t b, size_t* out) { return !__builtin_mul_overflow(a, b, out); }
inline bool checked_add(size_t a, size_t b, size_t* out) { return !__builtin_add_overflow(a, b, out); }

inline int32_t ensure_len_at_least(const char* name, size_t actual, size_t minimum) {
    if (actual < minimum) return fail(SINGE_HIP_LENGTH_TOO_SHORT, name, minimum, actual);
    return 0;
}

// fmha_prefill.cpp: the bf16 / f16 matrix-core prefill with the options of the dense op.  sinks [heads] and mask are
// in the element type of the query; any pointer may be null, window negative and softcap 0 when absent.
struct DenseOptions {
    // Scratch for key splits (null: none), see singe_hip_scaled_dot_product_attention_scratch.
    void* scratch = nullptr;
    size_t scratch_bytes = 0;
    const uint16_t* sinks = nullptr;
    const int32_t* key_lengths = nullptr;
    const uint16_t* mask = nullptr;
    uint64_t mask_strides[4] = {0, 0, 0, 0};
    long long window = -1;
    float softcap = 0.0f;
};
int32_t dense_prefill_with_options(void* stream, bool f16, uint16_t* out, size_t out_len, const uint16_t* query, size_t query_len,
                                   const uint16_t* key, size_t key_len, const uint16_t* value, size_t value_len,
                                   const SingeFmhaPrefillConfig* config, const DenseOptions& options);

// fmha_prefill.cpp: whether the matrix-core kernels take a call as it lies (a build for the head dimension, strides in
// multiples of eight elements, 16-byte aligned buffers, a (batch, head) slice of keys within 4 GiB).
bool dense_prefill_takes(const SingeFmhaPrefillConfig& config, const void* out, const void* query, const void* key, const void* value);

// fmha_prefill.cpp: the shares the matrix-core dense kernel would split this problem's keys into (1 = none) and the
// scratch they need.
uint32_t dense_prefill_splits(const SingeFmhaPrefillConfig& config);
size_t dense_prefill_scratch_bytes(const SingeFmhaPrefillConfig& config, uint32_t splits);
// Whether the launch gives the query heads of a kv head one tile (few query rows, grouped heads, no causal mask).
bool dense_prefill_packs_heads(const SingeFmhaPrefillConfig& config);

// paged_decode.cpp: the two launches of the matrix-core decode kernels (head_dim a multiple of 16 up to 128) for a config its caller has
// checked, and the workspace they need.  `row_starts` non-null: the table holds rows of their own lengths (row b
// starts at entry row_starts[b]; block_table_batch_stride is then the count of entries in all), the way the paged
// attention op's page lists lie; `lse` non-null: the reduce also leaves each row's base-two log-sum-exp.
struct PagedDecodeLaunch {
    void* stream = nullptr;
    uint16_t* out = nullptr;
    const uint16_t* query = nullptr;
    const void* key_cache = nullptr;
    const void* value_cache = nullptr;
    const float* key_scales = nullptr;
    const float* value_scales = nullptr;
    bool fp8 = false, f16 = false;
    const int32_t* actual_seq_lens = nullptr;
    const uint32_t* block_table = nullptr;
    void* workspace = nullptr;
    size_t workspace_bytes = 0;
    uint32_t phases = 3;
    const uint32_t* row_starts = nullptr;
    const uint32_t* row_begins = nullptr;  // with row_starts: keys at the front of each row that a window hides, or null
    float* lse = nullptr;
};
int32_t launch_paged_decode(const SingePagedKvDecodeAttentionConfig& config, const PagedDecodeLaunch& launch);
size_t paged_decode_workspace_bytes(const SingePagedKvDecodeAttentionConfig& config);

// attention_parameters.cpp: the shares a launch of `workgroups` workgroups over at most `keys` keys splits its keys
// into under the installed AttentionParameters (1 = no split).
uint32_t attention_key_splits(uint64_t workgroups, uint64_t keys);

// general_attention.cpp: the one-wave-per-row kernels behind entry points of other files, for head dimensions the
// matrix-core kernels are not built for.  Block-table prefill (query_lengths given) or decode (query_lengths null).
int32_t paged_table_general(int32_t data_type, void* stream, const char* op, const void* query_rows, const void* key_cache,
                            const void* value_cache, const int32_t* query_offsets, const int32_t* query_lengths,
                            const int32_t* key_lengths, const uint32_t* block_table, void* output, float* lse, uint64_t tokens,
                            uint64_t sequences, uint64_t heads, uint64_t kv_heads, uint64_t head_dim, uint64_t block_size,
                            uint64_t physical_blocks, uint64_t table_stride, bool causal, float scale);
// Dense attention through element strides over (batch, head, position); lse [batch, heads, query_len] natural log.
struct DenseGeneralOperands {
    const void* query = nullptr;
    const void* key = nullptr;
    const void* value = nullptr;
    const void* mask = nullptr;
    const void* sinks = nullptr;
    const int32_t* key_lengths = nullptr;
    void* out = nullptr;
    float* lse = nullptr;
    uint64_t query_strides[3] = {0, 0, 0}, key_strides[3] = {0, 0, 0}, value_strides[3] = {0, 0, 0}, out_strides[3] = {0, 0, 0};
    uint64_t mask_strides[4] = {0, 0, 0, 0};
    long long window = -1;
    uint64_t batch = 0, heads = 0, kv_heads = 0, query_len = 0, key_len = 0, head_dim = 0, value_dim = 0;
    bool causal = false, has_softcap = false;
    float scale = 1.0f, softcap = 0.0f;
    double scale_wide = 1.0;  // for f64 tensors
    // The additions of the singe-kernel surface's dense family (GeneralAttentionArgs says what each means).
    long long query_start = 0, key_start = 0, lookahead = -1;
    float output_scale = 1.0f, empty_lse = -__builtin_inff();
    const uint32_t* block_table = nullptr;
    uint64_t block_size = 0, physical_blocks = 0, table_stride = 0, key_block_stride = 0, value_block_stride = 0;
    bool ragged = false;
    uint64_t total_kv_tokens = 0;
    const int32_t* query_lengths = nullptr;
    const int32_t* kv_lengths = nullptr;
    const int32_t* sequence_offsets = nullptr;
};
int32_t dense_general(int32_t data_type, void* stream, const char* op, const DenseGeneralOperands& operands);

}  // namespace singe_hip
