/*
 * CPU oracle for the attention hot path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file restates, in plain C, the arithmetic of the reference's own CPU
 * attention functions so that the HIP kernels can be checked against it on
 * the same seeded inputs.  Nothing in the shipped library links or calls it:
 * only the tests, the smoke check and the CPU-baseline leg of the benchmark
 * load it.
 *
 * Faithfulness rules (they are what makes the restatement reproduce the
 * reference's f32 results):
 *   - every dot product and weighted sum is a left-to-right fmaf chain,
 *   - `score * scale` is a separate multiply,
 *   - exp/log/tanh are libm expf/logf/tanhf,
 *   - a softmax weight is expf(s - max) / denom (a divide, not a reciprocal),
 *   - accumulation runs over increasing key index,
 *   - build with -ffp-contract=off and without -ffast-math.
 *
 * Two liberties are taken, both bit-neutral:
 *   - the weight expf(s - max) / denom of one (row, key) pair is evaluated
 *     once and reused for every output dimension (the reference re-evaluates
 *     the same pure expression per dimension); `*_literal` keeps the
 *     reference's loop shape so a test can show the two agree bit for bit,
 *   - independent rows may run on several OpenMP threads (`threads` > 1).
 *
 * Parity pinning: the reference holds no numeric fixture for
 * paged_kv_decode_attention_f32, paged_kv_prefill_attention_f32,
 * fmha_prefill_lse_f32, attend_paged, paged_mla_attention or fmha_decode_splitk_f32 (which
 * has no CPU form in the reference at all: its restatement follows the GPU kernel), and the
 * Rust original cannot be compiled in this image, so their last-ulp f32 outputs are "parity
 * unpinned": pinned only by construction plus closed forms and invariants (see
 * tests/test_oracle.py and tests/test_fmha_decode_splitk_cpu.py) and, to 3e-6, by the
 * answers of a library routine kept as fixtures (tests/test_golden_fixtures.py);
 * everything integer (gather offsets, lengths, the paging error contract),
 * the GQA head map, the causal direction, the fp8 and bf16 codecs are pinned
 * against the reference's own test vectors.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define ORACLE_API __attribute__((visibility("default")))

/* ---- element codecs ------------------------------------------------------ */

/* singe-codegen/src/emit/cuda_c/prelude.rs:91-93  load_bfloat = bits << 16. */
ORACLE_API float oracle_bf16_to_f32(uint16_t bits) {
    uint32_t wide = (uint32_t)bits << 16;
    float value;
    memcpy(&value, &wide, sizeof value);
    return value;
}

/* singe-codegen/src/emit/cuda_c/prelude.rs:94-106  store_bfloat: round to
 * nearest even, NaN becomes a quiet NaN that keeps its top bits. */
ORACLE_API uint16_t oracle_f32_to_bf16(float value) {
    uint32_t bits;
    memcpy(&bits, &value, sizeof bits);
    if ((bits & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((bits >> 16) | 0x0040u);
    return (uint16_t)((bits + 0x7fffu + ((bits >> 16) & 1u)) >> 16);
}

/* singe-kernel/src/cpu/quantization.rs:265-280  f8e4m3_value. */
ORACLE_API float oracle_f8e4m3_value(uint8_t value) {
    float sign = (value & 0x80) == 0 ? 1.0f : -1.0f;
    int exponent = (value >> 3) & 0x0f;
    int mantissa = value & 0x07;
    if (exponent == 0x0f && mantissa == 0x07) return NAN;
    if (exponent == 0) {
        if (mantissa == 0) return sign * 0.0f;
        return sign * ((float)mantissa / 8.0f) * ldexpf(1.0f, -6);
    }
    return sign * (1.0f + (float)mantissa / 8.0f) * ldexpf(1.0f, exponent - 7);
}

/* singe-codegen/src/interpret/minifloat.rs:97-151  Minifloat::encode for the
 * finite e4m3 format (4 exponent bits, 3 mantissa bits, bias 7, largest 448):
 * round to nearest even, overflow and NaN become 0x7f with the sign kept. */
ORACLE_API uint8_t oracle_f8e4m3_encode(double value) {
    const int mantissa = 3, bias = 7;
    const double largest = 448.0;
    uint8_t sign = signbit(value) ? 0x80 : 0;
    uint8_t nan = sign | 0x7f;
    if (isnan(value)) return nan;
    double magnitude = fabs(value);
    if (isinf(magnitude)) return nan;
    if (magnitude == 0.0) return sign;
    int exponent = (int)floor(log2(magnitude));
    if (exponent < 1 - bias) exponent = 1 - bias;
    if (magnitude >= ldexp(1.0, exponent + 1)) exponent += 1;
    double units = nearbyint(magnitude * ldexp(1.0, mantissa - exponent)); /* ties to even */
    if (units * ldexp(1.0, exponent - mantissa) > largest) return nan;
    uint32_t whole = (uint32_t)units;
    if (whole >= (2u << mantissa)) {
        whole >>= 1;
        exponent += 1;
    }
    uint32_t exponent_field, mantissa_field;
    if (whole < (1u << mantissa)) {
        exponent_field = 0;
        mantissa_field = whole;
    } else {
        exponent_field = (uint32_t)(exponent + bias);
        mantissa_field = whole - (1u << mantissa);
    }
    return (uint8_t)(sign | ((exponent_field << mantissa) | mantissa_field));
}

/* ---- shared softmax pieces ------------------------------------------------ */

static float dot_fma(const float *a, const float *b, size_t n) {
    float sum = 0.0f;
    for (size_t i = 0; i < n; ++i) sum = fmaf(a[i], b[i], sum);
    return sum;
}

static float fold_max(const float *scores, size_t n) {
    float largest = -INFINITY;
    for (size_t i = 0; i < n; ++i) largest = fmaxf(largest, scores[i]);
    return largest;
}

/* Turns scores[0..n) into weights expf(s - max) / denom in place and returns
 * denom through *denominator.  Rows are short-lived, so the buffer is reused. */
static float normalise(float *scores, size_t n, float *denominator) {
    float largest = fold_max(scores, n);
    float denom = 0.0f;
    for (size_t i = 0; i < n; ++i) denom += expf(scores[i] - largest);
    for (size_t i = 0; i < n; ++i) scores[i] = expf(scores[i] - largest) / denom;
    *denominator = denom;
    return largest;
}

static int thread_count(int threads) {
#ifdef _OPENMP
    return threads > 0 ? threads : 1;
#else
    (void)threads;
    return 1;
#endif
}

/* ---- singe-kernel: paged decode ------------------------------------------ */

/* singe-kernel/src/cpu/attention.rs:1172-1246  paged_kv_decode_attention_f32.
 * query [batch, heads, dim]; caches [blocks, block_size, kv_heads, dim];
 * block = block_table[b * stride + key / block_size]; out [batch, heads, dim].
 * Returns through `gather` (optional, length = sum of seq lens per batch row,
 * laid out [batch][key]) the element offset of (key, kv_head 0, dim 0) so a
 * test can compare gather indices bit for bit. */
ORACLE_API void oracle_paged_kv_decode_attention_f32(
    float *out, const float *query, const float *key_cache, const float *value_cache,
    const int32_t *actual_seq_lens, const uint32_t *block_table, size_t batch, size_t heads,
    size_t kv_heads, size_t head_dim, size_t block_size, size_t block_table_batch_stride,
    float scale, int threads) {
    size_t group = heads / kv_heads;
    size_t token_stride = kv_heads * head_dim;
    size_t block_stride = block_size * token_stride;
    memset(out, 0, batch * heads * head_dim * sizeof(float));
    long rows = (long)(batch * heads);
#pragma omp parallel for schedule(dynamic, 1) num_threads(thread_count(threads))
    for (long row = 0; row < rows; ++row) {
        size_t b = (size_t)row / heads, head = (size_t)row % heads;
        size_t seq_len = (size_t)actual_seq_lens[b];
        if (seq_len == 0) continue;
        size_t kv_head = head / group;
        float *scores = (float *)malloc(seq_len * sizeof(float));
        const float *q = query + (b * heads + head) * head_dim;
        for (size_t key = 0; key < seq_len; ++key) {
            size_t block = block_table[b * block_table_batch_stride + key / block_size];
            size_t offset = block * block_stride + (key % block_size) * token_stride + kv_head * head_dim;
            scores[key] = dot_fma(q, key_cache + offset, head_dim) * scale;
        }
        float denom;
        normalise(scores, seq_len, &denom);
        float *o = out + (b * heads + head) * head_dim;
        for (size_t key = 0; key < seq_len; ++key) {
            size_t block = block_table[b * block_table_batch_stride + key / block_size];
            size_t offset = block * block_stride + (key % block_size) * token_stride + kv_head * head_dim;
            const float *v = value_cache + offset;
            float w = scores[key];
            for (size_t d = 0; d < head_dim; ++d) o[d] = fmaf(w, v[d], o[d]);
        }
        free(scores);
    }
}

/* Same function with the reference's loop shape kept literally: the weight is
 * recomputed for every output dimension and the block table is looked up again
 * per dimension (singe-kernel/src/cpu/attention.rs:1223-1242). */
ORACLE_API void oracle_paged_kv_decode_attention_f32_literal(
    float *out, const float *query, const float *key_cache, const float *value_cache,
    const int32_t *actual_seq_lens, const uint32_t *block_table, size_t batch, size_t heads,
    size_t kv_heads, size_t head_dim, size_t block_size, size_t block_table_batch_stride,
    float scale) {
    size_t group = heads / kv_heads;
    size_t token_stride = kv_heads * head_dim;
    size_t block_stride = block_size * token_stride;
    memset(out, 0, batch * heads * head_dim * sizeof(float));
    for (size_t b = 0; b < batch; ++b) {
        size_t seq_len = (size_t)actual_seq_lens[b];
        for (size_t head = 0; head < heads; ++head) {
            size_t kv_head = head / group;
            if (seq_len == 0) continue;
            float *scores = (float *)malloc(seq_len * sizeof(float));
            for (size_t key = 0; key < seq_len; ++key) {
                size_t block = block_table[b * block_table_batch_stride + key / block_size];
                size_t token = key % block_size;
                float score = 0.0f;
                for (size_t d = 0; d < head_dim; ++d) {
                    size_t qo = (b * heads + head) * head_dim + d;
                    size_t ko = block * block_stride + token * token_stride + kv_head * head_dim + d;
                    score = fmaf(query[qo], key_cache[ko], score);
                }
                scores[key] = score * scale;
            }
            float largest = fold_max(scores, seq_len);
            float denom = 0.0f;
            for (size_t key = 0; key < seq_len; ++key) denom += expf(scores[key] - largest);
            for (size_t d = 0; d < head_dim; ++d) {
                float sum = 0.0f;
                for (size_t key = 0; key < seq_len; ++key) {
                    size_t block = block_table[b * block_table_batch_stride + key / block_size];
                    size_t token = key % block_size;
                    size_t vo = block * block_stride + token * token_stride + kv_head * head_dim + d;
                    sum = fmaf(expf(scores[key] - largest) / denom, value_cache[vo], sum);
                }
                out[(b * heads + head) * head_dim + d] = sum;
            }
            free(scores);
        }
    }
}

/* The element offset of (key, kv_head, dim 0) inside a [blocks, block_size,
 * kv_heads, dim] cache, for every key of every batch row, in the order
 * [batch][key]; rows are separated by `actual_seq_lens`.  This is the gather
 * index the kernels must reproduce exactly
 * (singe-kernel/src/cpu/attention.rs:1196-1206). */
ORACLE_API void oracle_paged_gather_offsets(
    uint64_t *offsets, const int32_t *actual_seq_lens, const uint32_t *block_table, size_t batch,
    size_t kv_heads, size_t head_dim, size_t block_size, size_t block_table_batch_stride,
    size_t kv_head) {
    size_t token_stride = kv_heads * head_dim;
    size_t block_stride = block_size * token_stride;
    size_t at = 0;
    for (size_t b = 0; b < batch; ++b) {
        size_t seq_len = (size_t)actual_seq_lens[b];
        for (size_t key = 0; key < seq_len; ++key) {
            size_t block = block_table[b * block_table_batch_stride + key / block_size];
            offsets[at++] = block * block_stride + (key % block_size) * token_stride + kv_head * head_dim;
        }
    }
}

/* ---- singe-kernel: paged prefill (top-left causal) ------------------------ */

/* singe-kernel/src/cpu/attention.rs:1248-1341  paged_kv_prefill_attention_f32.
 * query/out [total_query_tokens, heads, dim]; lse [total_query_tokens, heads],
 * natural log, -1.0e20 for a row that sees no key.  Causal hides
 * key_index > query_index with no prefix offset. */
ORACLE_API void oracle_paged_kv_prefill_attention_f32(
    float *out, float *lse, const float *query, const float *key_cache, const float *value_cache,
    const int32_t *actual_seq_lens_q, const int32_t *actual_seq_lens_kv,
    const int32_t *actual_seq_offsets, const uint32_t *block_table, size_t batch,
    size_t total_query_tokens, size_t heads, size_t kv_heads, size_t head_dim, size_t block_size,
    size_t block_table_batch_stride, int causal, float scale, int threads) {
    size_t group = heads / kv_heads;
    size_t features = heads * head_dim;
    size_t token_stride = kv_heads * head_dim;
    size_t block_stride = block_size * token_stride;
    memset(out, 0, total_query_tokens * features * sizeof(float));
    memset(lse, 0, total_query_tokens * heads * sizeof(float));
    for (size_t b = 0; b < batch; ++b) {
        size_t len_q = (size_t)actual_seq_lens_q[b];
        size_t len_kv = (size_t)actual_seq_lens_kv[b];
        size_t seq_offset = (size_t)actual_seq_offsets[b];
        long rows = (long)(len_q * heads);
#pragma omp parallel for schedule(dynamic, 4) num_threads(thread_count(threads))
        for (long row = 0; row < rows; ++row) {
            size_t query_index = (size_t)row / heads, head = (size_t)row % heads;
            size_t token = seq_offset + query_index;
            size_t kv_head = head / group;
            size_t visible = causal ? (query_index + 1 < len_kv ? query_index + 1 : len_kv) : len_kv;
            if (visible == 0) {
                lse[token * heads + head] = -1.0e20f;
                continue;
            }
            float *scores = (float *)malloc(visible * sizeof(float));
            const float *q = query + token * features + head * head_dim;
            for (size_t key = 0; key < visible; ++key) {
                size_t block = block_table[b * block_table_batch_stride + key / block_size];
                size_t offset = block * block_stride + (key % block_size) * token_stride + kv_head * head_dim;
                scores[key] = dot_fma(q, key_cache + offset, head_dim) * scale;
            }
            float denom;
            float largest = normalise(scores, visible, &denom);
            lse[token * heads + head] = largest + logf(denom);
            float *o = out + token * features + head * head_dim;
            for (size_t key = 0; key < visible; ++key) {
                size_t block = block_table[b * block_table_batch_stride + key / block_size];
                size_t offset = block * block_stride + (key % block_size) * token_stride + kv_head * head_dim;
                const float *v = value_cache + offset;
                float w = scores[key];
                for (size_t d = 0; d < head_dim; ++d) o[d] = fmaf(w, v[d], o[d]);
            }
            free(scores);
        }
    }
}

/* ---- singe-kernel: dense prefill ------------------------------------------ */

/* singe-kernel/src/cpu/attention.rs:1758-1833  fmha_prefill_lse_f32.
 * query/out [batch, query_len, heads, dim] (BSHD), key/value
 * [batch, key_len, kv_heads, dim]; lse [batch, heads, query_len], natural log.
 * Causal is top-left.  A row that sees no key gets lse = -inf + ln 0 = NaN in
 * the reference only when key_len == 0, which its validators refuse. */
ORACLE_API void oracle_fmha_prefill_lse_f32(
    float *out, float *lse, const float *query, const float *key, const float *value, size_t batch,
    size_t query_len, size_t key_len, size_t heads, size_t kv_heads, size_t head_dim, float scale,
    int causal, int threads) {
    size_t q_features = heads * head_dim, kv_features = kv_heads * head_dim;
    size_t group = heads / kv_heads;
    memset(out, 0, batch * query_len * q_features * sizeof(float));
    long rows = (long)(batch * heads * query_len);
#pragma omp parallel for schedule(dynamic, 8) num_threads(thread_count(threads))
    for (long row = 0; row < rows; ++row) {
        size_t b = (size_t)row / (heads * query_len);
        size_t head = ((size_t)row / query_len) % heads;
        size_t query_index = (size_t)row % query_len;
        size_t kv_head = head / group;
        size_t visible = causal ? (query_index + 1 < key_len ? query_index + 1 : key_len) : key_len;
        float *scores = (float *)malloc((visible ? visible : 1) * sizeof(float));
        const float *q = query + b * query_len * q_features + query_index * q_features + head * head_dim;
        const float *k = key + b * key_len * kv_features + kv_head * head_dim;
        const float *v = value + b * key_len * kv_features + kv_head * head_dim;
        for (size_t j = 0; j < visible; ++j) scores[j] = dot_fma(q, k + j * kv_features, head_dim) * scale;
        float denom;
        float largest = normalise(scores, visible, &denom);
        lse[b * heads * query_len + head * query_len + query_index] = largest + logf(denom);
        float *o = out + b * query_len * q_features + query_index * q_features + head * head_dim;
        for (size_t j = 0; j < visible; ++j) {
            float w = scores[j];
            const float *vj = v + j * kv_features;
            for (size_t d = 0; d < head_dim; ++d) o[d] = fmaf(w, vj[d], o[d]);
        }
        free(scores);
    }
}

/* Same function with the reference's loop shape kept literally (cpu/attention.rs:1776-1830): one thread, the
 * weight expf(s - max) / denom re-evaluated for every output dimension; restricted to query rows
 * [row_first, row_first + row_count) of every (batch, head), so a benchmark can time a stated share of the rows.
 * Rows outside the range keep out = 0 and lse = 0. */
ORACLE_API void oracle_fmha_prefill_lse_f32_literal(
    float *out, float *lse, const float *query, const float *key, const float *value, size_t batch,
    size_t query_len, size_t key_len, size_t heads, size_t kv_heads, size_t head_dim, float scale,
    int causal, size_t row_first, size_t row_count) {
    size_t q_features = heads * head_dim, kv_features = kv_heads * head_dim;
    size_t group = heads / kv_heads;
    memset(out, 0, batch * query_len * q_features * sizeof(float));
    memset(lse, 0, batch * heads * query_len * sizeof(float));
    size_t row_end = row_first + row_count < query_len ? row_first + row_count : query_len;
    float *scores = (float *)malloc((key_len ? key_len : 1) * sizeof(float));
    size_t *kept = (size_t *)malloc((key_len ? key_len : 1) * sizeof(size_t));
    for (size_t b = 0; b < batch; ++b) {
        for (size_t head = 0; head < heads; ++head) {
            size_t kv_head = head / group;
            for (size_t query_index = row_first; query_index < row_end; ++query_index) {
                size_t count = 0;
                for (size_t key_index = 0; key_index < key_len; ++key_index) {
                    if (causal && key_index > query_index) continue;
                    float score = 0.0f;
                    for (size_t d = 0; d < head_dim; ++d) {
                        size_t qo = b * query_len * q_features + query_index * q_features + head * head_dim + d;
                        size_t ko = b * key_len * kv_features + key_index * kv_features + kv_head * head_dim + d;
                        score = fmaf(query[qo], key[ko], score);
                    }
                    kept[count] = key_index;
                    scores[count++] = score * scale;
                }
                float largest = fold_max(scores, count);
                float denom = 0.0f;
                for (size_t j = 0; j < count; ++j) denom += expf(scores[j] - largest);
                lse[b * heads * query_len + head * query_len + query_index] = largest + logf(denom);
                for (size_t d = 0; d < head_dim; ++d) {
                    float sum = 0.0f;
                    for (size_t j = 0; j < count; ++j) {
                        float weight = expf(scores[j] - largest) / denom;
                        size_t vo = b * key_len * kv_features + kept[j] * kv_features + kv_head * head_dim + d;
                        sum = fmaf(weight, value[vo], sum);
                    }
                    out[b * query_len * q_features + query_index * q_features + head * head_dim + d] = sum;
                }
            }
        }
    }
    free(kept);
    free(scores);
}

/* singe-kernel/src/cpu/attention.rs:1835-1925  softcapped_window_attention_f32.
 * query/out [batch, heads, query_len, dim] (BHSD), key/value
 * [batch, kv_heads, key_len, dim].  window_size 0 = no window; otherwise keys
 * with key + window < query or key > query + window are hidden (symmetric).
 * soft_cap applies when has_soft_cap: tanhf(score / cap) * cap. */
ORACLE_API void oracle_softcapped_window_attention_f32(
    float *out, const float *query, const float *key, const float *value, size_t batch,
    size_t query_len, size_t key_len, size_t heads, size_t kv_heads, size_t head_dim, float scale,
    int causal, size_t window_size, int has_soft_cap, float soft_cap, int threads) {
    size_t q_head_stride = query_len * head_dim, k_head_stride = key_len * head_dim;
    size_t group = heads / kv_heads;
    memset(out, 0, batch * heads * q_head_stride * sizeof(float));
    long rows = (long)(batch * heads * query_len);
#pragma omp parallel for schedule(dynamic, 8) num_threads(thread_count(threads))
    for (long row = 0; row < rows; ++row) {
        size_t b = (size_t)row / (heads * query_len);
        size_t head = ((size_t)row / query_len) % heads;
        size_t query_index = (size_t)row % query_len;
        size_t kv_head = head / group;
        const float *q = query + b * heads * q_head_stride + head * q_head_stride + query_index * head_dim;
        const float *k = key + b * kv_heads * k_head_stride + kv_head * k_head_stride;
        const float *v = value + b * kv_heads * k_head_stride + kv_head * k_head_stride;
        float *scores = (float *)malloc((key_len ? key_len : 1) * sizeof(float));
        size_t *kept = (size_t *)malloc((key_len ? key_len : 1) * sizeof(size_t));
        size_t count = 0;
        for (size_t j = 0; j < key_len; ++j) {
            if (causal && j > query_index) continue;
            if (window_size > 0 && (j + window_size < query_index || j > query_index + window_size)) continue;
            float score = dot_fma(q, k + j * head_dim, head_dim) * scale;
            if (has_soft_cap) score = tanhf(score / soft_cap) * soft_cap;
            scores[count] = score;
            kept[count++] = j;
        }
        if (count > 0) {
            float denom;
            normalise(scores, count, &denom);
            float *o = out + b * heads * q_head_stride + head * q_head_stride + query_index * head_dim;
            for (size_t i = 0; i < count; ++i) {
                float w = scores[i];
                const float *vj = v + kept[i] * head_dim;
                for (size_t d = 0; d < head_dim; ++d) o[d] = fmaf(w, vj[d], o[d]);
            }
        }
        free(kept);
        free(scores);
    }
}

/* singe-kernel/src/cpu/attention.rs:1089-1170  sliding_window_attention_f32.
 * BSHD, causal left window: a key is kept when key_abs <= query_abs and
 * key_abs + window > query_abs.  The reference's closed-form unit tests
 * (cpu/attention.rs:2199-2281) run on this function; it is restated so those
 * vectors pin the shared GQA map and causal direction. */
ORACLE_API void oracle_sliding_window_attention_f32(
    float *out, const float *query, const float *key, const float *value, size_t batch,
    size_t query_len, size_t key_len, size_t heads, size_t kv_heads, size_t head_dim,
    size_t query_start, size_t key_start, size_t window, float scale, float output_scale) {
    size_t q_features = heads * head_dim, kv_features = kv_heads * head_dim;
    size_t group = heads / kv_heads;
    memset(out, 0, batch * query_len * q_features * sizeof(float));
    float *scores = (float *)malloc((key_len ? key_len : 1) * sizeof(float));
    size_t *kept = (size_t *)malloc((key_len ? key_len : 1) * sizeof(size_t));
    for (size_t b = 0; b < batch; ++b)
        for (size_t qi = 0; qi < query_len; ++qi) {
            size_t query_abs = query_start + qi;
            for (size_t head = 0; head < heads; ++head) {
                size_t kv_head = head / group;
                const float *q = query + b * query_len * q_features + qi * q_features + head * head_dim;
                size_t count = 0;
                for (size_t j = 0; j < key_len; ++j) {
                    size_t key_abs = key_start + j;
                    if (key_abs > query_abs || key_abs + window <= query_abs) continue;
                    const float *k = key + b * key_len * kv_features + j * kv_features + kv_head * head_dim;
                    scores[count] = dot_fma(q, k, head_dim) * scale;
                    kept[count++] = j;
                }
                if (count == 0) continue;
                float denom;
                normalise(scores, count, &denom);
                for (size_t d = 0; d < head_dim; ++d) {
                    float sum = 0.0f;
                    for (size_t i = 0; i < count; ++i) {
                        size_t vo = b * key_len * kv_features + kept[i] * kv_features + kv_head * head_dim + d;
                        sum = fmaf(scores[i], value[vo], sum);
                    }
                    out[b * query_len * q_features + qi * q_features + head * head_dim + d] = sum * output_scale;
                }
            }
        }
    free(kept);
    free(scores);
}

/* singe-kernel/src/cpu/attention.rs:1343-1420  ragged_kv_prefill_attention_f32.
 * query [tokens, heads, dim], key / value [kv_tokens, kv_heads, dim] packed by
 * sequence; sequence b owns query tokens offsets[b] .. + lens_q[b] and keys
 * offsets[b] .. + lens_kv[b]; top-left causal; lse [tokens, heads] natural log,
 * -1e20 where a token sees no key.  Tokens no sequence owns stay zero. */
ORACLE_API void oracle_ragged_kv_prefill_attention_f32(
    float *out, float *lse, const float *query, const float *key, const float *value,
    const int32_t *lens_q, const int32_t *lens_kv, const int32_t *offsets, size_t batch,
    size_t total_query_tokens, size_t heads, size_t kv_heads, size_t head_dim, int causal, float scale) {
    size_t group = heads / kv_heads, features = heads * head_dim, kv_features = kv_heads * head_dim;
    memset(out, 0, total_query_tokens * features * sizeof(float));
    memset(lse, 0, total_query_tokens * heads * sizeof(float));
    for (size_t b = 0; b < batch; ++b) {
        size_t seq_q = (size_t)lens_q[b], seq_kv = (size_t)lens_kv[b], offset = (size_t)offsets[b];
        float *scores = (float *)malloc((seq_kv ? seq_kv : 1) * sizeof(float));
        size_t *kept = (size_t *)malloc((seq_kv ? seq_kv : 1) * sizeof(size_t));
        for (size_t qi = 0; qi < seq_q; ++qi) {
            size_t token = offset + qi;
            for (size_t head = 0; head < heads; ++head) {
                size_t kv_head = head / group, count = 0;
                const float *q = query + token * features + head * head_dim;
                for (size_t j = 0; j < seq_kv; ++j) {
                    if (causal && j > qi) continue;
                    scores[count] = dot_fma(q, key + (offset + j) * kv_features + kv_head * head_dim, head_dim) * scale;
                    kept[count++] = j;
                }
                if (count == 0) {
                    lse[token * heads + head] = -1.0e20f;
                    continue;
                }
                float denom;
                float largest = normalise(scores, count, &denom);
                lse[token * heads + head] = largest + logf(denom);
                float *o = out + token * features + head * head_dim;
                for (size_t d = 0; d < head_dim; ++d) {
                    float sum = 0.0f;
                    for (size_t i = 0; i < count; ++i)
                        sum = fmaf(scores[i], value[(offset + kept[i]) * kv_features + kv_head * head_dim + d], sum);
                    o[d] = sum;
                }
            }
        }
        free(kept);
        free(scores);
    }
}

/* singe-kernel/src/cpu/attention.rs:1927-1998  softcapped_window_decode_lse_f32.
 * query / out [batch, heads, dim], key / value [batch, kv_heads, key_len, dim]
 * (BHSD); the query sits at position key_len - 1; window_size w > 0 hides keys
 * with key + w < that position; lse [batch, heads] natural log. */
ORACLE_API void oracle_softcapped_window_decode_lse_f32(
    float *out, float *lse, const float *query, const float *key, const float *value, size_t batch,
    size_t key_len, size_t heads, size_t kv_heads, size_t head_dim, float scale, size_t window_size,
    int has_soft_cap, float soft_cap) {
    size_t key_head_stride = key_len * head_dim, group = heads / kv_heads, position = key_len - 1;
    float *scores = (float *)malloc((key_len ? key_len : 1) * sizeof(float));
    size_t *kept = (size_t *)malloc((key_len ? key_len : 1) * sizeof(size_t));
    for (size_t b = 0; b < batch; ++b)
        for (size_t head = 0; head < heads; ++head) {
            size_t kv_head = head / group, count = 0;
            const float *q = query + b * heads * head_dim + head * head_dim;
            const float *k = key + b * kv_heads * key_head_stride + kv_head * key_head_stride;
            const float *v = value + b * kv_heads * key_head_stride + kv_head * key_head_stride;
            for (size_t j = 0; j < key_len; ++j) {
                if (window_size > 0 && j + window_size < position) continue;
                float score = dot_fma(q, k + j * head_dim, head_dim) * scale;
                if (has_soft_cap) score = tanhf(score / soft_cap) * soft_cap;
                scores[count] = score;
                kept[count++] = j;
            }
            float denom;
            float largest = normalise(scores, count, &denom);
            lse[b * heads + head] = largest + logf(denom);
            float *o = out + b * heads * head_dim + head * head_dim;
            for (size_t d = 0; d < head_dim; ++d) {
                float sum = 0.0f;
                for (size_t i = 0; i < count; ++i) sum = fmaf(scores[i], v[kept[i] * head_dim + d], sum);
                o[d] = sum;
            }
        }
    free(kept);
    free(scores);
}

/* singe-kernel/src/cpu/attention.rs:2073-2155  attention_sink_prefill_f32.
 * BSHD; query q sits at start_q + q; causal hides later keys; window w != 0
 * hides keys before position - (w - 1) (saturating); the head's sink logit
 * joins the row's maximum and denominator and weighs no value.  The weighted
 * sum runs key by key over every dim (an fma into the output row). */
ORACLE_API void oracle_attention_sink_prefill_f32(
    float *out, const float *query, const float *key, const float *value, const float *sinks,
    size_t batch, size_t query_len, size_t key_len, size_t heads, size_t kv_heads, size_t head_dim,
    size_t start_q, size_t window, float scale, int causal) {
    size_t q_features = heads * head_dim, kv_features = kv_heads * head_dim, group = heads / kv_heads;
    memset(out, 0, batch * query_len * q_features * sizeof(float));
    float *scores = (float *)malloc((key_len + 1) * sizeof(float));
    size_t *kept = (size_t *)malloc((key_len + 1) * sizeof(size_t));
    for (size_t b = 0; b < batch; ++b)
        for (size_t qi = 0; qi < query_len; ++qi) {
            size_t position = start_q + qi;
            size_t window_start = window == 0 ? 0 : (position >= window - 1 ? position - (window - 1) : 0);
            for (size_t head = 0; head < heads; ++head) {
                size_t kv_head = head / group, count = 0;
                const float *q = query + b * query_len * q_features + qi * q_features + head * head_dim;
                scores[count++] = sinks[head];
                for (size_t j = 0; j < key_len; ++j) {
                    if ((causal && j > position) || (window != 0 && j < window_start)) continue;
                    kept[count] = j;
                    scores[count++] = dot_fma(q, key + b * key_len * kv_features + j * kv_features + kv_head * head_dim, head_dim) * scale;
                }
                float largest = fold_max(scores, count), denom = 0.0f;
                for (size_t i = 0; i < count; ++i) {
                    scores[i] = expf(scores[i] - largest);
                    denom += scores[i];
                }
                float *o = out + b * query_len * q_features + qi * q_features + head * head_dim;
                for (size_t i = 1; i < count; ++i) {
                    float weight = scores[i] / denom;
                    const float *v = value + b * key_len * kv_features + kept[i] * kv_features + kv_head * head_dim;
                    for (size_t d = 0; d < head_dim; ++d) o[d] = fmaf(weight, v[d], o[d]);
                }
            }
        }
    free(kept);
    free(scores);
}

/* The arithmetic of the reference's sliding_window_attention_paged_kv_f32 kernel
 * (singe-kernel/src/cuda/cutile/kernel/attention/local.rs:9150-9330; the CPU
 * module has no paged form): sliding_window_attention_f32 over keys behind a
 * block table, key j of batch b in slot j % block_size of block
 * table[b * table_stride + j / block_size]; a block id >= physical_blocks hides
 * the key.  Caches [physical_blocks, block_size, kv_heads, dim] contiguous,
 * query / out BSHD contiguous. */
ORACLE_API void oracle_sliding_window_attention_paged_kv_f32(
    float *out, const float *query, const float *key_cache, const float *value_cache,
    const uint32_t *block_table, size_t batch, size_t query_len, size_t key_len, size_t heads,
    size_t kv_heads, size_t head_dim, size_t query_start, size_t key_start, size_t window,
    size_t block_size, size_t physical_blocks, size_t table_stride, float scale, float output_scale) {
    size_t q_features = heads * head_dim, kv_features = kv_heads * head_dim, group = heads / kv_heads;
    memset(out, 0, batch * query_len * q_features * sizeof(float));
    float *scores = (float *)malloc((key_len ? key_len : 1) * sizeof(float));
    size_t *kept = (size_t *)malloc((key_len ? key_len : 1) * sizeof(size_t));
    for (size_t b = 0; b < batch; ++b)
        for (size_t qi = 0; qi < query_len; ++qi) {
            size_t query_abs = query_start + qi;
            for (size_t head = 0; head < heads; ++head) {
                size_t kv_head = head / group, count = 0;
                const float *q = query + b * query_len * q_features + qi * q_features + head * head_dim;
                for (size_t j = 0; j < key_len; ++j) {
                    size_t key_abs = key_start + j;
                    if (key_abs > query_abs || key_abs + window <= query_abs) continue;
                    size_t block = block_table[b * table_stride + j / block_size];
                    if (block >= physical_blocks) continue;
                    size_t row = (block * block_size + j % block_size) * kv_features + kv_head * head_dim;
                    scores[count] = dot_fma(q, key_cache + row, head_dim) * scale;
                    kept[count++] = row;
                }
                if (count == 0) continue;
                float denom;
                normalise(scores, count, &denom);
                float *o = out + b * query_len * q_features + qi * q_features + head * head_dim;
                for (size_t d = 0; d < head_dim; ++d) {
                    float sum = 0.0f;
                    for (size_t i = 0; i < count; ++i) sum = fmaf(scores[i], value_cache[kept[i] + d], sum);
                    o[d] = sum * output_scale;
                }
            }
        }
    free(kept);
    free(scores);
}

/* singe-kernel/src/cpu/attention.rs:2157-2193  splitk_reduce_f32.
 * attn [batch, heads, splits, dim], lse [batch, heads, splits] (natural log);
 * out = sum_s exp(lse_s - max) * attn_s / sum_s exp(lse_s - max). */
ORACLE_API void oracle_splitk_reduce_f32(float *out, const float *attn, const float *lse, size_t batch,
                                         size_t heads, size_t splits, size_t head_dim) {
    for (size_t b = 0; b < batch; ++b)
        for (size_t head = 0; head < heads; ++head) {
            const float *l = lse + b * heads * splits + head * splits;
            float largest = fold_max(l, splits);
            float denom = 0.0f;
            for (size_t s = 0; s < splits; ++s) denom += expf(l[s] - largest);
            for (size_t d = 0; d < head_dim; ++d) {
                float sum = 0.0f;
                for (size_t s = 0; s < splits; ++s) {
                    float weight = expf(l[s] - largest);
                    sum = fmaf(weight, attn[b * heads * splits * head_dim + head * splits * head_dim + s * head_dim + d], sum);
                }
                out[b * heads * head_dim + head * head_dim + d] = sum / denom;
            }
        }
}

/* singe-kernel/src/cuda/cutile/kernel/attention/local.rs:6127-6272  fmha_decode_splitk_f32 (the reference has
 * no CPU form of this function; this restates its kernel, one output element at a time as the kernel does).
 * query [batch, heads, dim], key / value [batch, key_len, kv_heads, dim], contiguous; split s covers keys
 * s * per_split .. + per_split, clipped to key_len.  Two passes like the kernel: the maximum (starting from
 * -1e20, strictly greater wins), then weights expf(score - max); score = (sum_d q_d * k_d) * scale with a
 * multiply and an add per term.  out [batch, heads, splits, dim] = sum / denom, or 0 when denom is 0;
 * lse [batch, heads, splits] = max + logf(denom), or -1e20 when denom is 0. */
ORACLE_API void oracle_fmha_decode_splitk_f32(float *out, float *lse, const float *query, const float *key,
                                              const float *value, size_t batch, size_t key_len, size_t heads,
                                              size_t kv_heads, size_t splits, size_t per_split, size_t head_dim,
                                              float scale) {
    size_t group = heads / kv_heads;
    for (size_t b = 0; b < batch; ++b)
        for (size_t head = 0; head < heads; ++head)
            for (size_t split = 0; split < splits; ++split) {
                const float *q = query + (b * heads + head) * head_dim;
                size_t kv_head = head / group, start = split * per_split;
                float largest = -1.0e20f;
                for (size_t offset = 0; offset < per_split; ++offset) {
                    size_t k = start + offset;
                    if (k >= key_len) continue;
                    const float *row = key + ((b * key_len + k) * kv_heads + kv_head) * head_dim;
                    float score = 0.0f;
                    for (size_t d = 0; d < head_dim; ++d) score = score + q[d] * row[d];
                    score = score * scale;
                    if (score > largest) largest = score;
                }
                float denom = 0.0f;
                float *o = out + ((b * heads + head) * splits + split) * head_dim;
                for (size_t d = 0; d < head_dim; ++d) o[d] = 0.0f;
                for (size_t offset = 0; offset < per_split; ++offset) {
                    size_t k = start + offset;
                    if (k >= key_len) continue;
                    const float *row = key + ((b * key_len + k) * kv_heads + kv_head) * head_dim;
                    const float *v = value + ((b * key_len + k) * kv_heads + kv_head) * head_dim;
                    float score = 0.0f;
                    for (size_t d = 0; d < head_dim; ++d) score = score + q[d] * row[d];
                    score = score * scale;
                    float weight = expf(score - largest);
                    denom = denom + weight;
                    for (size_t d = 0; d < head_dim; ++d) o[d] = o[d] + weight * v[d];
                }
                int has_keys = denom > 0.0f;
                for (size_t d = 0; d < head_dim; ++d) o[d] = has_keys ? o[d] / denom : 0.0f;
                lse[(b * heads + head) * splits + split] = has_keys ? largest + logf(denom) : -1.0e20f;
            }
}

/* ---- singe: dense scaled-dot-product attention ----------------------------- */

/* singe/src/backend/cpu/normalization/attention.rs:191-276
 * execute_scaled_dot_product_attention (f32).  query [batch, heads, L, dim],
 * key [batch, heads, S, dim], value [batch, heads, S, value_dim]: grouped key
 * heads are repeated by the caller before this runs (attention.rs:42-62), so
 * `kv_heads` here does that repeat by index: head h reads kv head h / (heads /
 * kv_heads).  Options: causal (top-left), window (key + window <= query
 * hidden, -1 = none), softcap, additive mask [batch, heads, L, S], one sink
 * logit per head, per-batch key lengths.  All optional pointers may be NULL. */
ORACLE_API void oracle_scaled_dot_product_attention_f32(
    float *out, const float *query, const float *key, const float *value, const float *mask,
    const float *sinks, const int32_t *key_lengths, size_t batch, size_t heads, size_t kv_heads,
    size_t query_len, size_t key_len, size_t head_dim, size_t value_dim, float scale, int causal,
    int64_t window, int has_softcap, float softcap, int threads) {
    size_t group = heads / kv_heads;
    long rows = (long)(batch * heads * query_len);
#pragma omp parallel for schedule(dynamic, 8) num_threads(thread_count(threads))
    for (long row = 0; row < rows; ++row) {
        size_t batch_head = (size_t)row / query_len;
        size_t query_index = (size_t)row % query_len;
        size_t b = batch_head / heads, head = batch_head % heads;
        size_t kv_batch_head = b * kv_heads + head / group;
        const float *q = query + (size_t)row * head_dim;
        const float *keys = key + kv_batch_head * key_len * head_dim;
        const float *values = value + kv_batch_head * key_len * value_dim;
        float *o = out + (size_t)row * value_dim;
        for (size_t f = 0; f < value_dim; ++f) o[f] = 0.0f;
        size_t end = causal ? (key_len < query_index + 1 ? key_len : query_index + 1) : key_len;
        if (key_lengths) {
            int32_t length = key_lengths[b];
            size_t bound = length > 0 ? (size_t)length : 0;
            if (bound < end) end = bound;
        }
        size_t start = 0;
        if (window >= 0) start = query_index + 1 > (size_t)window ? query_index + 1 - (size_t)window : 0;
        if (end < start) end = start;
        size_t visible = end - start;
        float *scores = (float *)malloc((visible ? visible : 1) * sizeof(float));
        for (size_t j = 0; j < visible; ++j) {
            float score = dot_fma(q, keys + (start + j) * head_dim, head_dim) * scale;
            if (has_softcap) score = tanhf(score / softcap) * softcap;
            if (mask) score = score + mask[(size_t)row * key_len + start + j];
            scores[j] = score;
        }
        float largest = fold_max(scores, visible);
        if (sinks) largest = fmaxf(largest, sinks[head]);
        float total = 0.0f;
        for (size_t j = 0; j < visible; ++j) total = total + expf(scores[j] - largest);
        if (sinks) total = total + expf(sinks[head] - largest);
        for (size_t j = 0; j < visible; ++j) {
            float w = expf(scores[j] - largest) / total;
            const float *vj = values + (start + j) * value_dim;
            for (size_t f = 0; f < value_dim; ++f) o[f] = fmaf(w, vj[f], o[f]);
        }
        free(scores);
    }
}

/* ---- singe: paged attention in FlashInfer form ----------------------------- */

/* singe/src/backend/spec/neural/attention.rs:372-406  check_paged_values.
 * Returns 0 when every paging value stays inside the queries, the page table
 * and the cache, 1 (index out of bounds) otherwise.  A sequence with no pages
 * skips the last-page-length and page checks. */
ORACLE_API int oracle_check_paged_values(const int64_t *query_offsets, const int64_t *page_offsets,
                                         const int64_t *pages, const int64_t *last_page_lengths,
                                         size_t sequences, int64_t table, int64_t tokens,
                                         int64_t cache_pages, int64_t page_size) {
    for (size_t s = 0; s < sequences; ++s) {
        int64_t qf = query_offsets[s], ql = query_offsets[s + 1];
        int64_t pf = page_offsets[s], pl = page_offsets[s + 1];
        if (!(0 <= qf && qf <= ql && ql <= tokens)) return 1;
        if (!(0 <= pf && pf <= pl && pl <= table)) return 1;
        if (pf == pl) continue;
        if (!(0 <= last_page_lengths[s] && last_page_lengths[s] <= page_size)) return 1;
        for (int64_t p = pf; p < pl; ++p)
            if (!(0 <= pages[p] && pages[p] < cache_pages)) return 1;
    }
    return 0;
}

/* singe/src/backend/cpu/normalization/attention.rs:424-538  attend_paged (f32).
 * query/out [tokens, heads, dim]; caches [pages, page_size, kv_heads, dim];
 * lse [tokens, heads] base two, -inf for a row that sees no key.  Queries are a
 * sequence's last tokens: query q sits at key position
 * saturating_sub(keys + q, queries) (bottom-right causal).  Returns 1 without
 * touching the outputs when the paging values fail oracle_check_paged_values. */
ORACLE_API int oracle_paged_attention_f32(
    float *out, float *lse, const float *query, const float *key_cache, const float *value_cache,
    const int64_t *query_offsets, const int64_t *page_offsets, const int64_t *pages,
    const int64_t *last_page_lengths, size_t sequences, size_t table, size_t tokens, size_t heads,
    size_t kv_heads, size_t head_dim, size_t page_size, size_t cache_pages, float scale, int causal,
    int64_t window, int has_softcap, float softcap, int threads) {
    if (oracle_check_paged_values(query_offsets, page_offsets, pages, last_page_lengths, sequences,
                                  (int64_t)table, (int64_t)tokens, (int64_t)cache_pages,
                                  (int64_t)page_size))
        return 1;
    const float ln2 = 0.693147180559945309417232121458176568f; /* std::f32::consts::LN_2 */
    size_t group = heads / (kv_heads ? kv_heads : 1);
    if (group == 0) group = 1;
    for (size_t i = 0; i < tokens * heads * head_dim; ++i) out[i] = 0.0f;
    for (size_t i = 0; i < tokens * heads; ++i) lse[i] = -INFINITY;
    for (size_t s = 0; s < sequences; ++s) {
        size_t first_query = (size_t)query_offsets[s], end_query = (size_t)query_offsets[s + 1];
        const int64_t *sequence_pages = pages + page_offsets[s];
        size_t page_count = (size_t)(page_offsets[s + 1] - page_offsets[s]);
        size_t keys = page_count == 0 ? 0 : (page_count - 1) * page_size + (size_t)last_page_lengths[s];
        size_t queries = end_query > first_query ? end_query - first_query : 0;
        long rows = (long)(queries * heads);
#pragma omp parallel for schedule(dynamic, 4) num_threads(thread_count(threads))
        for (long row = 0; row < rows; ++row) {
            size_t token = first_query + (size_t)row / heads, head = (size_t)row % heads;
            size_t reach = keys + token - first_query;
            size_t position = reach > queries ? reach - queries : 0;
            size_t end = causal ? (keys < position + 1 ? keys : position + 1) : keys;
            size_t start = 0;
            if (window >= 0) start = position + 1 > (size_t)window ? position + 1 - (size_t)window : 0;
            if (end < start) end = start;
            size_t visible = end - start;
            if (visible == 0) continue;
            size_t kv_head = head / group;
            const float *q = query + (token * heads + head) * head_dim;
            float *weights = (float *)malloc(visible * sizeof(float));
            for (size_t j = 0; j < visible; ++j) {
                size_t key = start + j;
                size_t slot = (size_t)sequence_pages[key / page_size] * page_size + key % page_size;
                float score = dot_fma(q, key_cache + (slot * kv_heads + kv_head) * head_dim, head_dim) * scale;
                if (has_softcap) score = tanhf(score / softcap) * softcap;
                weights[j] = score;
            }
            float largest = fold_max(weights, visible);
            float total = 0.0f;
            for (size_t j = 0; j < visible; ++j) {
                weights[j] = expf(weights[j] - largest);
                total = total + weights[j];
            }
            lse[token * heads + head] = (largest + logf(total)) / ln2;
            float *o = out + (token * heads + head) * head_dim;
            for (size_t j = 0; j < visible; ++j) {
                size_t key = start + j;
                size_t slot = (size_t)sequence_pages[key / page_size] * page_size + key % page_size;
                const float *v = value_cache + (slot * kv_heads + kv_head) * head_dim;
                float w = weights[j] / total;
                for (size_t d = 0; d < head_dim; ++d) o[d] = fmaf(w, v[d], o[d]);
            }
            free(weights);
        }
    }
    return 0;
}

/* Latent attention over paged caches (singe/src/backend/cpu/normalization/attention.rs:540-679): every head
 * of a token attends over one shared latent cache [pages, page_size, latent], whose rows are the keys, with a
 * positional part [pages, page_size, positional] beside them, and the values.  In f64 as the reference
 * computes it: score = (q_latent . c_latent + q_positional . c_positional) * scale, weights = exp(score -
 * largest) / total, out = sum weights * c_latent; lse = (largest + ln total) / ln 2 as f32, -inf where a row
 * sees no key (:648-658).  Queries are the sequence's last tokens (:620-621).  `out` is f64 -> f32 (the caller
 * rounds to the queries' type as the reference's cast does, :675).  Returns 1 without touching the outputs
 * when the paging values fail oracle_check_paged_values (:589-594). */
ORACLE_API int oracle_paged_mla_attention(
    float *out, float *lse, const float *query, const float *query_positions, const float *latent_cache,
    const float *position_cache, const int64_t *query_offsets, const int64_t *page_offsets, const int64_t *pages,
    const int64_t *last_page_lengths, size_t sequences, size_t table, size_t tokens, size_t heads, size_t latent,
    size_t positional, size_t page_size, size_t cache_pages, int has_scale, float scale_value, int causal, int threads) {
    if (oracle_check_paged_values(query_offsets, page_offsets, pages, last_page_lengths, sequences,
                                  (int64_t)table, (int64_t)tokens, (int64_t)cache_pages, (int64_t)page_size))
        return 1;
    const double ln2 = 0.693147180559945309417232121458176568; /* std::f64::consts::LN_2 */
    const double scale = has_scale ? (double)scale_value : 1.0 / sqrt((double)(latent + positional));
    for (size_t i = 0; i < tokens * heads * latent; ++i) out[i] = 0.0f;
    for (size_t i = 0; i < tokens * heads; ++i) lse[i] = -INFINITY;
    for (size_t s = 0; s < sequences; ++s) {
        size_t first_query = (size_t)query_offsets[s], end_query = (size_t)query_offsets[s + 1];
        const int64_t *sequence_pages = pages + page_offsets[s];
        size_t page_count = (size_t)(page_offsets[s + 1] - page_offsets[s]);
        size_t keys = page_count == 0 ? 0 : (page_count - 1) * page_size + (size_t)last_page_lengths[s];
        size_t queries = end_query > first_query ? end_query - first_query : 0;
        long rows = (long)(queries * heads);
#pragma omp parallel for schedule(dynamic, 4) num_threads(thread_count(threads))
        for (long row_index = 0; row_index < rows; ++row_index) {
            size_t token = first_query + (size_t)row_index / heads, head = (size_t)row_index % heads;
            size_t reach = keys + token - first_query;
            size_t position = reach > queries ? reach - queries : 0;
            size_t end = causal ? (keys < position + 1 ? keys : position + 1) : keys;
            if (end == 0) continue;
            size_t row = token * heads + head;
            const float *latent_query = query + row * latent;
            const float *position_query = query_positions + row * positional;
            double *scores = (double *)malloc(end * sizeof(double));
            double largest = -INFINITY;
            for (size_t key = 0; key < end; ++key) {
                size_t slot = (size_t)sequence_pages[key / page_size] * page_size + key % page_size;
                double first = 0.0, second = 0.0;
                for (size_t d = 0; d < latent; ++d) first += (double)latent_query[d] * (double)latent_cache[slot * latent + d];
                for (size_t d = 0; d < positional; ++d) second += (double)position_query[d] * (double)position_cache[slot * positional + d];
                scores[key] = (first + second) * scale;
                if (scores[key] > largest) largest = scores[key];
            }
            double total = 0.0;
            for (size_t key = 0; key < end; ++key) {
                scores[key] = exp(scores[key] - largest);
                total += scores[key];
            }
            lse[row] = (float)((largest + log(total)) / ln2);
            double *sum = (double *)calloc(latent, sizeof(double));
            for (size_t key = 0; key < end; ++key) {
                size_t slot = (size_t)sequence_pages[key / page_size] * page_size + key % page_size;
                double weight = scores[key] / total;
                for (size_t d = 0; d < latent; ++d) sum[d] += weight * (double)latent_cache[slot * latent + d];
            }
            for (size_t d = 0; d < latent; ++d) out[row * latent + d] = (float)sum[d];
            free(sum);
            free(scores);
        }
    }
    return 0;
}

/* The cache row (slot) of every key of every sequence, in the order
 * [sequence][key]: slot = pages[page_offsets[s] + key / page_size] * page_size
 * + key % page_size (attention.rs:477-479), and each sequence's key count
 * (attention.rs:470-475).  Returns the number of slots written. */
ORACLE_API size_t oracle_paged_slots(uint64_t *slots, uint64_t *key_counts, const int64_t *page_offsets,
                                     const int64_t *pages, const int64_t *last_page_lengths,
                                     size_t sequences, size_t page_size) {
    size_t at = 0;
    for (size_t s = 0; s < sequences; ++s) {
        const int64_t *sequence_pages = pages + page_offsets[s];
        size_t page_count = (size_t)(page_offsets[s + 1] - page_offsets[s]);
        size_t keys = page_count == 0 ? 0 : (page_count - 1) * page_size + (size_t)last_page_lengths[s];
        key_counts[s] = keys;
        if (slots)
            for (size_t key = 0; key < keys; ++key)
                slots[at++] = (uint64_t)sequence_pages[key / page_size] * page_size + key % page_size;
        else
            at += keys;
    }
    return at;
}

/* ---- rotation and cache append ---------------------------------------------- */

/* singe/src/backend/cpu/normalization/attention.rs:132-188  rotary_embedding
 * (f32): rows of head_dim values; row r sits at position r % sequence and
 * rotates its leading `rotary_pairs` INTERLEAVED pairs (2p, 2p+1) by the
 * angles cos/sin [sequence, rotary_pairs]; the rest of the row is copied. */
ORACLE_API void oracle_rotary_embedding_f32(float *out, const float *input, const float *cos_table,
                                            const float *sin_table, size_t rows, size_t sequence,
                                            size_t head_dim, size_t rotary_pairs) {
    memcpy(out, input, rows * head_dim * sizeof(float));
    for (size_t row = 0; row < rows; ++row) {
        const float *token = input + row * head_dim;
        float *o = out + row * head_dim;
        size_t position = row % sequence * rotary_pairs;
        for (size_t pair = 0; pair < rotary_pairs; ++pair) {
            float c = cos_table[position + pair], s = sin_table[position + pair];
            float even = token[2 * pair], odd = token[2 * pair + 1];
            o[2 * pair] = fmaf(odd, -s, even * c);
            o[2 * pair + 1] = fmaf(even, s, odd * c);
        }
    }
}

/* One head of the fused rotation kernel
 * (singe/src/backend/cuda/kernel_plan/source/rotary_cache.rs:92-185): an
 * optional RMS normalisation, scale = rsqrt(mean(x^2) + eps) times an
 * optional weight per element, then HALF-SPLIT pairs (p, p + dim/2):
 * first = a cos - b sin, second = b cos + a sin, angles [dim/2] of the token. */
static void rotate_head(float *out, const float *x, const float *c, const float *s, size_t dim,
                        int has_norm, float eps, const float *weight) {
    size_t half = dim / 2;
    float scale = 1.0f;
    if (has_norm) {
        float squares = 0.0f;
        for (size_t pair = 0; pair < half; ++pair)
            squares += x[pair] * x[pair] + x[pair + half] * x[pair + half];
        scale = 1.0f / sqrtf(squares / (float)dim + eps);
    }
    for (size_t pair = 0; pair < half; ++pair) {
        float a = x[pair], b = x[pair + half];
        if (has_norm) {
            a = a * scale;
            b = b * scale;
            if (weight) {
                a = a * weight[pair];
                b = b * weight[pair + half];
            }
        }
        out[pair] = a * c[pair] - b * s[pair];
        out[pair + half] = b * c[pair] + a * s[pair];
    }
}

/* The fused step before attention, as the reference's kernel runs it
 * (rotary_cache.rs:249-427): rotates queries [T, H, D] into query_out, rotates
 * keys [T, G, D] into key_cache[page[t], slot[t], :, :] and copies values
 * [T, G, D] into value_cache at the same cell; caches are [P, S, G, D] and
 * only the selected cells are written.  A negative page or slot counts from
 * the end (rotary_cache.rs:376-381); one still outside its extent makes the
 * token's cache writes vanish and the status 1.  query may be NULL (H = 0).
 * Returns the status. */
ORACLE_API int oracle_rotary_cache_write_f32(float *query_out, float *key_cache, float *value_cache,
                                             const float *query, const float *key, const float *value,
                                             const float *cos_table, const float *sin_table,
                                             const int64_t *pages, const int64_t *slots, size_t tokens,
                                             size_t query_heads, size_t cache_heads, size_t head_dim,
                                             size_t cache_pages, size_t page_slots, int has_query_norm,
                                             float query_eps, const float *query_weight,
                                             int has_key_norm, float key_eps, const float *key_weight) {
    int status = 0;
    size_t half = head_dim / 2;
    for (size_t t = 0; t < tokens; ++t) {
        const float *c = cos_table + t * half, *s = sin_table + t * half;
        for (size_t h = 0; query && h < query_heads; ++h)
            rotate_head(query_out + (t * query_heads + h) * head_dim, query + (t * query_heads + h) * head_dim,
                        c, s, head_dim, has_query_norm, query_eps, query_weight);
        int64_t page = pages[t], slot = slots[t];
        if (page < 0) page += (int64_t)cache_pages;
        if (slot < 0) slot += (int64_t)page_slots;
        if (page < 0 || page >= (int64_t)cache_pages || slot < 0 || slot >= (int64_t)page_slots) {
            status = 1;
            continue;
        }
        size_t cell = ((size_t)page * page_slots + (size_t)slot) * cache_heads;
        for (size_t g = 0; g < cache_heads; ++g) {
            rotate_head(key_cache + (cell + g) * head_dim, key + (t * cache_heads + g) * head_dim, c, s,
                        head_dim, has_key_norm, key_eps, key_weight);
            memcpy(value_cache + (cell + g) * head_dim, value + (t * cache_heads + g) * head_dim,
                   head_dim * sizeof(float));
        }
    }
    return status;
}

/* The conversion from CSR paging to block-table paging as the reference's
 * kernel does it (kernel_plan/source/paged_attention.rs:325-398): packed
 * offsets from the query offsets clamped into [0, tokens] and made monotone,
 * query lengths, key lengths ((pages - 1) * page_size + last length, 0 for a
 * sequence the bounds check refuses), and the page table [sequences, width],
 * zero-padded, a refused page id left at zero.  Returns the status. */
ORACLE_API int oracle_paging_indices(int32_t *packed_offsets, int32_t *query_lengths, int32_t *key_lengths,
                                     int32_t *page_table, const int64_t *query_offsets,
                                     const int64_t *page_offsets, const int64_t *pages,
                                     const int64_t *last_page_lengths, size_t sequences, int64_t tokens,
                                     int64_t page_count, int64_t page_size, int64_t cache_pages, size_t width,
                                     int64_t row_elements) {
    int status = 0;
    memset(page_table, 0, sequences * width * sizeof(int32_t));
    /* prefix[i] = max over j <= i of the clamped offsets: sequence s starts at
     * prefix[s] and ends at prefix[s + 1] (paged_attention.rs:366-381). */
    int64_t running = 0, start = 0;
    for (size_t i = 0; i <= sequences; ++i) {
        int64_t offset = query_offsets[i];
        offset = offset < 0 ? 0 : (offset > tokens ? tokens : offset);
        if (offset > running) running = offset;
        if (i > 0) query_lengths[i - 1] = (int32_t)(running - start);
        packed_offsets[i] = (int32_t)(running * row_elements);
        start = running;
    }
    for (size_t s = 0; s < sequences; ++s) {
        key_lengths[s] = 0;
        int64_t qs = query_offsets[s], qe = query_offsets[s + 1], ps = page_offsets[s], pe = page_offsets[s + 1];
        int64_t last = last_page_lengths[s];
        if (qs < 0 || qe < qs || qe > tokens || ps < 0 || pe < ps || pe > page_count ||
            (pe > ps && (last < 0 || last > page_size))) {
            status = 1;
            continue;
        }
        key_lengths[s] = (int32_t)(pe > ps ? (pe - ps - 1) * page_size + last : 0);
        for (size_t entry = 0; entry < width && ps + (int64_t)entry < pe; ++entry) {
            int64_t page = pages[ps + (int64_t)entry];
            if (page < 0 || page >= cache_pages) {
                status = 1;
                continue;
            }
            page_table[s * width + entry] = (int32_t)page;
        }
    }
    return status;
}

/* ---- fp8 KV cache --------------------------------------------------------- */

/* Dequantises an fp8-e4m3 cache [blocks, block_size, kv_heads, dim] with one
 * f32 scale per (block, kv_head) to the bf16 values the bf16 oracle then
 * reads: bf16_rne(f8e4m3_value(code) * scale), widened back to f32
 * (quantization.rs:245-263 for value * scale; the rounding to bf16 is the
 * contract of the fp8-KV configuration). */
ORACLE_API void oracle_dequantize_f8e4m3_cache(float *out, const uint8_t *codes, const float *scales,
                                               size_t blocks, size_t block_size, size_t kv_heads,
                                               size_t head_dim) {
    for (size_t block = 0; block < blocks; ++block)
        for (size_t token = 0; token < block_size; ++token)
            for (size_t g = 0; g < kv_heads; ++g) {
                float scale = scales[block * kv_heads + g];
                size_t base = ((block * block_size + token) * kv_heads + g) * head_dim;
                for (size_t d = 0; d < head_dim; ++d)
                    out[base + d] = oracle_bf16_to_f32(oracle_f32_to_bf16(oracle_f8e4m3_value(codes[base + d]) * scale));
            }
}

ORACLE_API int oracle_max_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
