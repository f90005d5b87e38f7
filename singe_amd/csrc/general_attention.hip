// Attention for any element type (f32, bf16, f16) and any head dimension up to 256: the fallback the
// tensor-core kernels do not cover, the gfx950 counterpart of the reference's warp-per-row kernels
// (singe/src/backend/cuda/kernel_plan/source/paged_general.rs:73-247) and of the CPU paths
// singe/src/backend/cpu/normalization/attention.rs:191-276 (dense: causal, window, softcap, additive mask,
// sinks, key lengths) and :424-538 (paged, FlashInfer form).
//
// One wave64 per query row.  Lanes take keys 64 apart; a lane's score is the same left-to-right fma chain
// over the head dimension as the CPU path, in f32 for f32 / bf16 / f16 storage (the CPU path widens bf16/f16
// to f32 first: attention.rs:63-69, 297-330) and in f64 for f64 storage (the CPU path and the reference's general
// kernel compute f64 in f64: attention.rs:63-69, paged_general.rs:91-99); its softmax is online in natural base
// with exp, and the 64 per-lane partial rows are merged once at the end.
#include "common.hip.h"
#include "kernel_args.h"
#include "paging.hip.h"

namespace general {

template <uint32_t ELEMENT>
struct Element;
template <>
struct Element<kElementF32> {
    typedef float type;
    typedef float real;  // the type the arithmetic runs in
    static SINGE_DEVICE float load(const type* at) { return *at; }
    static SINGE_DEVICE void store(type* at, float value) { *at = value; }
};
template <>
struct Element<kElementF64> {
    typedef double type;
    typedef double real;
    static SINGE_DEVICE double load(const type* at) { return *at; }
    static SINGE_DEVICE void store(type* at, double value) { *at = value; }
};
template <>
struct Element<kElementBf16> {
    typedef unsigned short type;
    typedef float real;
    static SINGE_DEVICE float load(const type* at) { return __builtin_bit_cast(float, static_cast<unsigned int>(*at) << 16); }
    static SINGE_DEVICE void store(type* at, float value) { *at = f32_to_bf16_bits(value); }
};
template <>
struct Element<kElementF16> {
    typedef _Float16 type;
    typedef float real;
    static SINGE_DEVICE float load(const type* at) { return static_cast<float>(*at); }
    static SINGE_DEVICE void store(type* at, float value) { *at = static_cast<_Float16>(value); }  // round to nearest even
};

// exp, log, tanh and fma in the arithmetic's own precision.
SINGE_DEVICE float real_exp(float x) { return expf(x); }
SINGE_DEVICE double real_exp(double x) { return exp(x); }
SINGE_DEVICE float real_log(float x) { return logf(x); }
SINGE_DEVICE double real_log(double x) { return log(x); }
SINGE_DEVICE float real_tanh(float x) { return tanhf(x); }
SINGE_DEVICE double real_tanh(double x) { return tanh(x); }
SINGE_DEVICE float real_fma(float a, float b, float c) { return fmaf(a, b, c); }
SINGE_DEVICE double real_fma(double a, double b, double c) { return fma(a, b, c); }
SINGE_DEVICE float real_max(float a, float b) { return fmaxf(a, b); }
SINGE_DEVICE double real_max(double a, double b) { return fmax(a, b); }

// The scale in the arithmetic's precision (the CPU path derives its default in the tensors' type: attention.rs:82-87).
template <class R, class Args>
SINGE_DEVICE R own_scale(const Args& a) {
    if constexpr (std::is_same<R, double>::value) return a.scale_wide;
    else return a.scale;
}

// Per-lane running state over the keys a lane has seen.
template <int DMAX, class R = float>
struct LaneState {
    R acc[DMAX];
    R largest;
    R total;
};

template <int DMAX, class R>
SINGE_DEVICE void reset(LaneState<DMAX, R>& state) {
#pragma unroll
    for (int d = 0; d < DMAX; ++d) state.acc[d] = 0;
    state.largest = -INFINITY;
    state.total = 0;
}

// Folds one key into a lane's state.  A score of -inf (a masked key) weighs nothing.
template <class E, int DMAX>
SINGE_DEVICE void fold_key(LaneState<DMAX, typename E::real>& state, const typename E::real* q_row, const typename E::type* k_row,
                           const typename E::type* v_row, unsigned int dim, unsigned int value_dim, typename E::real scale,
                           bool has_softcap, float softcap, typename E::real additive) {
    typedef typename E::real R;
    R score = 0;
    if (k_row != nullptr)
        for (unsigned int d = 0; d < dim; ++d) score = real_fma(q_row[d], static_cast<R>(E::load(k_row + d)), score);
    score *= scale;
    if (has_softcap) score = real_tanh(score / static_cast<R>(softcap)) * static_cast<R>(softcap);
    score += additive;
    if (score == -INFINITY) return;
    const R moved = real_max(state.largest, score);
    const R rescale = real_exp(state.largest - moved);  // exp(-inf) = 0 on the first key
    const R weight = real_exp(score - moved);
    state.total = state.total * rescale + weight;
    state.largest = moved;
#pragma unroll
    for (int d = 0; d < DMAX; ++d)
        if (static_cast<unsigned int>(d) < value_dim)
            state.acc[d] = real_fma(weight, v_row != nullptr ? static_cast<R>(E::load(v_row + d)) : R(0), state.acc[d] * rescale);
}

// Merges the 64 lanes and writes the row.  `sink` joins the softmax without weighing a value
// (attention.rs:255-262); pass -inf for none.  Returns max + ln(sum) of the row, -inf when it saw nothing.
template <class E, int DMAX>
SINGE_DEVICE typename E::real finish_row(const LaneState<DMAX, typename E::real>& state, typename E::type* out, unsigned int value_dim,
                                         unsigned int lane, typename E::real sink, typename E::real output_scale = 1) {
    typedef typename E::real R;
    R row_max = state.largest;
#pragma unroll
    for (int step = 32; step >= 1; step >>= 1) row_max = real_max(row_max, __shfl_xor(row_max, step, 64));
    row_max = real_max(row_max, sink);
    const R mine = state.largest == -INFINITY ? R(0) : real_exp(state.largest - row_max);
    R row_sum = state.total * mine;
#pragma unroll
    for (int step = 32; step >= 1; step >>= 1) row_sum += __shfl_xor(row_sum, step, 64);
    if (sink != -INFINITY) row_sum += real_exp(sink - row_max);
    const R inverse = row_sum > 0 ? R(1) / row_sum : R(0);
#pragma unroll
    for (int d = 0; d < DMAX; ++d) {
        if (static_cast<unsigned int>(d) < value_dim) {
            R value = state.acc[d] * mine;
#pragma unroll
            for (int step = 32; step >= 1; step >>= 1) value += __shfl_xor(value, step, 64);
            // A row that sees no key stays zero (attention.rs:503-515; a key count of zero gives zeros).
            if (lane == (d & 63)) E::store(out + d, output_scale == R(1) ? value * inverse : value * inverse * output_scale);
        }
    }
    return row_sum > 0 ? row_max + real_log(row_sum) : R(-INFINITY);
}

template <uint32_t ELEMENT, int DMAX>
SINGE_DEVICE void dense_body(const GeneralAttentionArgs& a, typename Element<ELEMENT>::real* lds) {
    typedef Element<ELEMENT> E;
    typedef typename E::type T;
    typedef typename E::real R;
    const unsigned int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const unsigned long long row = static_cast<unsigned long long>(blockIdx.x) * 4 + wave;
    const unsigned long long rows = static_cast<unsigned long long>(a.ragged ? 1u : a.batch) * a.heads * a.query_len;
    if (row >= rows) return;
    // The row: (batch, head, query) of a dense problem; with ragged sequences (token, head), the token's sequence
    // found by the lanes (the last sequence that owns it, as the CPU loop's later writes win).
    unsigned int query, head, batch, key_len = a.key_len;
    unsigned long long query_at, key_base = 0, lse_at;
    if (a.ragged) {
        const unsigned int token = static_cast<unsigned int>(row / a.heads);
        head = static_cast<unsigned int>(row % a.heads);
        int owner = -1;
        for (unsigned int first_sequence = 0; first_sequence < a.batch; first_sequence += 64) {
            const unsigned int sequence = first_sequence + lane;
            bool mine = false;
            if (sequence < a.batch) {
                const long long offset = a.sequence_offsets[sequence], count = a.query_lengths[sequence];
                mine = offset >= 0 && count > 0 && static_cast<long long>(token) >= offset && static_cast<long long>(token) < offset + count;
            }
            const unsigned long long owners = __ballot(mine);
            if (owners != 0) owner = static_cast<int>(first_sequence + 63u - static_cast<unsigned int>(__builtin_clzll(owners)));
        }
        if (owner < 0) return;
        batch = 0;
        const long long offset = a.sequence_offsets[owner], keys = a.kv_lengths[owner];
        query = token - static_cast<unsigned int>(offset);
        query_at = token;
        key_base = static_cast<unsigned long long>(offset);
        const long long room = static_cast<long long>(a.total_kv_tokens) - offset;
        key_len = keys <= 0 || room <= 0 ? 0u : static_cast<unsigned int>(keys < room ? keys : room);
        lse_at = static_cast<unsigned long long>(token) * a.heads + head;
    } else {
        query = static_cast<unsigned int>(row % a.query_len);
        head = static_cast<unsigned int>((row / a.query_len) % a.heads);
        batch = static_cast<unsigned int>(row / (static_cast<unsigned long long>(a.query_len) * a.heads));
        query_at = query;
        lse_at = row;  // (batch * heads + head) * query_len + query
    }
    const unsigned int kv_head = head / (a.heads / a.kv_heads);
    const T* q = static_cast<const T*>(a.query) + batch * a.query_strides[0] + head * a.query_strides[1] + query_at * a.query_strides[2];
    const T* k = static_cast<const T*>(a.key) + batch * a.key_strides[0] + kv_head * a.key_strides[1] + key_base * a.key_strides[2];
    const T* v = static_cast<const T*>(a.value) + batch * a.value_strides[0] + kv_head * a.value_strides[1] + key_base * a.value_strides[2];
    const T* mask = a.mask == nullptr ? nullptr
                                      : static_cast<const T*>(a.mask) + batch * a.mask_strides[0] + head * a.mask_strides[1] +
                                            query * a.mask_strides[2];

    R* q_row = lds + wave * DMAX;
    for (unsigned int d = lane; d < a.head_dim; d += 64) q_row[d] = E::load(q + d);
    __builtin_amdgcn_wave_barrier();

    // Keys the row may see (attention.rs:225-246): top-left causal, per-batch key count, the window's
    // `key + window <= query` rule and the look-ahead bound, on positions query_start + query and key_start + key.
    long long first = 0, end = key_len;
    const long long position = a.query_start + static_cast<long long>(query) - a.key_start;  // of the query, in key indices
    if (a.causal && position + 1 < end) end = position + 1;
    if (a.lookahead >= 0 && position + a.lookahead + 1 < end) end = position + a.lookahead + 1;
    if (a.key_lengths != nullptr) {
        const int length = a.key_lengths[batch];
        const long long bound = length > 0 ? length : 0;
        if (bound < end) end = bound;
    }
    if (a.window >= 0 && position + 1 - a.window > first) first = position + 1 - a.window;
    if (end < 0) end = 0;

    LaneState<DMAX, R> state;
    reset(state);
    for (long long key = first + lane; key < end; key += 64) {
        const R additive = mask != nullptr ? static_cast<R>(E::load(mask + key * a.mask_strides[3])) : R(0);
        const T* k_row = k + static_cast<size_t>(key) * a.key_strides[2];
        const T* v_row = v + static_cast<size_t>(key) * a.value_strides[2];
        if (a.block_table != nullptr) {
            const unsigned long long block = a.block_table[static_cast<size_t>(batch) * a.table_stride + static_cast<size_t>(key) / a.block_size];
            if (block >= a.physical_blocks) continue;  // a block outside the cache hides its keys
            const size_t slot = static_cast<size_t>(key) % a.block_size;
            k_row = static_cast<const T*>(a.key) + block * a.key_block_stride + slot * a.key_strides[2] + kv_head * a.key_strides[1];
            v_row = static_cast<const T*>(a.value) + block * a.value_block_stride + slot * a.value_strides[2] + kv_head * a.value_strides[1];
        }
        fold_key<E, DMAX>(state, q_row, k_row, v_row, a.head_dim, a.value_dim, own_scale<R>(a), a.has_softcap != 0, a.softcap, additive);
    }
    const R sink = a.sinks != nullptr ? static_cast<R>(E::load(static_cast<const T*>(a.sinks) + head)) : R(-INFINITY);
    T* out = static_cast<T*>(a.out) + batch * a.out_strides[0] + head * a.out_strides[1] + query_at * a.out_strides[2];
    const R lse = finish_row<E, DMAX>(state, out, a.value_dim, lane, sink, static_cast<R>(a.output_scale));
    if (a.lse != nullptr && lane == 0) a.lse[lse_at] = lse == -INFINITY ? a.empty_lse : static_cast<float>(lse);
}

template <uint32_t ELEMENT, int DMAX, int FORM, bool DECODE = false>
SINGE_DEVICE void paged_rows(const GeneralPagedArgs& a, typename Element<ELEMENT>::real* lds) {
    typedef Element<ELEMENT> E;
    typedef typename E::type T;
    typedef typename E::real R;
    const unsigned int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    // Decoding, every sequence has `heads` rows and a.row_blocks workgroups; otherwise the workgroups of all
    // sequences form one list in sequence order (find_row_unit), which the grid covers without a workgroup for
    // every row a sequence might have had.
    unsigned int sequence, block;
    if (DECODE) {
        sequence = blockIdx.x / a.row_blocks;
        block = blockIdx.x % a.row_blocks;
    } else {
        if (!find_row_unit<FORM>(a.query_offsets, a.query_lengths, a.sequences, a.tokens, a.heads, 4u, blockIdx.x, sequence, block)) return;
        sequence = __builtin_amdgcn_readfirstlane(sequence);
        block = __builtin_amdgcn_readfirstlane(block);
    }
    const unsigned int local_row = block * 4 + wave;  // (query, head) of the sequence
    SequenceSpan span;
    if (DECODE) {
        // One query per sequence, at row `sequence`; a key count is clamped to what the table row addresses.
        const int raw = static_cast<const int*>(a.last_page_lengths)[sequence];
        const unsigned long long reach = static_cast<unsigned long long>(a.page_table) * a.page_size;
        span.query_start = sequence;
        span.page_start = static_cast<long long>(sequence) * a.page_table;
        span.queries = 1;
        span.keys = raw < 0 ? 0u : static_cast<unsigned int>(static_cast<unsigned long long>(raw) < reach ? static_cast<unsigned long long>(raw) : reach);
        span.valid = true;
    } else {
        span = load_span<FORM>(sequence, a.query_offsets, a.page_offsets, a.last_page_lengths, a.query_lengths, a.tokens, a.page_table,
                               a.page_size);
    }
    if (!span.valid) {
        if (threadIdx.x == 0) report_index_error(a.status);
        return;
    }
    if (local_row >= span.queries * a.heads) return;
    const unsigned int query = local_row / a.heads, head = local_row % a.heads;
    const unsigned int kv_head = head / (a.heads / a.kv_heads);
    const size_t flat = (static_cast<size_t>(span.query_start) + query) * a.heads + head;
    const T* q = static_cast<const T*>(a.query_rows) + flat * a.head_dim;

    R* q_row = lds + wave * DMAX;
    for (unsigned int d = lane; d < a.head_dim; d += 64) q_row[d] = E::load(q + d);
    __builtin_amdgcn_wave_barrier();

    // Bottom-right alignment with the CPU path's saturating position (attention.rs:482-488); the block-table form
    // aligns a sequence's queries with its first keys (cpu/attention.rs:1283).
    const long long raw = FORM == kTable ? static_cast<long long>(query)
                                         : static_cast<long long>(span.keys) - static_cast<long long>(span.queries) + query;
    const unsigned int position = raw < 0 ? 0u : static_cast<unsigned int>(raw);
    unsigned int first = 0, end = span.keys;
    if (a.causal && position + 1 < end) end = position + 1;
    if (a.window >= 0) {
        const unsigned long long window = static_cast<unsigned long long>(a.window);
        if (static_cast<unsigned long long>(position) + 1 > window) first = static_cast<unsigned int>(position + 1 - window);
    }

    LaneState<DMAX, R> state;
    reset(state);
    const T* key_cache = static_cast<const T*>(a.key_cache);
    const T* value_cache = static_cast<const T*>(a.value_cache);
    for (unsigned int key = first + lane; key < end; key += 64) {
        const unsigned long long page = read_page<FORM>(a.pages, static_cast<size_t>(span.page_start) + key / a.page_size);
        const bool valid = page < static_cast<unsigned long long>(a.cache_pages);
        if (!valid) report_index_error(a.status);
        if (FORM == kTable && !valid) continue;  // a table entry that is no cache block hides its keys
        // A key behind a bad page id is read as zeros; the status word tells the caller.
        const size_t offset = ((page * a.page_size + key % a.page_size) * a.kv_heads + kv_head) * a.head_dim;
        fold_key<E, DMAX>(state, q_row, valid ? key_cache + offset : nullptr, valid ? value_cache + offset : nullptr, a.head_dim,
                          a.head_dim, own_scale<R>(a), a.has_softcap != 0, a.softcap, R(0));
    }
    const R lse = finish_row<E, DMAX>(state, static_cast<T*>(a.output) + flat * a.head_dim, a.head_dim, lane, R(-INFINITY));
    if (a.lse != nullptr && lane == 0) {
        if (FORM == kTable) a.lse[flat] = lse == -INFINITY ? -1.0e20f : static_cast<float>(lse);  // natural log (cpu/attention.rs:1304-1317)
        else a.lse[flat] = static_cast<float>(lse * static_cast<R>(1.4426950408889634074));       // base two; -inf stays -inf
    }
}

template <uint32_t ELEMENT, int DMAX>
SINGE_DEVICE void paged_body(const GeneralPagedArgs& a, typename Element<ELEMENT>::real* lds) {
    if (a.form == 1)
        paged_rows<ELEMENT, DMAX, kCsrI64>(a, lds);
    else if (a.form == 2)
        paged_rows<ELEMENT, DMAX, kTable>(a, lds);
    else if (a.form == 3)
        paged_rows<ELEMENT, DMAX, kTable, true>(a, lds);
    else
        paged_rows<ELEMENT, DMAX, kCsrI32>(a, lds);
}

}  // namespace general

#define SINGE_GENERAL_KERNELS(TAG, ELEMENT, DMAX)                                                                            \
    extern "C" __global__ __launch_bounds__(256) void singe_attention_general_##TAG##_d##DMAX(GeneralAttentionArgs args) {   \
        __shared__ general::Element<ELEMENT>::real rows[4 * DMAX];                                                           \
        general::dense_body<ELEMENT, DMAX>(args, rows);                                                                      \
    }                                                                                                                        \
    extern "C" __global__ __launch_bounds__(256) void singe_paged_attention_general_##TAG##_d##DMAX(GeneralPagedArgs args) { \
        __shared__ general::Element<ELEMENT>::real rows[4 * DMAX];                                                           \
        general::paged_body<ELEMENT, DMAX>(args, rows);                                                                      \
    }

// The build compiles this file once per element type (SINGE_GENERAL_ELEMENT = 0 f32, 1 bf16, 2 f16), each into its
// own part of the code object.
#ifndef SINGE_GENERAL_ELEMENT
#error "define SINGE_GENERAL_ELEMENT: 0 (f32), 1 (bf16), 2 (f16) or 3 (f64)"
#endif
#if SINGE_GENERAL_ELEMENT == 0
SINGE_GENERAL_KERNELS(f32, kElementF32, 64)
SINGE_GENERAL_KERNELS(f32, kElementF32, 128)
SINGE_GENERAL_KERNELS(f32, kElementF32, 256)
#elif SINGE_GENERAL_ELEMENT == 1
SINGE_GENERAL_KERNELS(bf16, kElementBf16, 64)
SINGE_GENERAL_KERNELS(bf16, kElementBf16, 128)
SINGE_GENERAL_KERNELS(bf16, kElementBf16, 256)
#elif SINGE_GENERAL_ELEMENT == 2
SINGE_GENERAL_KERNELS(f16, kElementF16, 64)
SINGE_GENERAL_KERNELS(f16, kElementF16, 128)
SINGE_GENERAL_KERNELS(f16, kElementF16, 256)
#else
SINGE_GENERAL_KERNELS(f64, kElementF64, 64)
SINGE_GENERAL_KERNELS(f64, kElementF64, 128)
SINGE_GENERAL_KERNELS(f64, kElementF64, 256)
#endif
