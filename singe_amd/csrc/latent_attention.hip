// Latent attention over paged caches (DeepSeek's absorbed MLA), any element type: every head of a token attends
// over one shared latent cache [pages, page_size, latent], whose rows are the keys, with a positional part
// [pages, page_size, positional] beside them, and the values.  The gfx950 counterpart of the CPU
// paged_mla_attention (singe/src/backend/cpu/normalization/attention.rs:540-679) and of the reference's
// kernel plan (singe/src/backend/cuda/kernel_plan/source/mla.rs), in the FlashInfer paging form with the same
// in-kernel checks as paged attention.  score = (q_latent . c_latent + q_positional . c_positional) * scale;
// out [tokens, heads, latent]; lse [tokens, heads] base two, -inf for a row that sees no key.
//
// One wave64 per (token, head) row, keys in chunks of 64.  Scoring: lane j takes key j of the chunk, the whole
// key width against the query held in LDS.  Output: lane l owns latent dims l, l + 64, ...; the chunk's
// weights and cache rows go round by lane index.  f32 arithmetic whatever the storage type.  This is the
// general, vector-unit form: correct for every shape the op allows up to a latent width of 512 and a
// positional width of 128, not a matrix-core kernel.
#include "common.hip.h"
#include "kernel_args.h"
#include "paging.hip.h"

namespace latent {

constexpr int kMaxLatent = 512, kMaxPositional = 128;

template <uint32_t ELEMENT> struct Element;
template <> struct Element<kElementF32> {
    typedef float type;
    static SINGE_DEVICE float load(const type* at) { return *at; }
    static SINGE_DEVICE void store(type* at, float value) { *at = value; }
};
template <> struct Element<kElementBf16> {
    typedef unsigned short type;
    static SINGE_DEVICE float load(const type* at) { return __builtin_bit_cast(float, static_cast<unsigned int>(*at) << 16); }
    static SINGE_DEVICE void store(type* at, float value) { *at = f32_to_bf16_bits(value); }
};
template <> struct Element<kElementF16> {
    typedef _Float16 type;
    static SINGE_DEVICE float load(const type* at) { return static_cast<float>(*at); }
    static SINGE_DEVICE void store(type* at, float value) { *at = static_cast<_Float16>(value); }
};

SINGE_DEVICE float wave_max(float value) {
#pragma unroll
    for (int step = 32; step > 0; step >>= 1) value = fmaxf(value, __shfl_xor(value, step, 64));
    return value;
}
SINGE_DEVICE float wave_sum(float value) {
#pragma unroll
    for (int step = 32; step > 0; step >>= 1) value += __shfl_xor(value, step, 64);
    return value;
}

template <uint32_t ELEMENT, int FORM>
SINGE_DEVICE void latent_rows(const LatentAttentionArgs& a, float* lds) {
    typedef Element<ELEMENT> E;
    typedef typename E::type T;
    const unsigned int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    // The workgroups of all sequences form one list in sequence order (find_row_unit), four rows each.
    unsigned int sequence, block;
    if (!find_row_unit<FORM>(a.query_offsets, nullptr, a.sequences, a.tokens, a.heads, 4u, blockIdx.x, sequence, block)) return;
    sequence = __builtin_amdgcn_readfirstlane(sequence);
    block = __builtin_amdgcn_readfirstlane(block);
    const unsigned int local_row = block * 4 + wave;  // (query, head) of the sequence
    const SequenceSpan span = load_span<FORM>(sequence, a.query_offsets, a.page_offsets, a.last_page_lengths, nullptr, a.tokens,
                                              a.page_table, a.page_size);
    if (!span.valid) {
        if (threadIdx.x == 0) report_index_error(a.status);
        return;
    }
    if (local_row >= span.queries * a.heads) return;
    const unsigned int query = local_row / a.heads, head = local_row % a.heads;
    const size_t flat = (static_cast<size_t>(span.query_start) + query) * a.heads + head;
    const unsigned int width = a.latent_dim + a.position_dim;

    float* q_row = lds + wave * (kMaxLatent + kMaxPositional);
    const T* latent_query = static_cast<const T*>(a.latent_queries) + flat * a.latent_dim;
    const T* position_query = static_cast<const T*>(a.positional_queries) + flat * a.position_dim;
    for (unsigned int d = lane; d < width; d += 64)
        q_row[d] = d < a.latent_dim ? E::load(latent_query + d) : E::load(position_query + (d - a.latent_dim));
    __builtin_amdgcn_wave_barrier();

    // Queries are the sequence's last tokens, with the CPU path's saturating position (attention.rs:619-627).
    const long long raw = static_cast<long long>(span.keys) - static_cast<long long>(span.queries) + query;
    const unsigned int position = raw < 0 ? 0u : static_cast<unsigned int>(raw);
    unsigned int end = span.keys;
    if (a.causal && position + 1 < end) end = position + 1;

    const T* latent_cache = static_cast<const T*>(a.latent_cache);
    const T* position_cache = static_cast<const T*>(a.positional_cache);
    float acc[kMaxLatent / 64];
#pragma unroll
    for (int i = 0; i < kMaxLatent / 64; ++i) acc[i] = 0.0f;
    float largest = -INFINITY, total = 0.0f;
    for (unsigned int base = 0; base < end; base += 64) {
        const unsigned int key = base + lane;
        const bool live = key < end;
        float score = -INFINITY;
        unsigned long long slot = 0;
        bool readable = false;
        if (live) {
            const unsigned long long page = read_page<FORM>(a.pages, static_cast<size_t>(span.page_start) + key / a.page_size);
            readable = page < static_cast<unsigned long long>(a.cache_pages);
            if (!readable) report_index_error(a.status);
            slot = page * a.page_size + key % a.page_size;
            float first = 0.0f, second = 0.0f;
            if (readable) {  // a key behind a bad page id is read as zeros; the status word tells the caller
                const T* row = latent_cache + slot * a.latent_dim;
                for (unsigned int d = 0; d < a.latent_dim; ++d) first = fmaf(q_row[d], E::load(row + d), first);
                const T* tail = position_cache + slot * a.position_dim;
                for (unsigned int d = 0; d < a.position_dim; ++d) second = fmaf(q_row[a.latent_dim + d], E::load(tail + d), second);
            }
            score = (first + second) * a.scale;
        }
        const float moved = fmaxf(largest, wave_max(score));
        const float rescale = expf(largest - moved);  // exp(-inf) = 0 on the first chunk
        const float weight = live ? expf(score - moved) : 0.0f;
        total = total * rescale + wave_sum(weight);
        largest = moved;
#pragma unroll
        for (int i = 0; i < kMaxLatent / 64; ++i) acc[i] *= rescale;
        const unsigned int count = end - base < 64u ? end - base : 64u;
        const unsigned int slot_low = static_cast<unsigned int>(slot), slot_high = static_cast<unsigned int>(slot >> 32);
        for (unsigned int k = 0; k < count; ++k) {
            const float w = __shfl(weight, k, 64);
            const unsigned long long from = (static_cast<unsigned long long>(__shfl(slot_high, k, 64)) << 32) | __shfl(slot_low, k, 64);
            const bool usable = __shfl(readable ? 1 : 0, k, 64) != 0;
            if (!usable) continue;
            const T* row = latent_cache + from * a.latent_dim;
#pragma unroll
            for (int i = 0; i < kMaxLatent / 64; ++i) {
                const unsigned int d = lane + 64u * i;
                if (d < a.latent_dim) acc[i] = fmaf(w, E::load(row + d), acc[i]);
            }
        }
    }
    T* out = static_cast<T*>(a.output) + flat * a.latent_dim;
    const float inverse = total > 0.0f ? 1.0f / total : 0.0f;
#pragma unroll
    for (int i = 0; i < kMaxLatent / 64; ++i) {
        const unsigned int d = lane + 64u * i;
        if (d < a.latent_dim) E::store(out + d, acc[i] * inverse);
    }
    if (a.lse != nullptr && lane == 0) a.lse[flat] = total > 0.0f ? (largest + logf(total)) * kLog2e : -INFINITY;
}

template <uint32_t ELEMENT>
SINGE_DEVICE void latent_body(const LatentAttentionArgs& a, float* lds) {
    if (a.wide_index)
        latent_rows<ELEMENT, kCsrI64>(a, lds);
    else
        latent_rows<ELEMENT, kCsrI32>(a, lds);
}

}  // namespace latent

#define SINGE_LATENT_KERNEL(TAG, ELEMENT)                                                                            \
    extern "C" __global__ __launch_bounds__(256) void singe_paged_mla_attention_general_##TAG(LatentAttentionArgs args) { \
        __shared__ float rows[4 * (latent::kMaxLatent + latent::kMaxPositional)];                                   \
        latent::latent_body<ELEMENT>(args, rows);                                                                    \
    }

SINGE_LATENT_KERNEL(f32, kElementF32)
SINGE_LATENT_KERNEL(bf16, kElementBf16)
SINGE_LATENT_KERNEL(f16, kElementF16)
