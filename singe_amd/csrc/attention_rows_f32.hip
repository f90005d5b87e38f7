// f32 attention rows on the vector unit: one loop, four ops.  Its first form is dense decode over a slice of the
// keys, the gfx950 counterpart of fmha_decode_splitk_f32 (kernel
// singe-kernel/src/cuda/cutile/kernel/attention/local.rs:6127-6272, launch API
// singe-kernel/src/cuda/attention/fmha.rs:1074-1118), the first half of the reference's split-KV convention
// (fmha_decode_splitk_reduce_f32, fmha.rs:1155-1250); splitk_reduce.hip is the second half.
//
// query [batch, heads, dim], key / value [batch, key_len, kv_heads, dim] through element strides.  Split s of
// (batch b, head h) covers keys s * kv_len_per_split .. + kv_len_per_split (clipped to key_len) and writes
//   out[b, h, s, :] = sum_k exp(score_k - max) v_k / sum_k exp(score_k - max)      (zeros when the slice is empty)
//   lse[b, h, s]    = max + ln sum_k exp(score_k - max)                            (-1e20 when the slice is empty)
// with score_k = (q . k_k) * scale, as the reference kernel does.
//
// The reference runs one thread per output element and reads the slice twice per thread.  Here a workgroup of
// four waves owns one (batch, kv head, split) and reads its K and V rows once for every query head of the
// group: LANES lanes share a key (each holds 4 * VEC dims of it, one 16-byte load per 4 dims), so a wave folds
// 64 / LANES keys per step, the dot products finish with log2(LANES) cross-lane adds, and each set of lanes
// keeps its own running softmax state, merged across lane sets and waves once at the end.  Query heads are
// taken four at a time to bound registers (a group of more than four re-reads the slice from L2).
//
// The same loop serves the dense f32 prefill ops at these head dimensions (fmha_prefill_f32, fmha_prefill_lse_f32,
// softcapped_window_attention_f32) and the f32 forms of the two block-table ops, paged_kv_decode_attention_f32 and
// paged_kv_prefill_attention_f32 (singe-kernel/src/cpu/attention.rs:1172-1341; launch API
// singe-kernel/src/cuda/attention/paged.rs): only where the rows come from and where the result goes differ.
#include "common.hip.h"
#include "kernel_args.h"

namespace {

constexpr int kDecodeHeadsPerPass = 4;
constexpr float kEmptySliceLse = -1.0e20f;

template <bool ALIGNED>
SINGE_DEVICE float4 load4(const float* p) {
    if constexpr (ALIGNED) return *reinterpret_cast<const float4*>(p);
    return make_float4(p[0], p[1], p[2], p[3]);
}

// Running softmax state of one query head over the keys a set of lanes has seen.
template <int VEC>
struct DecodeState {
    float largest, sum;
    float4 acc[VEC];
};

template <int VEC>
SINGE_DEVICE void merge(DecodeState<VEC>& mine, float other_largest, float other_sum, const float4 (&other_acc)[VEC]) {
    const float largest = fmaxf(mine.largest, other_largest);
    const float keep = __expf(mine.largest - largest), take = __expf(other_largest - largest);
    mine.sum = mine.sum * keep + other_sum * take;
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
        mine.acc[v].x = mine.acc[v].x * keep + other_acc[v].x * take;
        mine.acc[v].y = mine.acc[v].y * keep + other_acc[v].y * take;
        mine.acc[v].z = mine.acc[v].z * keep + other_acc[v].z * take;
        mine.acc[v].w = mine.acc[v].w * keep + other_acc[v].w * take;
    }
    mine.largest = largest;
}

// The loop all three kernels of this file share.  `rows` says what the workgroup works on:
//   rows.groups, rows.begin, rows.end          query heads that share the key rows, and the keys to fold
//   rows.query(head_in_group)                  that head's dims
//   rows.key(k), rows.value(k)                 row k of the group's KV head
//   rows.shape(score)                          what the scaled score becomes (a soft cap, or itself)
//   rows.store(head_in_group, part, total)     takes the finished state; called by the LANES lanes that hold the dims
template <int LANES, int VEC, bool ALIGNED, class Rows>
SINGE_DEVICE void fold_rows(const Rows& rows, float scale, float* lds) {
    constexpr int kDim = LANES * 4 * VEC, kKeysPerWave = 64 / LANES;
    const unsigned int lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const unsigned int part = lane % LANES, set = lane / LANES;  // which dims of a key, which key of the wave's step
    const unsigned int begin = rows.begin, end = rows.end;

    for (unsigned int pass = 0; pass < rows.groups; pass += kDecodeHeadsPerPass) {
        const unsigned int live = rows.groups - pass < kDecodeHeadsPerPass ? rows.groups - pass : kDecodeHeadsPerPass;
        float4 q[kDecodeHeadsPerPass][VEC];
        DecodeState<VEC> state[kDecodeHeadsPerPass];
#pragma unroll
        for (int g = 0; g < kDecodeHeadsPerPass; ++g) {
            const float* row = rows.query(pass + (g < static_cast<int>(live) ? g : 0)) + part * (4 * VEC);
#pragma unroll
            for (int v = 0; v < VEC; ++v) {
                q[g][v] = load4<ALIGNED>(row + 4 * v);
                state[g].acc[v] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            }
            state[g].largest = kEmptySliceLse;
            state[g].sum = 0.0f;
        }
        for (unsigned int base = begin + wave * kKeysPerWave; base < end; base += 4 * kKeysPerWave) {
            const unsigned int key = base + set;
            const bool valid = key < end;
            const unsigned int row = valid ? key : end - 1;
            const float* key_row = rows.key(row) + part * (4 * VEC);
            const float* value_row = rows.value(row) + part * (4 * VEC);
            float4 k[VEC], v[VEC];
#pragma unroll
            for (int i = 0; i < VEC; ++i) {
                k[i] = load4<ALIGNED>(key_row + 4 * i);
                v[i] = load4<ALIGNED>(value_row + 4 * i);
            }
#pragma unroll
            for (int g = 0; g < kDecodeHeadsPerPass; ++g) {
                if (g >= static_cast<int>(live)) break;  // the same in every lane of the workgroup
                float score = 0.0f;
#pragma unroll
                for (int i = 0; i < VEC; ++i) {
                    score = fmaf(q[g][i].x, k[i].x, score);
                    score = fmaf(q[g][i].y, k[i].y, score);
                    score = fmaf(q[g][i].z, k[i].z, score);
                    score = fmaf(q[g][i].w, k[i].w, score);
                }
#pragma unroll
                for (int step = 1; step < LANES; step *= 2) score += wave_xor(score, step);
                score = rows.shape(score * scale);
                if (valid) {
                    DecodeState<VEC>& s = state[g];
                    const float largest = fmaxf(s.largest, score);
                    const float keep = __expf(s.largest - largest), weight = __expf(score - largest);
                    s.sum = s.sum * keep + weight;
#pragma unroll
                    for (int i = 0; i < VEC; ++i) {
                        s.acc[i].x = fmaf(weight, v[i].x, s.acc[i].x * keep);
                        s.acc[i].y = fmaf(weight, v[i].y, s.acc[i].y * keep);
                        s.acc[i].z = fmaf(weight, v[i].z, s.acc[i].z * keep);
                        s.acc[i].w = fmaf(weight, v[i].w, s.acc[i].w * keep);
                    }
                    s.largest = largest;
                }
            }
        }
        // The lane sets of a wave, then the waves through LDS: [wave][head of the pass][2 + dim].
        constexpr int kSlot = 2 + kDim;
#pragma unroll
        for (int g = 0; g < kDecodeHeadsPerPass; ++g) {
            DecodeState<VEC>& s = state[g];
#pragma unroll
            for (int step = LANES; step < 64; step *= 2) {
                const float other_largest = wave_xor(s.largest, step), other_sum = wave_xor(s.sum, step);
                float4 other_acc[VEC];
#pragma unroll
                for (int i = 0; i < VEC; ++i)
                    other_acc[i] = make_float4(wave_xor(s.acc[i].x, step), wave_xor(s.acc[i].y, step), wave_xor(s.acc[i].z, step),
                                               wave_xor(s.acc[i].w, step));
                merge(s, other_largest, other_sum, other_acc);
            }
            if (set == 0) {
                float* slot = lds + (wave * kDecodeHeadsPerPass + g) * kSlot;
                if (part == 0) {
                    slot[0] = s.largest;
                    slot[1] = s.sum;
                }
#pragma unroll
                for (int i = 0; i < VEC; ++i) {
                    float* dims = slot + 2 + part * (4 * VEC) + 4 * i;
                    dims[0] = s.acc[i].x; dims[1] = s.acc[i].y; dims[2] = s.acc[i].z; dims[3] = s.acc[i].w;
                }
            }
        }
        __syncthreads();
        // Wave g of the workgroup finishes head g of the pass: lane `part` of its first set holds the dims.
        if (wave < live && set == 0) {
            DecodeState<VEC> total;
            total.largest = kEmptySliceLse;
            total.sum = 0.0f;
#pragma unroll
            for (int i = 0; i < VEC; ++i) total.acc[i] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            for (unsigned int w = 0; w < 4; ++w) {
                const float* slot = lds + (w * kDecodeHeadsPerPass + wave) * kSlot;
                float4 other_acc[VEC];
#pragma unroll
                for (int i = 0; i < VEC; ++i) {
                    const float* dims = slot + 2 + part * (4 * VEC) + 4 * i;
                    other_acc[i] = make_float4(dims[0], dims[1], dims[2], dims[3]);
                }
                merge(total, slot[0], slot[1], other_acc);
            }
            rows.store(pass + wave, part, total);
        }
        __syncthreads();
    }
}

// out[0 .. 4 VEC) = acc / sum (zeros for a row that saw no key), and what the row's LSE is.
template <int VEC>
SINGE_DEVICE float finish(float* out, const DecodeState<VEC>& total) {
    const bool has_keys = total.sum > 0.0f;
    const float inverse = has_keys ? 1.0f / total.sum : 0.0f;
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
        out[4 * i + 0] = total.acc[i].x * inverse;
        out[4 * i + 1] = total.acc[i].y * inverse;
        out[4 * i + 2] = total.acc[i].z * inverse;
        out[4 * i + 3] = total.acc[i].w * inverse;
    }
    return has_keys ? total.largest + __logf(total.sum) : kEmptySliceLse;
}

// fmha_decode_splitk_f32: workgroup = (batch, kv head, split) of dense [batch, key_len, kv_heads, dim] keys.
template <int VEC>
struct DenseSplitRows {
    const FmhaDecodeSplitKArgs& a;
    unsigned int groups, begin, end, batch, kv_head, split;
    SINGE_DEVICE explicit DenseSplitRows(const FmhaDecodeSplitKArgs& args) : a(args) {
        groups = a.heads / a.kv_heads;
        unsigned int unit = blockIdx.x;
        split = unit % a.splits;
        unit /= a.splits;
        kv_head = unit % a.kv_heads;
        batch = unit / a.kv_heads;
        const unsigned long long first = static_cast<unsigned long long>(split) * a.kv_len_per_split;
        begin = first < a.key_len ? static_cast<unsigned int>(first) : a.key_len;
        end = first + a.kv_len_per_split < a.key_len ? static_cast<unsigned int>(first + a.kv_len_per_split) : a.key_len;
    }
    SINGE_DEVICE const float* query(unsigned int g) const {
        return a.query + batch * a.query_batch_stride + (kv_head * groups + g) * a.query_head_stride;
    }
    SINGE_DEVICE const float* key(unsigned int k) const {
        return a.key + batch * a.key_batch_stride + kv_head * a.key_head_stride + k * a.key_sequence_stride;
    }
    SINGE_DEVICE const float* value(unsigned int k) const {
        return a.value + batch * a.value_batch_stride + kv_head * a.value_head_stride + k * a.value_sequence_stride;
    }
    SINGE_DEVICE float shape(float score) const { return score; }
    SINGE_DEVICE void store(unsigned int g, unsigned int part, const DecodeState<VEC>& total) const {
        const unsigned int head = kv_head * groups + g;
        const float lse = finish(a.out + batch * a.output_batch_stride + head * a.output_head_stride + split * a.output_split_stride +
                                     part * (4 * VEC), total);
        if (part == 0) a.lse[batch * a.lse_batch_stride + head * a.lse_head_stride + split] = lse;
    }
};

// fmha_prefill_f32 / fmha_prefill_lse_f32 / softcapped_window_attention_f32 (cpu/attention.rs:1758-1925):
// workgroup = (batch, query, kv head) of dense tensors addressed through element strides.  Top-left causal
// hides key > query; a window hides keys more than window_size away on either side (cpu/attention.rs:1860-1869).
template <int VEC>
struct DensePrefillRows {
    const PrefillF32Args& a;
    unsigned int groups, begin, end, batch, query_index, kv_head;
    SINGE_DEVICE explicit DensePrefillRows(const PrefillF32Args& args) : a(args) {
        groups = a.heads / a.kv_heads;
        unsigned int unit = blockIdx.x;
        kv_head = unit % a.kv_heads;
        unit /= a.kv_heads;
        query_index = unit % a.query_len;
        batch = unit / a.query_len;
        begin = 0;
        end = a.key_len;
        if (a.causal && query_index + 1 < end) end = query_index + 1;
        if (a.window_size > 0) {
            if (query_index > a.window_size) begin = query_index - a.window_size;
            const unsigned long long last = static_cast<unsigned long long>(query_index) + a.window_size + 1;
            if (last < end) end = static_cast<unsigned int>(last);
        }
        if (begin > end) begin = end;
    }
    SINGE_DEVICE const float* query(unsigned int g) const {
        return a.query + batch * a.query_batch_stride + static_cast<size_t>(query_index) * a.query_sequence_stride +
               (kv_head * groups + g) * a.query_head_stride;
    }
    SINGE_DEVICE const float* key(unsigned int k) const {
        return a.key + batch * a.key_batch_stride + kv_head * a.key_head_stride + static_cast<size_t>(k) * a.key_sequence_stride;
    }
    SINGE_DEVICE const float* value(unsigned int k) const {
        return a.value + batch * a.value_batch_stride + kv_head * a.value_head_stride + static_cast<size_t>(k) * a.value_sequence_stride;
    }
    SINGE_DEVICE float shape(float score) const { return a.has_soft_cap ? tanhf(score / a.soft_cap) * a.soft_cap : score; }
    SINGE_DEVICE void store(unsigned int g, unsigned int part, const DecodeState<VEC>& total) const {
        const unsigned int head = kv_head * groups + g;
        const float lse = finish(a.out + batch * a.output_batch_stride + static_cast<size_t>(query_index) * a.output_sequence_stride +
                                     head * a.output_head_stride + part * (4 * VEC), total);
        // A row that sees no key (a window wholly past the keys) stays zero; its LSE is ln 0.
        if (a.lse != nullptr && part == 0)
            a.lse[(static_cast<size_t>(batch) * a.heads + head) * a.query_len + query_index] = total.sum > 0.0f ? lse : -INFINITY;
    }
};

// The two paged forms read rows [block, slot, kv head, dim] through a block table
// (block = table[sequence * stride + key / block_size], slot = key % block_size: cpu/attention.rs:1196-1206).
// A table entry past the cache is clamped to its last block: the reference does not check it, and a wild
// entry must not become a wild address here; nor must a length the table has no entries for.
struct PagedCaches {
    const PagedRowsF32Args& a;
    unsigned int sequence, kv_head, dim;
    // Keys one row of the table can name; a sequence length beyond it is cut there (the host checks that the
    // product fits 32 bits).
    SINGE_DEVICE unsigned int capacity() const { return a.block_table_batch_stride * a.block_size; }
    SINGE_DEVICE size_t row(unsigned int k) const {
        unsigned int block = a.block_table[static_cast<size_t>(sequence) * a.block_table_batch_stride + k / a.block_size];
        block = block < a.physical_blocks ? block : a.physical_blocks - 1;
        return ((static_cast<size_t>(block) * a.block_size + k % a.block_size) * a.kv_heads + kv_head) * dim;
    }
};

// paged_kv_decode_attention_f32 (cpu/attention.rs:1172-1246), split over the keys: workgroup = (sequence, kv head,
// split); split s of a sequence of L keys covers ceil(L / splits) of them.  Partials in the layout
// splitk_reduce_f32 takes: out [batch, heads, splits, dim], lse [batch, heads, splits].
template <int VEC>
struct PagedDecodeRows {
    const PagedRowsF32Args& a;
    PagedCaches caches;
    unsigned int groups, begin, end, split;
    SINGE_DEVICE PagedDecodeRows(const PagedRowsF32Args& args, unsigned int dim) : a(args), caches{args, 0, 0, dim} {
        groups = a.heads / a.kv_heads;
        unsigned int unit = blockIdx.x;
        split = unit % a.splits;
        unit /= a.splits;
        caches.kv_head = unit % a.kv_heads;
        caches.sequence = unit / a.kv_heads;
        const int length = a.seq_lens_kv[caches.sequence];
        unsigned int keys = length > 0 ? static_cast<unsigned int>(length) : 0u;
        keys = keys < caches.capacity() ? keys : caches.capacity();
        const unsigned int per = (keys + a.splits - 1) / a.splits;
        begin = split * per < keys ? split * per : keys;
        end = begin + per < keys ? begin + per : keys;
    }
    SINGE_DEVICE const float* query(unsigned int g) const {
        return a.query + (static_cast<size_t>(caches.sequence) * a.heads + caches.kv_head * groups + g) * caches.dim;
    }
    SINGE_DEVICE const float* key(unsigned int k) const { return a.key_cache + caches.row(k); }
    SINGE_DEVICE const float* value(unsigned int k) const { return a.value_cache + caches.row(k); }
    SINGE_DEVICE float shape(float score) const { return score; }
    SINGE_DEVICE void store(unsigned int g, unsigned int part, const DecodeState<VEC>& total) const {
        const size_t row = (static_cast<size_t>(caches.sequence) * a.heads + caches.kv_head * groups + g) * a.splits + split;
        const float lse = finish(a.out + row * caches.dim + part * (4 * VEC), total);
        if (part == 0) a.lse[row] = lse;
    }
};

// paged_kv_prefill_attention_f32 (cpu/attention.rs:1248-1341): workgroup = (token, kv head).  Token t belongs to
// the last sequence b with offsets[b] <= t < offsets[b] + len_q[b] (the reference walks the sequences in order,
// so a later one overwrites); query i of a sequence sees keys 0 .. min(i + 1, len_kv) under the causal mask, all
// len_kv without.  A token of no sequence gets zeros and an LSE of 0, a row without keys zeros and -1e20.
template <int VEC>
struct PagedPrefillRows {
    const PagedRowsF32Args& a;
    PagedCaches caches;
    unsigned int groups, begin, end, token;
    bool owned;
    SINGE_DEVICE PagedPrefillRows(const PagedRowsF32Args& args, unsigned int dim) : a(args), caches{args, 0, 0, dim} {
        groups = a.heads / a.kv_heads;
        token = blockIdx.x / a.kv_heads;
        caches.kv_head = blockIdx.x % a.kv_heads;
        owned = false;
        begin = end = 0;
        for (unsigned int b = 0; b < a.batch; ++b) {
            const int offset = a.seq_offsets[b], queries = a.seq_lens_q[b];
            if (offset < 0 || queries <= 0 || static_cast<int>(token) < offset || static_cast<long long>(token) >= static_cast<long long>(offset) + queries) continue;
            owned = true;
            caches.sequence = b;
            const int length = a.seq_lens_kv[b];
            unsigned int keys = length > 0 ? static_cast<unsigned int>(length) : 0u;
            keys = keys < caches.capacity() ? keys : caches.capacity();
            const unsigned int index = token - static_cast<unsigned int>(offset);
            end = a.causal && index + 1 < keys ? index + 1 : keys;
        }
    }
    SINGE_DEVICE const float* query(unsigned int g) const {
        return a.query + (static_cast<size_t>(token) * a.heads + caches.kv_head * groups + g) * caches.dim;
    }
    SINGE_DEVICE const float* key(unsigned int k) const { return a.key_cache + caches.row(k); }
    SINGE_DEVICE const float* value(unsigned int k) const { return a.value_cache + caches.row(k); }
    SINGE_DEVICE float shape(float score) const { return score; }
    SINGE_DEVICE void store(unsigned int g, unsigned int part, const DecodeState<VEC>& total) const {
        const size_t row = static_cast<size_t>(token) * a.heads + caches.kv_head * groups + g;
        const float lse = finish(a.out + row * caches.dim + part * (4 * VEC), total);
        if (part == 0) a.lse[row] = owned ? lse : 0.0f;
    }
};

}  // namespace

#define SINGE_F32_ROW_KERNELS(DIM, LANES, VEC)                                                                               \
    extern "C" __global__ __launch_bounds__(256) void singe_fmha_decode_splitk_f32_d##DIM(FmhaDecodeSplitKArgs args) {       \
        __shared__ float lds[4 * kDecodeHeadsPerPass * (2 + DIM)];                                                           \
        const DenseSplitRows<VEC> rows(args);                                                                                \
        if (args.aligned) fold_rows<LANES, VEC, true>(rows, args.scale, lds);                                                \
        else fold_rows<LANES, VEC, false>(rows, args.scale, lds);                                                            \
    }                                                                                                                        \
    extern "C" __global__ __launch_bounds__(256) void singe_fmha_prefill_rows_f32_d##DIM(PrefillF32Args args) {              \
        __shared__ float lds[4 * kDecodeHeadsPerPass * (2 + DIM)];                                                           \
        const DensePrefillRows<VEC> rows(args);                                                                              \
        if (args.aligned) fold_rows<LANES, VEC, true>(rows, args.scale, lds);                                                \
        else fold_rows<LANES, VEC, false>(rows, args.scale, lds);                                                            \
    }                                                                                                                        \
    extern "C" __global__ __launch_bounds__(256) void singe_paged_kv_decode_splitk_f32_d##DIM(PagedRowsF32Args args) {       \
        __shared__ float lds[4 * kDecodeHeadsPerPass * (2 + DIM)];                                                           \
        const PagedDecodeRows<VEC> rows(args, DIM);                                                                          \
        if (args.aligned) fold_rows<LANES, VEC, true>(rows, args.scale, lds);                                                \
        else fold_rows<LANES, VEC, false>(rows, args.scale, lds);                                                            \
    }                                                                                                                        \
    extern "C" __global__ __launch_bounds__(256) void singe_paged_kv_prefill_f32_d##DIM(PagedRowsF32Args args) {             \
        __shared__ float lds[4 * kDecodeHeadsPerPass * (2 + DIM)];                                                           \
        const PagedPrefillRows<VEC> rows(args, DIM);                                                                         \
        if (args.aligned) fold_rows<LANES, VEC, true>(rows, args.scale, lds);                                                \
        else fold_rows<LANES, VEC, false>(rows, args.scale, lds);                                                            \
    }

SINGE_F32_ROW_KERNELS(4, 1, 1)
SINGE_F32_ROW_KERNELS(8, 2, 1)
SINGE_F32_ROW_KERNELS(16, 4, 1)
SINGE_F32_ROW_KERNELS(32, 8, 1)
SINGE_F32_ROW_KERNELS(64, 16, 1)
SINGE_F32_ROW_KERNELS(128, 16, 2)
SINGE_F32_ROW_KERNELS(256, 16, 4)
