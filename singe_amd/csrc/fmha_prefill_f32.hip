// Dense attention in f32 for any head_dim up to 256 and any element strides: the GPU counterpart of
// singe-kernel/src/cpu/attention.rs:1758-1833 (fmha_prefill_lse_f32) and :1835-1925
// (softcapped_window_attention_f32), replacing the cuTile fmha_prefill_f32 /
// softcapped_window_attention_f32 kernels (singe-kernel/src/cuda/attention/fmha.rs:48-290).
//
// This is the accuracy anchor (f32 in, f32 arithmetic, results within 1e-4 of the CPU path), not a
// throughput kernel: one wave64 per query row.  Lanes take keys 64 apart; a lane's score is the same
// left-to-right fma chain over the head dimension as the CPU path, its softmax is online in natural
// base with expf, and the 64 per-lane partial rows are merged once at the end.
#include "common.hip.h"
#include "kernel_args.h"

namespace {

template <int DMAX>
SINGE_DEVICE void fmha_prefill_f32_body(const PrefillF32Args& a, float* lds) {
    const unsigned int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const unsigned long long row = static_cast<unsigned long long>(blockIdx.x) * 4 + wave;
    const unsigned long long rows = static_cast<unsigned long long>(a.batch) * a.heads * a.query_len;
    if (row >= rows) return;
    const unsigned int query = static_cast<unsigned int>(row % a.query_len);
    const unsigned int head = static_cast<unsigned int>((row / a.query_len) % a.heads);
    const unsigned int batch = static_cast<unsigned int>(row / (static_cast<unsigned long long>(a.query_len) * a.heads));
    const unsigned int kv_head = head / (a.heads / a.kv_heads);
    const unsigned int dim = a.head_dim;

    const float* q = a.query + batch * a.query_batch_stride + static_cast<size_t>(query) * a.query_sequence_stride + head * a.query_head_stride;
    const float* k = a.key + batch * a.key_batch_stride + kv_head * a.key_head_stride;
    const float* v = a.value + batch * a.value_batch_stride + kv_head * a.value_head_stride;

    // The query row, shared by the lanes through LDS (every lane reads the same address: a broadcast).
    float* q_row = lds + wave * DMAX;
    for (unsigned int d = lane; d < dim; d += 64) q_row[d] = q[d];
    __builtin_amdgcn_wave_barrier();

    // Keys the row may see: top-left causal hides key > query; a window hides keys more than
    // window_size away on either side (cpu/attention.rs:1860-1869).
    unsigned int first = 0, end = a.key_len;
    if (a.causal && query + 1 < end) end = query + 1;
    if (a.window_size > 0) {
        if (query > a.window_size) first = query - a.window_size;
        const unsigned long long last = static_cast<unsigned long long>(query) + a.window_size + 1;
        if (last < end) end = static_cast<unsigned int>(last);
    }

    float acc[DMAX];
#pragma unroll
    for (int d = 0; d < DMAX; ++d) acc[d] = 0.0f;
    float largest = -INFINITY, total = 0.0f;
    for (unsigned int key = first + lane; key < end; key += 64) {
        const float* k_row = k + static_cast<size_t>(key) * a.key_sequence_stride;
        float score = 0.0f;
        for (unsigned int d = 0; d < dim; ++d) score = fmaf(q_row[d], k_row[d], score);
        score *= a.scale;
        if (a.has_soft_cap) score = tanhf(score / a.soft_cap) * a.soft_cap;
        const float moved = fmaxf(largest, score);
        const float rescale = expf(largest - moved);  // exp(-inf) = 0 on the first key
        const float weight = expf(score - moved);
        total = total * rescale + weight;
        largest = moved;
        const float* v_row = v + static_cast<size_t>(key) * a.value_sequence_stride;
#pragma unroll
        for (int d = 0; d < DMAX; ++d)
            if (static_cast<unsigned int>(d) < dim) acc[d] = fmaf(weight, v_row[d], acc[d] * rescale);
    }

    // Merge the 64 lanes: common maximum, then weighted sums.
    float row_max = largest;
#pragma unroll
    for (int step = 32; step >= 1; step >>= 1) row_max = fmaxf(row_max, __shfl_xor(row_max, step, 64));
    const float mine = largest == -INFINITY ? 0.0f : expf(largest - row_max);
    float row_sum = total * mine;
#pragma unroll
    for (int step = 32; step >= 1; step >>= 1) row_sum += __shfl_xor(row_sum, step, 64);
    const float inverse = row_sum > 0.0f ? 1.0f / row_sum : 0.0f;

    float* out = a.out + batch * a.output_batch_stride + static_cast<size_t>(query) * a.output_sequence_stride + head * a.output_head_stride;
#pragma unroll
    for (int d = 0; d < DMAX; ++d) {
        if (static_cast<unsigned int>(d) < dim) {
            float value = acc[d] * mine;
#pragma unroll
            for (int step = 32; step >= 1; step >>= 1) value += __shfl_xor(value, step, 64);
            // A row that sees no key stays zero (cpu/attention.rs:1892-1894).
            if (lane == (d & 63)) out[d] = value * inverse;
        }
    }
    if (a.lse != nullptr && lane == 0)
        a.lse[(static_cast<size_t>(batch) * a.heads + head) * a.query_len + query] = row_max + logf(row_sum);
}

}  // namespace

#define SINGE_PREFILL_F32_KERNEL(DMAX)                                                                \
    extern "C" __global__ __launch_bounds__(256) void singe_fmha_prefill_f32_d##DMAX(PrefillF32Args args) { \
        __shared__ float rows[4 * DMAX];                                                              \
        fmha_prefill_f32_body<DMAX>(args, rows);                                                      \
    }

SINGE_PREFILL_F32_KERNEL(32)
SINGE_PREFILL_F32_KERNEL(64)
SINGE_PREFILL_F32_KERNEL(128)
SINGE_PREFILL_F32_KERNEL(256)
