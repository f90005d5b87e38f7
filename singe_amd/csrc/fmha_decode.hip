// Dense f32 decode attention over a slice of the keys: the gfx950 counterpart of fmha_decode_splitk_f32
// (kernel singe-kernel/src/cuda/cutile/kernel/attention/local.rs:6127-6272, launch API
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

template <int LANES, int VEC, bool ALIGNED>
SINGE_DEVICE void fmha_decode_splitk_body(const FmhaDecodeSplitKArgs& a, float* lds) {
    constexpr int kDim = LANES * 4 * VEC, kKeysPerWave = 64 / LANES;
    const unsigned int lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const unsigned int part = lane % LANES, set = lane / LANES;  // which dims of a key, which key of the wave's step
    const unsigned int groups = a.heads / a.kv_heads;
    unsigned int unit = blockIdx.x;
    const unsigned int split = unit % a.splits;
    unit /= a.splits;
    const unsigned int kv_head = unit % a.kv_heads, batch = unit / a.kv_heads;
    const unsigned long long first = static_cast<unsigned long long>(split) * a.kv_len_per_split;
    const unsigned int begin = first < a.key_len ? static_cast<unsigned int>(first) : a.key_len;
    const unsigned int end = first + a.kv_len_per_split < a.key_len ? static_cast<unsigned int>(first + a.kv_len_per_split) : a.key_len;
    const float* keys = a.key + batch * a.key_batch_stride + kv_head * a.key_head_stride + part * (4 * VEC);
    const float* values = a.value + batch * a.value_batch_stride + kv_head * a.value_head_stride + part * (4 * VEC);

    for (unsigned int pass = 0; pass < groups; pass += kDecodeHeadsPerPass) {
        const unsigned int live = groups - pass < kDecodeHeadsPerPass ? groups - pass : kDecodeHeadsPerPass;
        float4 q[kDecodeHeadsPerPass][VEC];
        DecodeState<VEC> state[kDecodeHeadsPerPass];
#pragma unroll
        for (int g = 0; g < kDecodeHeadsPerPass; ++g) {
            const unsigned int head = kv_head * groups + pass + (g < static_cast<int>(live) ? g : 0);
            const float* row = a.query + batch * a.query_batch_stride + head * a.query_head_stride + part * (4 * VEC);
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
            float4 k[VEC], v[VEC];
#pragma unroll
            for (int i = 0; i < VEC; ++i) {
                k[i] = load4<ALIGNED>(keys + row * a.key_sequence_stride + 4 * i);
                v[i] = load4<ALIGNED>(values + row * a.value_sequence_stride + 4 * i);
            }
#pragma unroll
            for (int g = 0; g < kDecodeHeadsPerPass; ++g) {
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
                score *= a.scale;
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
            const unsigned int g = wave;
            DecodeState<VEC> total;
            total.largest = kEmptySliceLse;
            total.sum = 0.0f;
#pragma unroll
            for (int i = 0; i < VEC; ++i) total.acc[i] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            for (unsigned int w = 0; w < 4; ++w) {
                const float* slot = lds + (w * kDecodeHeadsPerPass + g) * kSlot;
                float4 other_acc[VEC];
#pragma unroll
                for (int i = 0; i < VEC; ++i) {
                    const float* dims = slot + 2 + part * (4 * VEC) + 4 * i;
                    other_acc[i] = make_float4(dims[0], dims[1], dims[2], dims[3]);
                }
                merge(total, slot[0], slot[1], other_acc);
            }
            const unsigned int head = kv_head * groups + pass + g;
            const bool has_keys = total.sum > 0.0f;
            const float inverse = has_keys ? 1.0f / total.sum : 0.0f;
            float* out = a.out + batch * a.output_batch_stride + head * a.output_head_stride + split * a.output_split_stride + part * (4 * VEC);
#pragma unroll
            for (int i = 0; i < VEC; ++i) {
                out[4 * i + 0] = total.acc[i].x * inverse;
                out[4 * i + 1] = total.acc[i].y * inverse;
                out[4 * i + 2] = total.acc[i].z * inverse;
                out[4 * i + 3] = total.acc[i].w * inverse;
            }
            if (part == 0)
                a.lse[batch * a.lse_batch_stride + head * a.lse_head_stride + split] =
                    has_keys ? total.largest + __logf(total.sum) : kEmptySliceLse;
        }
        __syncthreads();
    }
}

}  // namespace

#define SINGE_FMHA_DECODE_SPLITK_KERNEL(DIM, LANES, VEC)                                                                   \
    extern "C" __global__ __launch_bounds__(256) void singe_fmha_decode_splitk_f32_d##DIM(FmhaDecodeSplitKArgs args) {     \
        __shared__ float lds[4 * kDecodeHeadsPerPass * (2 + DIM)];                                                         \
        if (args.aligned) fmha_decode_splitk_body<LANES, VEC, true>(args, lds);                                            \
        else fmha_decode_splitk_body<LANES, VEC, false>(args, lds);                                                        \
    }

SINGE_FMHA_DECODE_SPLITK_KERNEL(4, 1, 1)
SINGE_FMHA_DECODE_SPLITK_KERNEL(8, 2, 1)
SINGE_FMHA_DECODE_SPLITK_KERNEL(16, 4, 1)
SINGE_FMHA_DECODE_SPLITK_KERNEL(32, 8, 1)
SINGE_FMHA_DECODE_SPLITK_KERNEL(64, 16, 1)
SINGE_FMHA_DECODE_SPLITK_KERNEL(128, 16, 2)
SINGE_FMHA_DECODE_SPLITK_KERNEL(256, 16, 4)
