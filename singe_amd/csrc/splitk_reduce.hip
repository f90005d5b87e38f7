// Combines per-split attention partials: the gfx950 counterpart of splitk_reduce_f32
// (singe-kernel/src/cpu/attention.rs:2157-2193; launch API singe-kernel/src/cuda/attention/fmha.rs:1038-1067).
//
// attn [batch, heads, splits, dim] and lse [batch, heads, splits] (natural log) with element strides;
// out[b, h, :] = sum_s exp(lse_s - max) * attn_s / sum_s exp(lse_s - max), both sums in increasing split
// order like the CPU loop.  One wave per (batch, head); a lane owns dims lane, lane + 64, ...
#include "common.hip.h"
#include "kernel_args.h"

extern "C" __global__ __launch_bounds__(256) void singe_splitk_reduce_f32(SplitKReduceArgs a) {
    const unsigned int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const unsigned long long unit = static_cast<unsigned long long>(blockIdx.x) * 4 + wave;
    if (unit >= static_cast<unsigned long long>(a.batch) * a.heads) return;
    const unsigned int batch = static_cast<unsigned int>(unit / a.heads), head = static_cast<unsigned int>(unit % a.heads);
    const float* lse = a.lse + batch * a.lse_batch_stride + head * a.lse_head_stride;
    const float* attn = a.attn + batch * a.attn_batch_stride + head * a.attn_head_stride;
    float* out = a.out + batch * a.output_batch_stride + head * a.output_head_stride;

    float largest = -INFINITY;
    for (unsigned int split = 0; split < a.splits; ++split) largest = fmaxf(largest, lse[split]);
    float denom = 0.0f;
    for (unsigned int split = 0; split < a.splits; ++split) denom += expf(lse[split] - largest);
    for (unsigned int dim = lane; dim < a.head_dim; dim += 64) {
        float sum = 0.0f;
        for (unsigned int split = 0; split < a.splits; ++split)
            sum = fmaf(expf(lse[split] - largest), attn[split * a.attn_split_stride + dim], sum);
        out[dim] = sum / denom;
    }
}
