// Paged-attention decode over a block-table KV cache, one query token per sequence
// (the GPU counterpart of singe-kernel/src/cpu/attention.rs:1172-1246, replacing the cuTile kernels
// of singe-kernel/src/cuda/cutile/kernel/attention/local.rs:9349-...).
//
// Layouts (fixed by the reference API): query/out [batch, heads, dim]; caches
// [blocks, block_size, kv_heads, dim]; block_table [batch, stride] u32; actual_seq_lens [batch] i32.
//
// Decode reads every KV byte once and does ~4 flop per byte, so it is bound by HBM bandwidth.  The
// work unit is one wave64 over (sequence, kv head, chunk of keys): the query heads that share the kv
// head ride along as MFMA columns, so a key row is fetched once for the whole group.
//
//   scores   S^T[token, head] = K[token, :] . Q[head, :] on v_mfma_f32_16x16x32_bf16 (fp32 accum);
//            the group's heads are repeated across the 16 MFMA columns so every lane ends up with the
//            scores of "its" head for four consecutive tokens,
//   softmax  online, base two, per lane group of 16 (four independent streams per wave, merged once
//            at the end), so the loop needs no cross-lane reduction,
//   values   V rows are loaded as whole 256-byte rows (16 lanes x 16 B) and folded on the VALU with
//            the probabilities broadcast inside quads (DPP) or groups of 8/16 (ds_swizzle).
//
// Each chunk writes a normalised partial row and its natural-log LSE into caller-supplied scratch laid
// out [batch, heads, splits, dim] / [batch, heads, splits], the layout of the reference's split-KV
// scratch (singe-kernel/src/cuda/attention/mod.rs:2456-2539); singe_paged_decode_combine folds them
// as splitk_reduce_f32 does (cpu/attention.rs:2157-2193).
#include "common.hip.h"
#include "kernel_args.h"

namespace {

constexpr int kDim = 128;
constexpr int kTile = 32;  // keys folded per loop step: two 16-key MFMA tiles

struct KeyTile {
    uint4 k[2][4];  // [16-key tile][32-wide dim chunk]: lane (g, t) holds key t, dims 32g + 8c .. +8
    uint4 v[2][4];  // [16-key tile][row]: lane (g, t) holds key 4g + row, dims 8t .. 8t + 8
    unsigned int live;  // bit (tile * 4 + row): key tile*16 + 4g + row takes part in the softmax
};

// Element offset of (block, token-in-block, kv_head, 0) in a [blocks, block_size, kv_heads, 128] cache.
SINGE_DEVICE size_t cache_row(unsigned int block, unsigned int token, unsigned int block_size,
                              unsigned int kv_heads, unsigned int kv_head) {
    return ((static_cast<size_t>(block) * block_size + token) * kv_heads + kv_head) * kDim;
}

// Splits a key index into (table entry, slot in block).  Power-of-two block sizes take the shift.
SINGE_DEVICE void split_key(const DecodeArgs& a, unsigned int key, unsigned int& entry, unsigned int& slot) {
    if (a.block_shift >= 0) {
        entry = key >> a.block_shift;
        slot = key & (a.block_size - 1);
    } else {
        entry = key / a.block_size;
        slot = key - entry * a.block_size;
    }
}

// Loads the 32 keys from `first` (a multiple of 32) of a chunk that ends at `end` > 0.  Keys at or past
// `end`, and keys whose table entry is not a cache block, read an in-range row instead and are marked
// dead, so nothing is read out of bounds and no dead row can carry a NaN into the weighted sum.
template <bool ALIGNED16>
SINGE_DEVICE void load_tile(KeyTile& tile, const DecodeArgs& a, const unsigned int* table_row,
                            unsigned int first, unsigned int end, unsigned int kv_head, unsigned int g,
                            unsigned int t) {
    tile.live = 0;
#pragma unroll
    for (int half = 0; half < 2; ++half) {
        const unsigned int base = first + half * 16;
        if constexpr (ALIGNED16) {
            // block_size is a multiple of 16, so the 16 keys from `base` share one table entry; a
            // half tile wholly past the end re-reads the 16-key span that holds the last key.
            const unsigned int span = base < end ? base : ((end - 1) & ~15u);
            unsigned int entry, slot0, last_entry, last_slot;
            split_key(a, span, entry, slot0);
            split_key(a, end - 1, last_entry, last_slot);
            unsigned int block = table_row[entry];
            const bool known = block < a.physical_blocks;
            block = known ? block : 0;
            {
                const bool inside = base + t < end;
                const uint16_t* kp =
                    a.key_cache + cache_row(block, inside ? slot0 + t : last_slot, a.block_size, a.kv_heads, kv_head) + 32 * g;
#pragma unroll
                for (int c = 0; c < 4; ++c) tile.k[half][c] = *reinterpret_cast<const uint4*>(kp + 8 * c);
            }
#pragma unroll
            for (int row = 0; row < 4; ++row) {
                const bool inside = base + 4 * g + row < end;
                const uint16_t* vp =
                    a.value_cache + cache_row(block, inside ? slot0 + 4 * g + row : last_slot, a.block_size, a.kv_heads, kv_head) + 8 * t;
                tile.v[half][row] = *reinterpret_cast<const uint4*>(vp);
                if (inside && known) tile.live |= 1u << (half * 4 + row);
            }
        } else {
            // Any block size: every lane looks up the table entry of its own key.
            {
                const unsigned int key = base + t < end ? base + t : end - 1;
                unsigned int entry, slot;
                split_key(a, key, entry, slot);
                unsigned int block = table_row[entry];
                block = block < a.physical_blocks ? block : 0;
                const uint16_t* kp = a.key_cache + cache_row(block, slot, a.block_size, a.kv_heads, kv_head) + 32 * g;
#pragma unroll
                for (int c = 0; c < 4; ++c) tile.k[half][c] = *reinterpret_cast<const uint4*>(kp + 8 * c);
            }
#pragma unroll
            for (int row = 0; row < 4; ++row) {
                const unsigned int wanted = base + 4 * g + row;
                const bool inside = wanted < end;
                unsigned int entry, slot;
                split_key(a, inside ? wanted : end - 1, entry, slot);
                unsigned int block = table_row[entry];
                const bool known = block < a.physical_blocks;
                block = known ? block : 0;
                const uint16_t* vp = a.value_cache + cache_row(block, slot, a.block_size, a.kv_heads, kv_head) + 8 * t;
                tile.v[half][row] = *reinterpret_cast<const uint4*>(vp);
                if (inside && known) tile.live |= 1u << (half * 4 + row);
            }
        }
    }
}

// GROUPS = query heads per kv head rounded up to a power of two (1, 2, 4, 8, 16).
template <int GROUPS, bool ALIGNED16>
SINGE_DEVICE void paged_decode_body(const DecodeArgs& a) {
    const unsigned int lane = threadIdx.x;
    const unsigned int g = lane >> 4, t = lane & 15;
    const unsigned int split = blockIdx.x, kv_head = blockIdx.y, batch = blockIdx.z;
    const unsigned int group = a.heads / a.kv_heads;

    const unsigned int reach = a.block_table_batch_stride * a.block_size;
    int raw_len = a.actual_seq_lens[batch];
    const unsigned int seq_len = raw_len < 0 ? 0u : (static_cast<unsigned int>(raw_len) < reach ? static_cast<unsigned int>(raw_len) : reach);
    const unsigned int first = split * a.keys_per_split;
    if (first >= seq_len) return;
    const unsigned int end = seq_len < first + a.keys_per_split ? seq_len : first + a.keys_per_split;
    const unsigned int* table_row = a.block_table + static_cast<size_t>(batch) * a.block_table_batch_stride;

    // Query rows as the MFMA B operand: column j of the 16 carries head j % GROUPS.
    const unsigned int my_head = t % GROUPS;
    bf16x8_t q[4];
    {
        const bool real = my_head < group;
        const uint16_t* qp = a.query + (static_cast<size_t>(batch) * a.heads + kv_head * group + (real ? my_head : 0)) * kDim + 32 * g;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            uint4 bits = *reinterpret_cast<const uint4*>(qp + 8 * c);
            if (!real) bits = make_uint4(0, 0, 0, 0);
            q[c] = __builtin_bit_cast(bf16x8_t, bits);
        }
    }

    float acc[GROUPS][8];
#pragma unroll
    for (int h = 0; h < GROUPS; ++h)
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[h][e] = 0.0f;
    float running_max = -INFINITY;  // of this lane's head, over this lane group's keys, in log2 units
    float running_sum = 0.0f;

    KeyTile current, next;
    load_tile<ALIGNED16>(current, a, table_row, first, end, kv_head, g, t);
    for (unsigned int at = first; at < end; at += kTile) {
        const bool more = at + kTile < end;
        if (more) load_tile<ALIGNED16>(next, a, table_row, at + kTile, end, kv_head, g, t);

        f32x4_t s0 = {0.0f, 0.0f, 0.0f, 0.0f}, s1 = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, current.k[0][c]), q[c], s0, 0, 0, 0);
            s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, current.k[1][c]), q[c], s1, 0, 0, 0);
        }
        float p[8];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            p[r] = (current.live >> r) & 1u ? s0[r] * a.scale_log2e : -INFINITY;
            p[4 + r] = (current.live >> (4 + r)) & 1u ? s1[r] * a.scale_log2e : -INFINITY;
        }
        float largest = running_max;
#pragma unroll
        for (int r = 0; r < 8; ++r) largest = fmaxf(largest, p[r]);
        const float base = largest == -INFINITY ? 0.0f : largest;
        const float rescale = fast_exp2(running_max - base);
        float total = 0.0f;
#pragma unroll
        for (int r = 0; r < 8; ++r) {
            p[r] = fast_exp2(p[r] - base);
            total += p[r];
        }
        running_sum = running_sum * rescale + total;
        const bool moved = largest > running_max;
        running_max = largest;
        const bool any_moved = __any(moved);

        static_for<GROUPS>([&](auto head) {
            constexpr int h = decltype(head)::value;
            if (any_moved) {
                const float factor = group_broadcast<GROUPS, h>(rescale);
#pragma unroll
                for (int e = 0; e < 8; ++e) acc[h][e] *= factor;
            }
#pragma unroll
            for (int half = 0; half < 2; ++half)
#pragma unroll
                for (int row = 0; row < 4; ++row) {
                    const float weight = group_broadcast<GROUPS, h>(p[half * 4 + row]);
                    const uint4 bits = current.v[half][row];
                    acc[h][0] = fmaf(weight, bf16_lo(bits.x), acc[h][0]);
                    acc[h][1] = fmaf(weight, bf16_hi(bits.x), acc[h][1]);
                    acc[h][2] = fmaf(weight, bf16_lo(bits.y), acc[h][2]);
                    acc[h][3] = fmaf(weight, bf16_hi(bits.y), acc[h][3]);
                    acc[h][4] = fmaf(weight, bf16_lo(bits.z), acc[h][4]);
                    acc[h][5] = fmaf(weight, bf16_hi(bits.z), acc[h][5]);
                    acc[h][6] = fmaf(weight, bf16_lo(bits.w), acc[h][6]);
                    acc[h][7] = fmaf(weight, bf16_hi(bits.w), acc[h][7]);
                }
        });
        if (more) current = next;
    }

    // Merge the four lane groups' streams: lanes l, l^16, l^32, l^48 hold the same head.
    float all_max = fmaxf(running_max, wave_xor(running_max, 16));
    all_max = fmaxf(all_max, wave_xor(all_max, 32));
    const float all_base = all_max == -INFINITY ? 0.0f : all_max;
    const float weight = fast_exp2(running_max - all_base);
    float all_sum = running_sum * weight;
    all_sum += wave_xor(all_sum, 16);
    all_sum += wave_xor(all_sum, 32);
    const float inverse = all_sum > 0.0f ? 1.0f / all_sum : 0.0f;
    const float lse = all_sum > 0.0f ? (all_max + fast_log2(all_sum)) * kLn2 : -INFINITY;

    static_for<GROUPS>([&](auto head) {
        constexpr int h = decltype(head)::value;
        const float factor = group_broadcast<GROUPS, h>(weight);
        const float norm = group_broadcast<GROUPS, h>(inverse);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            float value = acc[h][e] * factor;
            value += wave_xor(value, 16);
            value += wave_xor(value, 32);
            acc[h][e] = value * norm;
        }
    });

    // Lane group g stores heads g, g + 4, ...; 16 lanes x 32 B cover one 128-wide row.
    static_for<GROUPS>([&](auto head) {
        constexpr int h = decltype(head)::value;
        if (h < group && (h & 3) == static_cast<int>(g)) {
            const size_t row = (static_cast<size_t>(batch) * a.heads + kv_head * group + h) * a.splits + split;
            float4* out = reinterpret_cast<float4*>(a.partial_out + row * kDim + 8 * t);
            out[0] = make_float4(acc[h][0], acc[h][1], acc[h][2], acc[h][3]);
            out[1] = make_float4(acc[h][4], acc[h][5], acc[h][6], acc[h][7]);
        }
    });
    if (g == 0 && t < GROUPS && t < group) {
        const size_t row = (static_cast<size_t>(batch) * a.heads + kv_head * group + t) * a.splits + split;
        a.partial_lse[row] = lse;
    }
}

}  // namespace

#define SINGE_DECODE_KERNEL(GROUPS, ALIGNED, SUFFIX)                                                     \
    extern "C" __global__ __launch_bounds__(64) void singe_paged_decode_bf16_d128_g##GROUPS##SUFFIX(      \
        DecodeArgs args) {                                                                              \
        paged_decode_body<GROUPS, ALIGNED>(args);                                                       \
    }

SINGE_DECODE_KERNEL(1, true, _b16)
SINGE_DECODE_KERNEL(2, true, _b16)
SINGE_DECODE_KERNEL(4, true, _b16)
SINGE_DECODE_KERNEL(8, true, _b16)
SINGE_DECODE_KERNEL(16, true, _b16)
SINGE_DECODE_KERNEL(1, false, _any)
SINGE_DECODE_KERNEL(2, false, _any)
SINGE_DECODE_KERNEL(4, false, _any)
SINGE_DECODE_KERNEL(8, false, _any)
SINGE_DECODE_KERNEL(16, false, _any)

// Folds the per-split partial rows of one (batch, head) into the bf16 output:
// out = sum_s exp(lse_s - max) * partial_s / sum_s exp(lse_s - max)
// (singe-kernel/src/cpu/attention.rs:2157-2193).  One thread per output element.
extern "C" __global__ __launch_bounds__(128) void singe_paged_decode_combine_bf16(CombineArgs a) {
    const unsigned int row = blockIdx.x;  // batch * heads + head
    const unsigned int batch = row / a.heads;
    int raw_len = a.actual_seq_lens[batch];
    const unsigned int seq_len = raw_len < 0 ? 0u : (static_cast<unsigned int>(raw_len) < a.reach ? static_cast<unsigned int>(raw_len) : a.reach);
    const unsigned int used = (seq_len + a.keys_per_split - 1) / a.keys_per_split;
    const float* lse = a.partial_lse + static_cast<size_t>(row) * a.splits;
    float largest = -INFINITY;
    for (unsigned int s = 0; s < used; ++s) largest = fmaxf(largest, lse[s]);
    for (unsigned int d = threadIdx.x; d < a.dim; d += blockDim.x) {
        float total = 0.0f, sum = 0.0f;
        if (largest != -INFINITY) {
            for (unsigned int s = 0; s < used; ++s) {
                const float weight = __expf(lse[s] - largest);
                total += weight;
                sum = fmaf(weight, a.partial_out[(static_cast<size_t>(row) * a.splits + s) * a.dim + d], sum);
            }
        }
        // A sequence with no keys keeps a zero row (cpu/attention.rs:1213-1215).
        a.out[static_cast<size_t>(row) * a.dim + d] = f32_to_bf16_bits(total > 0.0f ? sum / total : 0.0f);
    }
}
