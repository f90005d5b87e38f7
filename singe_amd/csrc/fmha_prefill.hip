// Dense flash-attention prefill, bf16, head_dim 128, optional top-left causal mask, grouped KV heads
// (the GPU counterpart of singe-kernel/src/cpu/attention.rs:1758-1833 fmha_prefill_lse_f32, replacing
// the cuTile fmha_prefill / fmha_prefill_mma kernels: singe-kernel/src/cuda/attention/fmha.rs:584-790).
// query/out [batch, query_len, heads, 128], key/value [batch, key_len, kv_heads, 128] with element
// strides from FmhaPrefillConfig; lse [batch, heads, query_len], natural log.
//
// A workgroup of four waves owns 128 query rows of one (batch, head); each wave owns 32 of them and
// walks the key axis in tiles of 64 keys staged in LDS (double buffered, one barrier per tile).
// Everything is kept transposed so the softmax weights never leave registers:
//
//   S^T[key, query] = K . Q^T      v_mfma_f32_32x32x16_bf16, A = K rows read from LDS (16-byte reads,
//                                  rows padded to 272 B so 16 lanes hit 64 distinct banks), B = the
//                                  wave's Q^T, resident in 32 VGPRs for the whole kernel;
//   online softmax                 base two with scale * log2(e) folded in; a lane holds the scores of
//                                  ONE query (its MFMA column), so the row maximum is 31 in-lane max
//                                  ops and one v_permlane32_swap, and rescaling O^T needs no broadcast;
//   O^T[dim, query] += V^T . P^T   A = V^T read from LDS with ds_read_b64_tr_b16 (the hardware transposes
//                                  four keys x four dims per 16 lanes; rows padded to 320 B), B = P^T
//                                  packed to bf16 straight from the S^T accumulator registers, whose
//                                  (lane, register) -> key map is what fixes the V^T read pattern.
//
// Probabilities are rounded to bf16 for the second product and summed unrounded, like the reference's
// tensor-core kernel (singe/src/backend/cuda/kernel_plan/source/tensor_core.rs:162-183).
//
// Grid: one workgroup per (batch, head, 128-row query tile).  Workgroup i lands on XCD i % 8, so ids
// are laid out to keep the query tiles of one head on one XCD (its K/V then stay in that XCD's L2),
// heaviest (last) query tiles first so the causal triangle drains evenly.
#include "common.hip.h"
#include "kernel_args.h"

namespace {

constexpr int kHeadDim = 128;
constexpr int kQueryTile = 128;       // query rows per workgroup
constexpr int kKeyTile = 64;          // keys per LDS stage
constexpr int kKeyRowBytes = 272;     // 256 B of K + 16 B pad
constexpr int kValueRowBytes = 320;   // 256 B of V + 64 B pad
constexpr int kKeyStageBytes = kKeyTile * kKeyRowBytes;
constexpr int kValueStageBytes = kKeyTile * kValueRowBytes;
constexpr int kStageBytes = kKeyStageBytes + kValueStageBytes;

typedef short v4i16_t __attribute__((ext_vector_type(4)));
typedef short v8i16_t __attribute__((ext_vector_type(8)));

SINGE_DEVICE float swap32_max(float value) {
    float kept = value, taken = value;
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(kept), "+v"(taken));
    return fmaxf(kept, taken);
}

SINGE_DEVICE float swap32_sum(float value) {
    float kept = value, taken = value;
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(kept), "+v"(taken));
    return kept + taken;
}

typedef __bf16 bf16x2v_t __attribute__((ext_vector_type(2)));
typedef float f32x2v_t __attribute__((ext_vector_type(2)));

SINGE_DEVICE unsigned int pack_pair(float lo, float hi) {
    f32x2v_t both = {lo, hi};
    return __builtin_bit_cast(unsigned int, __builtin_convertvector(both, bf16x2v_t));
}

// How far (log2 units) a row's maximum may run ahead of the reference point its weights are scaled
// by before the accumulators are rescaled.  Any reference point gives the same quotient; letting it lag
// by up to 2^6 keeps weights far inside bf16/f32 range and makes the rescale of O^T rare after the
// first tiles.
constexpr float kMaxLag = 6.0f;

template <bool CAUSAL>
SINGE_DEVICE void fmha_prefill_body(const PrefillArgs& a, unsigned char* lds) {
    const unsigned int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const unsigned int column = lane & 31, hi = lane >> 5;

    // Workgroup id -> (batch * heads + head, query tile): see the header comment.
    const unsigned int xcd = blockIdx.x & 7u, within = blockIdx.x >> 3;
    const unsigned int bh = (within / a.query_tiles) * 8u + xcd;
    if (bh >= a.batch * a.heads) return;
    const unsigned int query_tile = a.query_tiles - 1u - within % a.query_tiles;
    const unsigned int batch = bh / a.heads, head = bh % a.heads;
    const unsigned int kv_head = head / (a.heads / a.kv_heads);

    const unsigned int first_row = query_tile * kQueryTile + wave * 32u;  // of this wave
    const unsigned int my_query = first_row + column;
    const bool query_valid = my_query < a.query_len;

    const uint16_t* q_base = a.query + batch * a.query_batch_stride + head * a.query_head_stride;
    const uint16_t* k_base = a.key + batch * a.key_batch_stride + kv_head * a.key_head_stride;
    const uint16_t* v_base = a.value + batch * a.value_batch_stride + kv_head * a.value_head_stride;

    // Q^T as the MFMA B operand: lane (column = query, hi) holds dims 16s + 8hi .. +8 for s = 0..7.
    // A negative scale is moved into Q (sign bits flipped) so the softmax below can take the row
    // maximum of the raw scores and fold the positive factor into one fused multiply-add.
    const float factor = fabsf(a.scale_log2e);
    const unsigned int flip = a.scale_log2e < 0.0f ? 0x80008000u : 0u;
    bf16x8_t q[8];
    {
        const uint16_t* row = q_base + static_cast<size_t>(query_valid ? my_query : 0) * a.query_sequence_stride + 8 * hi;
#pragma unroll
        for (int s = 0; s < 8; ++s) {
            uint4 bits = *reinterpret_cast<const uint4*>(row + 16 * s);
            if (!query_valid) bits = make_uint4(0, 0, 0, 0);
            bits.x ^= flip; bits.y ^= flip; bits.z ^= flip; bits.w ^= flip;
            q[s] = __builtin_bit_cast(bf16x8_t, bits);
        }
    }

    // Keys this workgroup must visit, and its share of the tile loads: 1024 16-byte chunks per
    // operand per tile, four per thread.
    unsigned int key_end = a.key_len;
    if (CAUSAL) {
        const unsigned int reach = query_tile * kQueryTile + kQueryTile;
        key_end = key_end < reach ? key_end : reach;
    }
    const unsigned int tiles = (key_end + kKeyTile - 1) / kKeyTile;

    const unsigned int load_row = tid >> 4, load_col = tid & 15u;  // chunk i of a thread: row + 16 i
    // The next tile on its way from global memory to LDS: four 16-byte chunks of K and of V per thread
    // (named registers, not arrays, so they are never given a stack slot).
    uint4 k0, k1, k2, k3, v0, v1, v2, v3;
    auto fetch_row = [&](unsigned int tile, unsigned int i, uint4& key_bits, uint4& value_bits) __attribute__((always_inline)) {
        unsigned int key = tile * kKeyTile + load_row + 16u * i;
        key = key < a.key_len ? key : a.key_len - 1;  // rows past the end re-read the last key and are masked
        key_bits = *reinterpret_cast<const uint4*>(k_base + static_cast<size_t>(key) * a.key_sequence_stride + load_col * 8u);
        value_bits = *reinterpret_cast<const uint4*>(v_base + static_cast<size_t>(key) * a.value_sequence_stride + load_col * 8u);
    };
    auto fetch = [&](unsigned int tile) __attribute__((always_inline)) {
        fetch_row(tile, 0, k0, v0);
        fetch_row(tile, 1, k1, v1);
        fetch_row(tile, 2, k2, v2);
        fetch_row(tile, 3, k3, v3);
    };
    auto stash_row = [&](unsigned char* keys, unsigned char* values, unsigned int i, const uint4& key_bits, const uint4& value_bits) __attribute__((always_inline)) {
        const unsigned int row = load_row + 16u * i;
        *reinterpret_cast<uint4*>(keys + row * kKeyRowBytes + load_col * 16) = key_bits;
        *reinterpret_cast<uint4*>(values + row * kValueRowBytes + load_col * 16) = value_bits;
    };
    auto stash = [&](unsigned char* keys, unsigned char* values) __attribute__((always_inline)) {
        stash_row(keys, values, 0, k0, v0);
        stash_row(keys, values, 1, k1, v1);
        stash_row(keys, values, 2, k2, v2);
        stash_row(keys, values, 3, k3, v3);
    };

    f32x16_t out[4];
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) out[db][r] = 0.0f;
    // reference = the point the weights are scaled by (scaled log2 units); it trails the true row
    // maximum by at most kMaxLag.
    float reference = -INFINITY, running_sum = 0.0f;

    if (tiles > 0) {
        fetch(0);
        stash(lds, lds + kKeyStageBytes);
    }
    __syncthreads();

    // Per-lane LDS read offsets.  K: row = key (column), 16 B at dims 16s + 8hi.  V^T through the
    // transposing read: lane 16G + s of a 16-lane group points at key (s >> 2), dims 4 (s & 3) .. +4 of
    // the group's 16 dims; the hardware hands lane i the four keys of dim i.
    const unsigned int key_read = column * kKeyRowBytes + 16 * hi;
    const unsigned int group = lane >> 4, sub = lane & 15u;
    const unsigned int value_read = (4 * hi + (sub >> 2)) * kValueRowBytes + (16 * (group & 1u) + 4 * (sub & 3u)) * 2;

    // Folds the 64 keys staged at `keys` / `values` (tile index `tile`) into the running state.
    auto fold = [&](unsigned int tile, const unsigned char* keys, const unsigned char* values) __attribute__((always_inline)) {
        const unsigned int key0 = tile * kKeyTile;
        // A 32-key block wholly after the wave's last query contributes nothing under the causal mask.
        const bool live0 = !CAUSAL || key0 <= first_row + 31u;
        const bool live1 = !CAUSAL || key0 + 32u <= first_row + 31u;
        if (!live0) return;

        // Scores.  All eight K operands of a block are read before its MFMA chain starts, and the reads
        // of the second block are issued while the first chain runs, so the matrix core never waits on
        // a single LDS round trip.
        f32x16_t s0, s1;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            s0[r] = 0.0f;
            s1[r] = 0.0f;
        }
        uint4 ka[8], kb[8];
#pragma unroll
        for (int step = 0; step < 8; ++step) ka[step] = *reinterpret_cast<const uint4*>(keys + key_read + step * 32);
        if (live1) {
#pragma unroll
            for (int step = 0; step < 8; ++step) {
                kb[step] = *reinterpret_cast<const uint4*>(keys + 32 * kKeyRowBytes + key_read + step * 32);
                s0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, ka[step]), q[step], s0, 0, 0, 0);
            }
#pragma unroll
            for (int step = 0; step < 8; ++step)
                s1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, kb[step]), q[step], s1, 0, 0, 0);
        } else {
#pragma unroll
            for (int step = 0; step < 8; ++step)
                s0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, ka[step]), q[step], s0, 0, 0, 0);
        }

        // Hide what the query may not see: keys after it (causal), keys past the end of the tensor,
        // and the second block when it is wholly hidden.  Only tiles on an edge pay for this.
        const bool edge = (CAUSAL && key0 + kKeyTile - 1 > first_row) || key0 + kKeyTile > a.key_len;
        if (edge) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const unsigned int key = key0 + 8 * (r >> 2) + 4 * hi + (r & 3);
                if ((CAUSAL && key > my_query) || key >= a.key_len) s0[r] = -INFINITY;
                if ((CAUSAL && key + 32 > my_query) || key + 32 >= a.key_len || !live1) s1[r] = -INFINITY;
            }
        }

        float largest = fmaxf(s0[0], s1[0]);
#pragma unroll
        for (int r = 1; r < 16; ++r) largest = fmaxf(largest, fmaxf(s0[r], s1[r]));
        largest = swap32_max(largest) * factor;  // both lanes of a query agree from here on
        if (__any(largest > reference + kMaxLag || (reference == -INFINITY && largest != -INFINITY))) {
            const float moved = fmaxf(reference, largest);
            const float base = moved == -INFINITY ? 0.0f : moved;
            const float rescale = fast_exp2(reference - base);
            running_sum *= rescale;
#pragma unroll
            for (int db = 0; db < 4; ++db)
#pragma unroll
                for (int r = 0; r < 16; ++r) out[db][r] *= rescale;
            reference = moved;
        }
        const float shift = reference == -INFINITY ? 0.0f : -reference;
        float total = 0.0f;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            s0[r] = fast_exp2(fmaf(s0[r], factor, shift));
            s1[r] = fast_exp2(fmaf(s1[r], factor, shift));
            total += s0[r] + s1[r];
        }
        running_sum += total;

        // O^T += V^T . P^T, 16 keys per MFMA: registers 8j .. 8j+7 of a block are keys
        // 16j + {0..3, 8..11} + 4hi of it, which is what the two transposing reads fetch.
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const uint4 weights = make_uint4(pack_pair(s0[8 * j + 0], s0[8 * j + 1]), pack_pair(s0[8 * j + 2], s0[8 * j + 3]),
                                             pack_pair(s0[8 * j + 4], s0[8 * j + 5]), pack_pair(s0[8 * j + 6], s0[8 * j + 7]));
            const unsigned char* rows = values + (16 * j) * kValueRowBytes + value_read;
#pragma unroll
            for (int db = 0; db < 4; ++db) {
                const v4i16_t low = __builtin_amdgcn_ds_read_tr16_b64_v4i16((v4i16_t __attribute__((address_space(3)))*)(rows + db * 64));
                const v4i16_t high = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    (v4i16_t __attribute__((address_space(3)))*)(rows + 8 * kValueRowBytes + db * 64));
                const v8i16_t both = __builtin_shufflevector(low, high, 0, 1, 2, 3, 4, 5, 6, 7);
                out[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, both),
                                                                  __builtin_bit_cast(bf16x8_t, weights), out[db], 0, 0, 0);
            }
        }
        if (live1) {
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const uint4 weights = make_uint4(pack_pair(s1[8 * j + 0], s1[8 * j + 1]), pack_pair(s1[8 * j + 2], s1[8 * j + 3]),
                                                 pack_pair(s1[8 * j + 4], s1[8 * j + 5]), pack_pair(s1[8 * j + 6], s1[8 * j + 7]));
                const unsigned char* rows = values + (32 + 16 * j) * kValueRowBytes + value_read;
#pragma unroll
                for (int db = 0; db < 4; ++db) {
                    const v4i16_t low = __builtin_amdgcn_ds_read_tr16_b64_v4i16((v4i16_t __attribute__((address_space(3)))*)(rows + db * 64));
                    const v4i16_t high = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                        (v4i16_t __attribute__((address_space(3)))*)(rows + 8 * kValueRowBytes + db * 64));
                    const v8i16_t both = __builtin_shufflevector(low, high, 0, 1, 2, 3, 4, 5, 6, 7);
                    out[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, both),
                                                                      __builtin_bit_cast(bf16x8_t, weights), out[db], 0, 0, 0);
                }
            }
        }
    };

    unsigned char* const keys0 = lds;
    unsigned char* const values0 = lds + kKeyStageBytes;
    unsigned char* const keys1 = lds + kStageBytes;
    unsigned char* const values1 = lds + kStageBytes + kKeyStageBytes;
    for (unsigned int tile = 0; tile < tiles; tile += 2) {
        if (tile + 1 < tiles) fetch(tile + 1);
        fold(tile, keys0, values0);
        if (tile + 1 < tiles) stash(keys1, values1);
        __syncthreads();
        if (tile + 1 >= tiles) break;
        if (tile + 2 < tiles) fetch(tile + 2);
        fold(tile + 1, keys1, values1);
        if (tile + 2 < tiles) stash(keys0, values0);
        __syncthreads();
    }

    // Normalise and store.  Lane (query, hi) holds dims 32db + 8(r / 4) + 4hi + (r % 4).
    const float sum = swap32_sum(running_sum);
    const float inverse = sum > 0.0f ? 1.0f / sum : 0.0f;
    if (query_valid) {
        uint16_t* row = a.out + batch * a.output_batch_stride + static_cast<size_t>(my_query) * a.output_sequence_stride +
                        head * a.output_head_stride;
#pragma unroll
        for (int db = 0; db < 4; ++db)
#pragma unroll
            for (int quad = 0; quad < 4; ++quad) {
                uint2 packed;
                packed.x = pack_pair(out[db][4 * quad + 0] * inverse, out[db][4 * quad + 1] * inverse);
                packed.y = pack_pair(out[db][4 * quad + 2] * inverse, out[db][4 * quad + 3] * inverse);
                *reinterpret_cast<uint2*>(row + 32 * db + 8 * quad + 4 * hi) = packed;
            }
        if (a.lse != nullptr && hi == 0)
            a.lse[(static_cast<size_t>(batch) * a.heads + head) * a.query_len + my_query] =
                sum > 0.0f ? (reference + fast_log2(sum)) * kLn2 : -INFINITY;
    }
}

}  // namespace

extern "C" __global__ __launch_bounds__(256, 2) void singe_fmha_prefill_bf16_d128_causal(PrefillArgs args) {
    __shared__ __attribute__((aligned(16))) unsigned char prefill_lds[2 * kStageBytes];
    fmha_prefill_body<true>(args, prefill_lds);
}

extern "C" __global__ __launch_bounds__(256, 2) void singe_fmha_prefill_bf16_d128_full(PrefillArgs args) {
    __shared__ __attribute__((aligned(16))) unsigned char prefill_lds[2 * kStageBytes];
    fmha_prefill_body<false>(args, prefill_lds);
}
