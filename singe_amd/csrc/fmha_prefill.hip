// Dense flash-attention prefill, bf16, head_dim 128, optional top-left causal mask, grouped KV heads
// (the GPU counterpart of singe-kernel/src/cpu/attention.rs:1758-1833 fmha_prefill_lse_f32, replacing
// the cuTile fmha_prefill / fmha_prefill_mma kernels: singe-kernel/src/cuda/attention/fmha.rs:584-790).
// query/out [batch, query_len, heads, 128], key/value [batch, key_len, kv_heads, 128] with element
// strides from FmhaPrefillConfig; lse [batch, heads, query_len], natural log.
//
// A workgroup of four waves owns 128 query rows of one (batch, head); each wave owns 32 of them and
// walks the key axis in tiles of 64 keys staged in LDS (double buffered, one barrier per tile).
// The per-tile arithmetic (transposed products on v_mfma_f32_32x32x16_bf16, online softmax, transposing
// LDS reads for V) is the shared core in prefill_core.hip.h.
//
// Grid: one workgroup per (batch, head, 128-row query tile).  Workgroup i lands on XCD i % 8, so a
// (batch, head) is pinned to an XCD (its K/V then stay in that XCD's L2); within an XCD the workgroups
// run the heaviest (last) query tiles of every head first, so the causal triangle drains evenly.
#include "kernel_args.h"
#include "prefill_core.hip.h"

namespace {

using namespace prefill;

template <bool CAUSAL>
SINGE_DEVICE void fmha_prefill_body(const PrefillArgs& a, unsigned char* lds) {
    const unsigned int tid = threadIdx.x, lane = tid & 63;
    // The wave index is the same in all lanes; saying so keeps everything derived from it (which keys
    // are live, whether a tile is on the mask's edge) in scalar registers and scalar branches.
    const unsigned int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const unsigned int column = lane & 31, hi = lane >> 5;

    // Workgroup id -> (batch * heads + head, query tile): see the header comment.
    const unsigned int xcd = blockIdx.x & 7u, within = blockIdx.x >> 3;
    const unsigned int per_xcd = (a.batch * a.heads + 7u) / 8u;
    const unsigned int bh = (within % per_xcd) * 8u + xcd;
    if (bh >= a.batch * a.heads) return;
    const unsigned int query_tile = a.query_tiles - 1u - within / per_xcd;
    const unsigned int batch = bh / a.heads, head = bh % a.heads;
    const unsigned int kv_head = head / (a.heads / a.kv_heads);

    const unsigned int first_row = query_tile * kQueryTile + wave * 32u;  // of this wave
    const unsigned int my_query = first_row + column;
    const bool query_valid = my_query < a.query_len;

    const uint16_t* q_base = a.query + batch * a.query_batch_stride + head * a.query_head_stride;
    const uint16_t* k_base = a.key + batch * a.key_batch_stride + kv_head * a.key_head_stride;
    const uint16_t* v_base = a.value + batch * a.value_batch_stride + kv_head * a.value_head_stride;

    // Q^T as the MFMA B operand: lane (column = query, hi) holds dims 16s + 8hi .. +8 for s = 0..7.
    // A negative scale is moved into Q (sign bits flipped) so the softmax can take the row maximum of
    // the raw scores and fold the positive factor into one fused multiply-add.
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
    // Offsets inside one (batch, head) slice fit 32 bits (checked by the host), so a load is a uniform
    // base plus a 32-bit lane offset.
    const unsigned int key_stride_bytes = static_cast<unsigned int>(a.key_sequence_stride) * 2u;
    const unsigned int value_stride_bytes = static_cast<unsigned int>(a.value_sequence_stride) * 2u;
    const unsigned char* const k_bytes = reinterpret_cast<const unsigned char*>(k_base);
    const unsigned char* const v_bytes = reinterpret_cast<const unsigned char*>(v_base);
    auto fetch_row = [&](unsigned int tile, unsigned int i, uint4& key_bits, uint4& value_bits) __attribute__((always_inline)) {
        unsigned int key = tile * kKeyTile + load_row + 16u * i;
        key = key < a.key_len ? key : a.key_len - 1;  // rows past the end re-read the last key and are masked
        key_bits = *reinterpret_cast<const uint4*>(k_bytes + (key * key_stride_bytes + load_col * 16u));
        value_bits = *reinterpret_cast<const uint4*>(v_bytes + (key * value_stride_bytes + load_col * 16u));
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

    RowState state;
    reset(state);

    if (tiles > 0) {
        fetch(0);
        stash(lds, lds + kKeyStageBytes);
    }
    __syncthreads();

    const unsigned int key_read = key_read_offset(lane), value_read = value_read_offset(lane);

    // Folds the 64 keys staged at `keys` / `values` (tile index `tile`) into the running state.
    auto fold = [&](unsigned int tile, const unsigned char* keys, const unsigned char* values) __attribute__((always_inline)) {
        const unsigned int key0 = tile * kKeyTile;
        // A 32-key block wholly after the wave's last query contributes nothing under the causal mask.
        const bool live0 = !CAUSAL || key0 <= first_row + 31u;
        const bool live1 = !CAUSAL || key0 + 32u <= first_row + 31u;
        if (!live0) return;
        // Keys after the query (causal) and keys past the end of the tensor are hidden.
        const bool edge = (CAUSAL && key0 + kKeyTile - 1 > first_row) || key0 + kKeyTile > a.key_len;
        fold_staged_keys<false>(state, q, keys, values, key_read, value_read, hi, factor, live1, edge,
                                [&](unsigned int block, unsigned int key_in_block) {
                                    const unsigned int key = key0 + 32 * block + key_in_block;
                                    return (CAUSAL && key > my_query) || key >= a.key_len;
                                });
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
    const float sum = swap32_sum(state.running_sum);
    const float inverse = sum > 0.0f ? 1.0f / sum : 0.0f;
    if (query_valid) {
        uint16_t* row = a.out + batch * a.output_batch_stride + static_cast<size_t>(my_query) * a.output_sequence_stride +
                        head * a.output_head_stride;
#pragma unroll
        for (int db = 0; db < 4; ++db)
#pragma unroll
            for (int quad = 0; quad < 4; ++quad) {
                uint2 packed;
                packed.x = pack_pair(state.out[db][4 * quad + 0] * inverse, state.out[db][4 * quad + 1] * inverse);
                packed.y = pack_pair(state.out[db][4 * quad + 2] * inverse, state.out[db][4 * quad + 3] * inverse);
                *reinterpret_cast<uint2*>(row + 32 * db + 8 * quad + 4 * hi) = packed;
            }
        if (a.lse != nullptr && hi == 0)
            a.lse[(static_cast<size_t>(batch) * a.heads + head) * a.query_len + my_query] =
                sum > 0.0f ? (state.reference + fast_log2(sum)) * kLn2 : -INFINITY;
    }
}

}  // namespace

extern "C" __global__ __launch_bounds__(256, 2) void singe_fmha_prefill_bf16_d128_causal(PrefillArgs args) {
    __shared__ __attribute__((aligned(16))) unsigned char prefill_lds[2 * prefill::kStageBytes];
    fmha_prefill_body<true>(args, prefill_lds);
}

extern "C" __global__ __launch_bounds__(256, 2) void singe_fmha_prefill_bf16_d128_full(PrefillArgs args) {
    __shared__ __attribute__((aligned(16))) unsigned char prefill_lds[2 * prefill::kStageBytes];
    fmha_prefill_body<false>(args, prefill_lds);
}
