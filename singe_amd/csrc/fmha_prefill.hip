// Dense flash-attention prefill, bf16 or f16, head_dim 128 or 64 (one build each), optional top-left causal mask, grouped KV heads
// (the GPU counterpart of singe-kernel/src/cpu/attention.rs:1758-1833 fmha_prefill_lse_f32, replacing
// the cuTile fmha_prefill / fmha_prefill_mma kernels: singe-kernel/src/cuda/attention/fmha.rs:584-790).
// query/out [batch, query_len, heads, 128], key/value [batch, key_len, kv_heads, 128] with element
// strides from FmhaPrefillConfig; lse [batch, heads, query_len], natural log.
//
// A workgroup of kDensePrefillWaves (four) waves owns 32 query rows per wave of one (batch, head); each wave
// walks the key axis in blocks of 32 keys.  Tiles of 64 keys go from global memory straight into LDS
// (three K stages, two V stages, one barrier per tile): while tile t is worked on, K of tile t + 2 and V of
// tile t + 1 are on their way, so every load has a whole tile's arithmetic to land and no register holds
// data in transit.  The score products of a block are woven into the exponentials of the block before it
// (prefill_blocks.hip.h), which keeps the matrix core fed while the vector unit works.
//
// Grid: one workgroup per (batch, head, pair of 128-row query tiles): tile i from the end and tile i from
// the start, so under the causal mask every workgroup has the same amount of work.  Workgroup i lands on
// XCD i % 8; ids are laid out so the workgroups of one (batch, head) are neighbours on one XCD and walk
// its keys side by side, which keeps its K/V in that XCD's L2.
#include "kernel_args.h"
#include "prefill_blocks.hip.h"

namespace {

using namespace prefill;

// Whether the interior tiles read their K operands a block ahead (prefill_blocks.hip.h): measured, it gains
// nothing here (the other wave of the SIMD already covers the reads' latency) and costs 30 registers.
constexpr bool kDenseOperandsAhead = false;
// Waves of a workgroup, 32 query rows each: the K and V tiles a workgroup loads serve all of them.
constexpr int kDenseWaves = kDensePrefillWaves;

// One 128-row query tile of (batch, head) pair `bh`.
// OPTIONS: the dense op's additive mask, window and score cap, applied block by block to the scaled scores; every
// tile then takes the masked path.
template <bool CAUSAL, class Half, int WAVES, bool OPTIONS>
SINGE_DEVICE void fmha_prefill_tile(const PrefillArgs& a, unsigned char* lds, unsigned int bh, unsigned int query_tile, unsigned int split) {
    constexpr unsigned int kRows = 32u * WAVES;        // query rows of the workgroup
    constexpr unsigned int kLoadRows = 4u * WAVES;     // key rows one load instruction of every wave brings in
    constexpr unsigned int kLoads = kKeyTile / kLoadRows;
    const unsigned int tid = threadIdx.x, lane = tid & 63;
    // The wave index is the same in all lanes; saying so keeps everything derived from it (which blocks
    // are live, whether a block is on the mask's edge, LDS bases) in scalar registers and scalar branches.
    const unsigned int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const unsigned int column = lane & 31, hi = lane >> 5;

    // (packed_heads: `bh` counts (batch, kv head) pairs and the rows of the one tile are (query, head of the group) pairs.)
    const bool packed = a.packed_heads != 0;
    const unsigned int group = a.heads / a.kv_heads;
    const unsigned int batch = packed ? bh / a.kv_heads : bh / a.heads;
    // Keys that take part: all of them, or the batch entry's own count (singe/src/backend/cpu/normalization/attention.rs:191-276, key_lengths).
    unsigned int key_len = a.key_len;
    if (a.key_lengths != nullptr) {
        const int own = a.key_lengths[batch];
        const unsigned int bound = own > 0 ? static_cast<unsigned int>(own) : 0u;
        key_len = bound < key_len ? bound : key_len;
    }
    key_len = __builtin_amdgcn_readfirstlane(key_len);
    const unsigned int kv_head = packed ? bh % a.kv_heads : (bh % a.heads) / group;

    const unsigned int first_row = query_tile * kRows + wave * 32u;  // of this wave
    const unsigned int my_row = first_row + column;
    const unsigned int my_query = packed ? my_row / group : my_row;
    const unsigned int head = packed ? kv_head * group + my_row % group : bh % a.heads;
    const bool query_valid = my_query < a.query_len;

    const uint16_t* q_base = a.query + batch * a.query_batch_stride + head * a.query_head_stride;
    const unsigned char* const k_bytes = reinterpret_cast<const unsigned char*>(a.key + batch * a.key_batch_stride + kv_head * a.key_head_stride);
    const unsigned char* const v_bytes = reinterpret_cast<const unsigned char*>(a.value + batch * a.value_batch_stride + kv_head * a.value_head_stride);

    // Q^T as the MFMA B operand: lane (column = query, hi) holds dims 16s + 8hi .. +8 for s = 0..7.
    // A negative scale is moved into Q (sign bits flipped) so the softmax can take the row maximum of
    // the raw scores and fold the positive factor into one fused multiply-add.
    const float factor = fabsf(a.scale_log2e);
    const unsigned int flip = a.scale_log2e < 0.0f ? 0x80008000u : 0u;
    const Half half{};
    uint4 q[kSteps];
    {
        const uint16_t* row = q_base + static_cast<size_t>(query_valid ? my_query : 0) * a.query_sequence_stride + 8 * hi;
#pragma unroll
        for (int s = 0; s < kSteps; ++s) {
            uint4 bits = *reinterpret_cast<const uint4*>(row + 16 * s);
            if (!query_valid) bits = make_uint4(0, 0, 0, 0);
            bits.x ^= flip; bits.y ^= flip; bits.z ^= flip; bits.w ^= flip;
            q[s] = bits;
        }
    }

    // Keys this workgroup must visit, and the blocks of them this wave folds: under the causal mask a
    // block wholly after the wave's last query contributes nothing.
    unsigned int key_end = key_len;
    if (CAUSAL) {
        const unsigned int reach = query_tile * kRows + kRows;
        key_end = key_end < reach ? key_end : reach;
    }
    unsigned int tiles = (key_end + kKeyTile - 1) / kKeyTile;
    unsigned int wave_blocks = (key_end + 31u) / 32u;
    if (CAUSAL) {
        const unsigned int seen = (first_row + 31u) / 32u + 1u;
        wave_blocks = wave_blocks < seen ? wave_blocks : seen;
    }
    // The first tile any row of the workgroup can see: 0, or with a window the tile of the first key the
    // workgroup's first row still sees (later rows see later keys).
    unsigned int first_tile = 0;
    if (OPTIONS && a.window >= 0) {
        const unsigned long long low = static_cast<unsigned long long>(query_tile) * kRows + 1u;
        const unsigned long long window = static_cast<unsigned long long>(a.window);
        if (low > window) first_tile = static_cast<unsigned int>((low - window) / kKeyTile);
        first_tile = first_tile < tiles ? first_tile : tiles;
    }
    if (a.splits > 1) {
        // This workgroup's share of the tiles; a share may be empty, and ends with its last tile.
        const unsigned int share = tiles > first_tile ? (tiles - first_tile + a.splits - 1) / a.splits : 0u;
        first_tile += split * share;
        tiles = tiles < first_tile + share ? tiles : first_tile + share;
        first_tile = first_tile < tiles ? first_tile : tiles;
        wave_blocks = wave_blocks < 2u * tiles ? wave_blocks : 2u * tiles;
    }

    // A tile load is 1024 16-byte chunks per operand: instruction i of wave w fills rows 16 i + 4 w .. + 3
    // (1 KiB of LDS starting at a wave-uniform address), lane l the chunk position l % 16 of row
    // 16 i + 4 w + l / 16, fetched from the chunk the row's permutation puts there.  Offsets inside one
    // (batch, head) slice fit 32 bits (checked by the host).
    const unsigned int key_stride_bytes = static_cast<unsigned int>(a.key_sequence_stride) * 2u;
    const unsigned int value_stride_bytes = static_cast<unsigned int>(a.value_sequence_stride) * 2u;
    const unsigned int load_row = 4u * wave + (lane >> 4), position = lane & 15u;
    const unsigned int key_chunk = (position ^ (load_row & 15u)) * 16u, value_chunk = (position ^ (4u * (load_row & 3u))) * 16u;
    // At head_dim 64 a global row has eight chunks: the lanes whose position holds one of the other eight fetch nothing.
    const bool key_lane_live = key_chunk < kGlobalRowBytes, value_lane_live = value_chunk < kGlobalRowBytes;
    // A tile that lies wholly inside the keys is addressed as a scalar base (tile and instruction) plus a
    // per-lane offset that never changes, so its loads cost no vector arithmetic; the last, partial tile
    // clamps each row (rows past the end re-read the last key and are masked).
    const unsigned int key_lane = load_row * key_stride_bytes + key_chunk, value_lane = load_row * value_stride_bytes + value_chunk;
    auto load_tile = [&](const unsigned char* rows, unsigned int stride_bytes, unsigned int lane_offset, unsigned int chunk,
                         bool lane_live, unsigned int tile, unsigned char* stage) __attribute__((always_inline)) {
        // (only the load itself is predicated, so that the scalar address arithmetic stays outside the branch)
        const bool fetch = kGlobalRowBytes == kRowBytes || lane_live;
        if (tile * kKeyTile + kKeyTile <= key_len) {
            const unsigned char* base = rows + static_cast<size_t>(tile * kKeyTile) * stride_bytes;
            asm("" : "+s"(base));  // a scalar the compiler cannot fold the lane's part into
#pragma unroll
            for (unsigned int i = 0; i < kLoads; ++i) {
                // The offset is pinned to this spot as a 32-bit value: hoisted and widened, it would take the
                // load out of its scalar-base form and cost a 64-bit add per lane.
                unsigned int offset = lane_offset + kLoadRows * i * stride_bytes;
                asm volatile("" : "+v"(offset));
                if (fetch)
                    __builtin_amdgcn_global_load_lds(reinterpret_cast<const unsigned int*>(base + offset),
                                                     (lds_words_t)(stage + (kLoadRows * i + 4u * wave) * kRowBytes), 16, 0, 0);
            }
        } else {
#pragma unroll
            for (unsigned int i = 0; i < kLoads; ++i) {
                unsigned int key = tile * kKeyTile + kLoadRows * i + load_row;
                key = key < key_len ? key : key_len - 1;
                if (fetch)
                    __builtin_amdgcn_global_load_lds(reinterpret_cast<const unsigned int*>(rows + (key * stride_bytes + chunk)),
                                                 (lds_words_t)(stage + (kLoadRows * i + 4u * wave) * kRowBytes), 16, 0, 0);
            }
        }
    };
    auto load_keys = [&](unsigned int tile, unsigned char* stage) __attribute__((always_inline)) {
        load_tile(k_bytes, key_stride_bytes, key_lane, key_chunk, key_lane_live, tile, stage);
    };
    auto load_values = [&](unsigned int tile, unsigned char* stage) __attribute__((always_inline)) {
        load_tile(v_bytes, value_stride_bytes, value_lane, value_chunk, value_lane_live, tile, stage);
    };

    RowState state;
    reset(state);
    if (a.sinks != nullptr && split == 0) {
        // The head's sink: a score that is always there and weighs no value.  The row starts with it as its reference
        // point and a sum of one (held by one of the row's two lanes).
        const uint16_t bits = a.sinks[head];
        float sink;
        if constexpr (std::is_same_v<Half, F16>) sink = static_cast<float>(__builtin_bit_cast(_Float16, bits));
        else sink = __builtin_bit_cast(float, static_cast<unsigned int>(bits) << 16);
        state.reference = sink * kLog2e;
        state.running_sum = hi == 0 && state.reference != -INFINITY ? 1.0f : 0.0f;
    }
    const ReadOffsets offsets = read_offsets(lane);

    if (first_tile < tiles) {
        load_keys(first_tile, lds);
        load_values(first_tile, lds + kValueBase);
    }
    if (first_tile + 1 < tiles) load_keys(first_tile + 1, lds + kTileBytes);
    loads_landed();
    __syncthreads();

    // Folds block `block` (scores in `s`, values at `values`) with the mask's edges applied.
    auto fold = [&](unsigned int block, f32x16_t& s, const unsigned char* values) __attribute__((always_inline)) {
        const unsigned int key0 = block * 32u;
        if constexpr (OPTIONS) {
            // Scores in their final units (base-two logits): scaled, capped (singe/src/backend/cpu/normalization/
            // attention.rs:255-262: the cap, then the mask), the mask added.  Register r of lane (query, hi) is key
            // key0 + 8 (r / 4) + 4 hi + (r % 4).
            const bool capped = a.cap_log2e != 0.0f;
            const float to_units = capped ? a.cap_scale : factor;
            const uint16_t* mask_row = nullptr;
            if (a.mask != nullptr)
                mask_row = a.mask + batch * a.mask_strides[0] + head * a.mask_strides[1] + static_cast<size_t>(query_valid ? my_query : 0) * a.mask_strides[2];
            // The lane's keys come in four runs of four; a run inside the keys is one 8-byte load when the host found
            // every mask row to start on an 8-byte boundary with its keys side by side.
            uint16_t mask_bits[16];
            if (mask_row != nullptr) {
#pragma unroll
                for (int run = 0; run < 4; ++run) {
                    const unsigned int key = key0 + 8u * run + 4u * hi;
                    if (a.mask_packed && key + 3u < key_len) {
                        const uint2 four = *reinterpret_cast<const uint2*>(mask_row + key);
                        mask_bits[4 * run + 0] = static_cast<uint16_t>(four.x);
                        mask_bits[4 * run + 1] = static_cast<uint16_t>(four.x >> 16);
                        mask_bits[4 * run + 2] = static_cast<uint16_t>(four.y);
                        mask_bits[4 * run + 3] = static_cast<uint16_t>(four.y >> 16);
                    } else {
#pragma unroll
                        for (int i = 0; i < 4; ++i)
                            mask_bits[4 * run + i] = mask_row[static_cast<size_t>(key + i < key_len ? key + i : 0) * a.mask_strides[3]];
                    }
                }
            }
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                float x = s[r] * to_units;
                if (capped) x = fast_tanh(x) * a.cap_log2e;
                if (mask_row != nullptr) {
                    float extra;
                    if constexpr (std::is_same_v<Half, F16>) extra = static_cast<float>(__builtin_bit_cast(_Float16, mask_bits[r]));
                    else extra = __builtin_bit_cast(float, static_cast<unsigned int>(mask_bits[r]) << 16);
                    x += extra * kLog2e;
                }
                s[r] = x;
            }
            const bool windowed = a.window >= 0;
            const unsigned long long window = windowed ? static_cast<unsigned long long>(a.window) : 0ull;
            const float shift = begin_block(state, s, hi, 1.0f, true, [&](unsigned int key_in_block) {
                const unsigned int key = key0 + key_in_block;
                return (CAUSAL && key > my_query) || key >= key_len || (windowed && key + window <= my_query);
            });
            finish_block<false>(half, state, s, 1.0f, shift, values, offsets, s, q, values);
            return;
        }
        const bool edge = (CAUSAL && key0 + 31u > first_row) || key0 + 32u > key_len;
        const float shift = begin_block(state, s, hi, factor, edge, [&](unsigned int key_in_block) {
            const unsigned int key = key0 + key_in_block;
            return (CAUSAL && key > my_query) || key >= key_len;
        });
        finish_block<false>(half, state, s, factor, shift, values, offsets, s, q, values);
    };

    // One block ahead: while block b is folded, the scores of block b + 1 are computed; `scores` holds
    // those of the block that is folded next.
    f32x16_t scores;
    if (2u * first_tile < wave_blocks) score_block(half, scores, q, lds, offsets);
    unsigned int key_stage = 0, value_stage = 0;  // tile % 3, tile % 2
    // Names the stages a tile's iteration works on and loads into.  Everyone left the stages that held K of
    // tile - 1 and V of tile - 1 at the last barrier.
    auto enter = [&]() __attribute__((always_inline)) {
        const unsigned int next_key_stage = key_stage + 1 == kKeyStages ? 0 : key_stage + 1;
        const unsigned int spare_key_stage = next_key_stage + 1 == kKeyStages ? 0 : next_key_stage + 1;
        TileStages stages;
        stages.keys = lds + key_stage * kTileBytes;
        stages.next_keys = lds + next_key_stage * kTileBytes;
        stages.values = lds + kValueBase + value_stage * kTileBytes;
        stages.key_dest = lds + spare_key_stage * kTileBytes;
        stages.value_dest = lds + kValueBase + (value_stage ^ 1u) * kTileBytes;
        key_stage = next_key_stage;
        value_stage ^= 1u;
        return stages;
    };
    // Hands the stages on: this wave's loads have landed, and everyone has finished reading.
    auto leave = [&]() __attribute__((always_inline)) {
        loads_landed();
        __syncthreads();
    };

    // Tiles with no mask to apply and another block to come after them: straight-line code.  They come
    // first for every wave (the mask's edge and the end of the keys are the last tiles a wave works on).
    unsigned int interior_tiles = wave_blocks > 2 ? (wave_blocks - 1) / 2 : 0;  // tiles t with 2 t + 2 < wave_blocks
    if (CAUSAL) {
        const unsigned int unmasked = (first_row + 1) / kKeyTile;  // tiles t with 64 t + 63 <= first_row
        interior_tiles = interior_tiles < unmasked ? interior_tiles : unmasked;
    }
    {
        const unsigned int whole = key_len / kKeyTile;  // tiles t with 64 t + 64 <= key_len
        interior_tiles = interior_tiles < whole ? interior_tiles : whole;
    }
    // With options, a cap and a window leave the unmasked tiles their straight-line path (the cap is applied to each
    // block's scores before they are folded; the tiles that reach back past the window of the wave's last row come
    // first and take the masked path); an additive mask sends every tile down the masked one (its words held a tile
    // ahead in registers made the straight-line tiles spill, and the reloads wait for the K and V loads in flight).
    unsigned int inner_begin = first_tile;
    if (OPTIONS) {
        if (a.mask != nullptr) interior_tiles = 0;
        if (a.window >= 0) {
            // Tile t lies inside every row's window when 64 t + window > first_row + 31.
            const unsigned long long past = static_cast<unsigned long long>(first_row) + 32u, window = static_cast<unsigned long long>(a.window);
            if (past > window) {
                const unsigned long long whole = (past - window + kKeyTile - 1) / kKeyTile;
                inner_begin = whole < tiles ? static_cast<unsigned int>(whole) : tiles;
            }
            inner_begin = inner_begin > first_tile ? inner_begin : first_tile;
        }
    }
    unsigned int tile = first_tile;
    uint4 operand[kSteps];
    auto issue = [&](unsigned char* key_dest, unsigned char* value_dest) __attribute__((always_inline)) {
        if (tile + 2 < tiles) load_keys(tile + 2, key_dest);
        if (tile + 1 < tiles) load_values(tile + 1, value_dest);
    };
    if constexpr (OPTIONS) {
        for (; tile < inner_begin && tile < interior_tiles; ++tile) {
            const TileStages stages = enter();
            fold_edge_tile(half, scores, q, offsets, 2u * tile, wave_blocks, stages.keys, stages.next_keys, stages.values, stages.key_dest,
                           stages.value_dest, issue, fold);
            leave();
        }
    }
    if (kDenseOperandsAhead && tile < interior_tiles) read_key_operands(operand, lds + key_stage * kTileBytes + kBlockBytes, offsets);
    if constexpr (OPTIONS) {
        if (a.cap_log2e != 0.0f) {
            const float cap_scale = a.cap_scale, cap_log2e = a.cap_log2e;
            for (; tile < interior_tiles; ++tile) {
                const TileStages stages = enter();
                fold_interior_tile<kDenseOperandsAhead>(half, state, scores, operand, q, offsets, hi, 1.0f, stages.keys, stages.next_keys, stages.values,
                                                        stages.key_dest, stages.value_dest, issue, [&](f32x16_t& s, unsigned int) {
#pragma unroll
                                                            for (int r = 0; r < 16; ++r) s[r] = fast_tanh(s[r] * cap_scale) * cap_log2e;
                                                        });
                leave();
            }
        }
    }
    for (; tile < interior_tiles; ++tile) {
        const TileStages stages = enter();
        fold_interior_tile<kDenseOperandsAhead>(half, state, scores, operand, q, offsets, hi, factor, stages.keys, stages.next_keys, stages.values, stages.key_dest,
                           stages.value_dest, issue);
        leave();
    }
    // Tiles on the mask's edge and the last ones (and, for waves that have run out of blocks, the
    // workgroup's remaining loads and barriers).
    for (; tile < tiles; ++tile) {
        const TileStages stages = enter();
        fold_edge_tile(half, scores, q, offsets, 2u * tile, wave_blocks, stages.keys, stages.next_keys, stages.values, stages.key_dest,
                       stages.value_dest, issue, fold);
        leave();
    }

    // Normalise and store.  Lane (query, hi) holds dims 32db + 8(r / 4) + 4hi + (r % 4).
    const float sum = swap32_sum(state.running_sum);
    const float inverse = sum > 0.0f ? 1.0f / sum : 0.0f;
    if (query_valid && a.splits > 1) {
        const size_t flat = (static_cast<size_t>(batch) * a.heads + head) * a.query_len + my_query;
        const size_t slot = static_cast<size_t>(split) * a.batch * a.heads * a.query_len + flat;
        float* row = a.partial_out + slot * kHeadDim;
#pragma unroll
        for (int db = 0; db < kDimBlocks; ++db)
#pragma unroll
            for (int quad = 0; quad < 4; ++quad)
                if (32 * db + 8 * quad < kHeadDim)
                    *reinterpret_cast<float4*>(row + 32 * db + 8 * quad + 4 * hi) =
                    make_float4(state.out[db][4 * quad + 0] * inverse, state.out[db][4 * quad + 1] * inverse,
                                state.out[db][4 * quad + 2] * inverse, state.out[db][4 * quad + 3] * inverse);
        if (hi == 0) a.partial_lse[slot] = sum > 0.0f ? state.reference + fast_log2(sum) : -INFINITY;
    } else if (query_valid) {
        uint16_t* row = a.out + batch * a.output_batch_stride + static_cast<size_t>(my_query) * a.output_sequence_stride +
                        head * a.output_head_stride;
#pragma unroll
        for (int db = 0; db < kDimBlocks; ++db)
#pragma unroll
            for (int quad = 0; quad < 4; ++quad) {
                if (32 * db + 8 * quad >= kHeadDim) continue;
                uint2 packed;
                packed.x = pack_pair(half, state.out[db][4 * quad + 0] * inverse, state.out[db][4 * quad + 1] * inverse);
                packed.y = pack_pair(half, state.out[db][4 * quad + 2] * inverse, state.out[db][4 * quad + 3] * inverse);
                *reinterpret_cast<uint2*>(row + 32 * db + 8 * quad + 4 * hi) = packed;
            }
        if (a.lse != nullptr && hi == 0)
            a.lse[(static_cast<size_t>(batch) * a.heads + head) * a.query_len + my_query] =
                sum > 0.0f ? (state.reference + fast_log2(sum)) * kLn2 : -INFINITY;
    }
}

// Workgroup id -> (batch * heads + head, pair of query tiles): see the header comment.
template <bool CAUSAL, class Half, int WAVES, bool OPTIONS = false>
SINGE_DEVICE void fmha_prefill_body(const PrefillArgs& a, unsigned char* lds) {
    const unsigned int xcd = blockIdx.x & 7u;
    unsigned int within = blockIdx.x >> 3;
    const unsigned int split = within % a.splits;  // the shares of a query tile are neighbours
    within /= a.splits;
    const unsigned int pairs = (a.query_tiles + 1u) / 2u;
    const unsigned int bh = (within / pairs) * 8u + xcd;
    if (bh >= a.batch * (a.packed_heads != 0 ? a.kv_heads : a.heads)) return;
    const unsigned int light = within % pairs, heavy = a.query_tiles - 1u - light;
    fmha_prefill_tile<CAUSAL, Half, WAVES, OPTIONS>(a, lds, bh, heavy, split);
    if (light != heavy) fmha_prefill_tile<CAUSAL, Half, WAVES, OPTIONS>(a, lds, bh, light, split);
}

// Merges the key splits of a row: each share's rows weigh 2^(lse - largest) over the sum of those (the reference's
// combine, singe/src/backend/cuda/kernel_plan/source/attention.rs:588-654).  A wave per (batch, head, query) row; a lane
// takes two of the row's values.
template <class Half>
SINGE_DEVICE void fmha_prefill_combine_body(const PrefillArgs& a) {
    const unsigned int lane = threadIdx.x & 63u;
    const size_t rows_total = static_cast<size_t>(a.batch) * a.heads * a.query_len;
    const size_t flat = static_cast<size_t>(blockIdx.x) * 4u + (threadIdx.x >> 6);
    if (flat >= rows_total) return;
    const unsigned int query = static_cast<unsigned int>(flat % a.query_len);
    const unsigned int head = static_cast<unsigned int>((flat / a.query_len) % a.heads);
    const unsigned int batch = static_cast<unsigned int>(flat / (static_cast<size_t>(a.query_len) * a.heads));
    const float mine = lane < a.splits ? a.partial_lse[lane * rows_total + flat] : -INFINITY;
    float largest = mine;
#pragma unroll
    for (int step = 32; step > 0; step >>= 1) largest = fmaxf(largest, __shfl_xor(largest, step, 64));
    const float weight = mine == -INFINITY ? 0.0f : fast_exp2(mine - largest);  // an empty share weighs nothing
    float total = weight;
#pragma unroll
    for (int step = 32; step > 0; step >>= 1) total += __shfl_xor(total, step, 64);
    const bool holds_values = 2u * lane < static_cast<unsigned int>(kHeadDim);
    float2 merged = make_float2(0.0f, 0.0f);
    // Four shares' values are asked for together; what a share that weighs nothing holds is not used.
    const float* mine_of = a.partial_out + flat * kHeadDim + (holds_values ? 2u * lane : 0u);
    const size_t share_stride = rows_total * kHeadDim;
    auto fold = [&](unsigned int s, const float2& part) __attribute__((always_inline)) {
        const float w = __shfl(weight, s, 64);
        merged.x = w == 0.0f ? merged.x : fmaf(w, part.x, merged.x);
        merged.y = w == 0.0f ? merged.y : fmaf(w, part.y, merged.y);
    };
    unsigned int s = 0;
    for (; s + 4 <= a.splits; s += 4) {
        float2 part[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) part[i] = *reinterpret_cast<const float2*>(mine_of + (s + i) * share_stride);
#pragma unroll
        for (int i = 0; i < 4; ++i) fold(s + i, part[i]);
    }
    for (; s < a.splits; ++s) fold(s, *reinterpret_cast<const float2*>(mine_of + s * share_stride));
    const float inverse = total > 0.0f ? 1.0f / total : 0.0f;
    uint16_t* row = a.out + batch * a.output_batch_stride + static_cast<size_t>(query) * a.output_sequence_stride + head * a.output_head_stride;
    if (holds_values) reinterpret_cast<unsigned int*>(row)[lane] = pack_pair(Half{}, merged.x * inverse, merged.y * inverse);
    if (a.lse != nullptr && lane == 0) a.lse[flat] = total > 0.0f ? (largest + fast_log2(total)) * kLn2 : -INFINITY;
}

}  // namespace

#define SINGE_FMHA_PREFILL_KERNEL(NAME, CAUSAL, HALF)                                              \
    extern "C" __global__ __launch_bounds__(64 * kDenseWaves, 8 / kDenseWaves) void NAME(PrefillArgs args) { \
        __shared__ __attribute__((aligned(1024))) unsigned char prefill_lds[kStagedLdsBytes];        \
        fmha_prefill_body<CAUSAL, prefill::HALF, kDenseWaves>(args, prefill_lds);                   \
    }

#define SINGE_FMHA_PREFILL_OPTIONS_KERNEL(NAME, CAUSAL, HALF)                                      \
    extern "C" __global__ __launch_bounds__(64 * kDenseWaves, 8 / kDenseWaves) void NAME(PrefillArgs args) { \
        __shared__ __attribute__((aligned(1024))) unsigned char prefill_lds[kStagedLdsBytes];        \
        fmha_prefill_body<CAUSAL, prefill::HALF, kDenseWaves, true>(args, prefill_lds);             \
    }

// Names carry the head dimension of the build: singe_fmha_prefill_bf16_d128_causal, ..._d64_causal.
#define SINGE_PASTE3_(a, b, c) a##b##c
#define SINGE_PASTE3(a, b, c) SINGE_PASTE3_(a, b, c)
#define SINGE_PREFILL_NAME(TYPE, TAIL) SINGE_PASTE3(singe_fmha_prefill_##TYPE##_d, SINGE_HEAD_DIM, TAIL)

SINGE_FMHA_PREFILL_OPTIONS_KERNEL(SINGE_PREFILL_NAME(bf16, _causal_options), true, Bf16)
SINGE_FMHA_PREFILL_OPTIONS_KERNEL(SINGE_PREFILL_NAME(bf16, _full_options), false, Bf16)
SINGE_FMHA_PREFILL_OPTIONS_KERNEL(SINGE_PREFILL_NAME(f16, _causal_options), true, F16)
SINGE_FMHA_PREFILL_OPTIONS_KERNEL(SINGE_PREFILL_NAME(f16, _full_options), false, F16)
SINGE_FMHA_PREFILL_KERNEL(SINGE_PREFILL_NAME(bf16, _causal), true, Bf16)
SINGE_FMHA_PREFILL_KERNEL(SINGE_PREFILL_NAME(bf16, _full), false, Bf16)
SINGE_FMHA_PREFILL_KERNEL(SINGE_PREFILL_NAME(f16, _causal), true, F16)
SINGE_FMHA_PREFILL_KERNEL(SINGE_PREFILL_NAME(f16, _full), false, F16)
extern "C" __global__ __launch_bounds__(256) void SINGE_PREFILL_NAME(bf16, _combine)(PrefillArgs args) { fmha_prefill_combine_body<prefill::Bf16>(args); }
extern "C" __global__ __launch_bounds__(256) void SINGE_PREFILL_NAME(f16, _combine)(PrefillArgs args) { fmha_prefill_combine_body<prefill::F16>(args); }
