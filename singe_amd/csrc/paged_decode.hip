// Paged-attention decode over a block-table KV cache, one query token per sequence
// (the GPU counterpart of singe-kernel/src/cpu/attention.rs:1172-1246, replacing the cuTile kernels
// of singe-kernel/src/cuda/cutile/kernel/attention/local.rs:9349-...).
//
// Layouts (fixed by the reference API): query/out [batch, heads, 128] bf16; caches
// [blocks, block_size, kv_heads, 128], bf16 or fp8 e4m3 with one f32 scale per (block, kv head);
// block_table [batch, stride] u32; actual_seq_lens [batch] i32.
//
// Decode reads every KV byte once and does a few flop per byte, so it is bound by HBM bandwidth and,
// at these sizes (tens of microseconds), by how evenly and how early the chip is filled.
//
// Work split.  The keys of all sequences form one flat list of 32-key tiles (per-sequence tile counts,
// prefix-summed in LDS by every workgroup).  The list is cut into `workers` equal ranges; a wave is
// one worker for one kv head, so every wave does the same amount of work in a single round and the
// waves of a workgroup walk the same cache blocks for neighbouring kv heads at the same time (one
// 32 KiB block is fetched by one CU in one go).  A range that crosses a sequence boundary yields one
// partial row per sequence; partial row of (worker v, sequence b) lives in scratch slot v + b, which is
// unique because both grow along the list.  singe_paged_decode_combine folds a sequence's slots as
// splitk_reduce_f32 does (cpu/attention.rs:2157-2193).
//
// Inner loop, per 32-key tile, all on the matrix cores:
//   scores   S^T[key, head] = K[key, :] . Q[head, :]  (v_mfma_f32_16x16x32_bf16, fp32 accumulate).  Four
//            query heads share one MFMA, each repeated over 4 of the 16 columns.
//   softmax  online, base two; the tile maximum is shared by the wave (two v_permlane swaps), the
//            running sum stays per lane until the row is flushed.
//   values   V rows are loaded as whole rows (16 lanes x 16 B, the coalesced layout) and used as the
//            MFMA A operand exactly as loaded: for v_mfma_f32_16x16x16_bf16, A[chunk t][(g, e)] =
//            V[key 4g + i][8t + 4half + e].  The B operand is the probability of (head, key 4g + i)
//            placed at position e of column (head, e), zero elsewhere, so C[t][(head, e)] accumulates
//            O[head][8t + 4half + e].  That spends 3/4 of the MFMA's multiplies on zeros, which is free
//            here, and needs no transpose of V, no unpacking and no cross-lane traffic.  Probabilities
//            are rounded to bf16 for this product and summed unrounded, as the reference's tensor-core
//            kernel does (singe/src/backend/cuda/kernel_plan/source/tensor_core.rs:162-183).
//
// fp8 caches are widened to bf16 in registers on their way into the MFMA operands.  In the exact mode
// every element becomes bf16_rne(f8e4m3_value(code) * scale) first (the value the CPU path reads after
// dequantising the cache); in the relaxed mode the codes are widened exactly and the block's scale is
// applied to the 32 scores / probabilities of the tile instead, which saves the multiply and half of the
// conversions.  They take a different inner loop (WIDE below): an fp8 cache halves the bytes per key, so
// the one-hot form's spare multiplies and repeated exponentials are no longer free.
#include "common.hip.h"
#include "kernel_args.h"

namespace {

// The head dimension a build of these kernels is for: the source is compiled once per value (128, and the other
// multiples of 16 with -DSINGE_HEAD_DIM=, bf16 and f16 caches only), each into its own part of the code object.  Below
// 128 the register layouts stay as they are and only their front is live: at 64 a key's row is eight 16-byte chunks,
// so lanes t >= 8 fetch no values and the score products run over two 32-dim steps instead of four; at 32 a row is
// four chunks and there is one step; where the last step is half a step (16, 48, 80, 112) its upper sixteen
// dimensions are zeros in both operands.
#ifndef SINGE_HEAD_DIM
#define SINGE_HEAD_DIM 128
#endif
constexpr int kDim = SINGE_HEAD_DIM;
static_assert(kDim % 16 == 0 && kDim >= 16 && kDim <= 128, "head dimensions the decode kernels are built for");
constexpr int kDimSteps = (kDim + 31) / 32;  // score products per 16 keys
constexpr int kTile = 32;
constexpr float kReferenceLag = 6.0f;  // doublings a softmax reference point may lag the largest score seen

// One 32-key tile in registers, bf16 cache.  K and V are fetched the same way, as whole rows (16 lanes x 16 bytes, the
// coalesced layout: fetched in the matrix operand's layout, where neighbouring lanes read different rows, K alone
// held the kernel to 5.6 TB/s); K is turned into its operand layout through a per-wave LDS buffer when the tile is folded.
struct KeyTileBf16 {
    uint4 k[2][4];      // [16-key half][i]: lane (g, t) holds key 4g + i, dims 8t .. 8t + 8
    uint4 v[2][4];      // the same of the values
    unsigned int live;  // bit (half * 4 + i): key half*16 + 4g + i takes part in the softmax
};

// One 32-key tile in registers, fp8 cache: the same keys and dims per lane, one byte per element.
struct KeyTileFp8 {
    uint4 k[2][2];        // lane (g, t): key t, dims 32g + 16x .. +16
    uint2 v[2][4];        // lane (g, t): key 4g + i, dims 8t .. 8t + 8
    float key_scale[2];   // scale of this lane's key t (exact mode)
    float row_key_scale[2][4];    // scale of key 4g + i (relaxed mode: applied to its score)
    float row_value_scale[2][4];  // scale of key 4g + i's values
    unsigned int live;
};

// Element offset of (block, slot, kv_head, 0) in a [blocks, block_size, kv_heads, 128] cache.
SINGE_DEVICE size_t cache_row(unsigned int block, unsigned int slot, unsigned int block_size,
                              unsigned int kv_heads, unsigned int kv_head) {
    return ((static_cast<size_t>(block) * block_size + slot) * kv_heads + kv_head) * kDim;
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

// Where the keys of one 16-key half live: the cache row of this lane's K key (t) and of its four V
// keys (4g + i), whether each V key is live, and the blocks they came from (for fp8 scales).  Keys
// at or past `end`, and keys whose table entry is not a cache block, resolve to an in-range row and
// are dead, so nothing is read out of bounds and no dead row can carry a NaN into the sums.
struct HalfRows {
    unsigned int cache_lane;  // lane of the entry cache that holds this half's block (aligned path)
    size_t key_row;
    size_t value_row[4];
    unsigned int key_block;
    unsigned int value_block[4];
    unsigned int live;  // bit i
};

// 64 consecutive block-table entries of one sequence, one per lane, fetched with a single vector
// load (plus, for fp8 caches, the two scales of each block).  Tiles then pick their entry out of a
// register with v_readlane instead of paying a dependent scalar-load round trip per 16 keys.
struct EntryCache {
    unsigned int sequence = 0xffffffffu;
    unsigned int first_entry = 0;
    unsigned int blocks = 0;      // lane l: table[sequence][first_entry + l]
    float key_scales = 0.0f;      // lane l: scale of that block for this wave's kv head
    float value_scales = 0.0f;
};

template <bool FP8>
SINGE_DEVICE void fill_entries(EntryCache& cache, const DecodeArgs& a, unsigned int sequence, size_t row_base, unsigned int first_entry,
                               unsigned int kv_head, unsigned int lane) {
    cache.sequence = sequence;
    cache.first_entry = first_entry;
    const unsigned int index = first_entry + lane;
    unsigned int block = 0xffffffffu;
    // (rows of their own lengths: the table holds block_table_batch_stride entries in all)
    if (a.row_starts != nullptr ? row_base + index < a.block_table_batch_stride : index < a.block_table_batch_stride)
        block = a.block_table[row_base + index];
    cache.blocks = block;
    if constexpr (FP8) {
        const size_t at = static_cast<size_t>(block < a.physical_blocks ? block : 0) * a.kv_heads + kv_head;
        cache.key_scales = a.key_scales[at];
        cache.value_scales = a.value_scales[at];
    }
}

// LEAN: whole halves take a path of their own (measured: faster for the fp8 kernels, whose vector unit is what bounds
// them, and for the four-head bf16 / f16 kernels at head_dim 128; slower where the extra code costs the wide bf16 form its
// last free registers, and at the other head dimensions).
template <bool ALIGNED16, bool LEAN>
SINGE_DEVICE HalfRows locate_half(const DecodeArgs& a, const unsigned int* table_row, const EntryCache& cache,
                                  unsigned int base, unsigned int end, unsigned int kv_head, unsigned int g,
                                  unsigned int t) {
    HalfRows rows;
    rows.live = 0;
    if constexpr (ALIGNED16) {
        // block_size is a multiple of 16, so the 16 keys share one table entry.
        if (LEAN && base + 16u <= end) {
            // All sixteen keys are the sequence's (every half but a sequence's last one or two): the block and the row of
            // its first key are the same for every lane, and a lane's rows lie whole slots behind it; no key needs a
            // test of its own.  (The statement below keeps this a branch: as selects, the tests of the general path
            // would run for every half.)
            asm volatile("");
            unsigned int entry, slot0;
            split_key(a, base, entry, slot0);
            rows.cache_lane = entry - cache.first_entry;
            const unsigned int block = __builtin_amdgcn_readlane(cache.blocks, rows.cache_lane);
            const bool known = block < a.physical_blocks;
            const unsigned int safe = known ? block : 0;
            const size_t first_row = cache_row(safe, slot0, a.block_size, a.kv_heads, kv_head);
            const unsigned int slot_elements = a.kv_heads * static_cast<unsigned int>(kDim);
            rows.key_block = safe;
            rows.key_row = first_row + t * slot_elements;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                rows.value_block[i] = safe;
                rows.value_row[i] = first_row + (4 * g + i) * slot_elements;
            }
            rows.live = known ? 0xfu : 0u;
            return rows;
        }
        // A half that holds the sequence's last key, or lies wholly past it and re-reads the 16-key span that holds it.
        unsigned int last_entry, last_slot, entry, slot0;
        split_key(a, end - 1, last_entry, last_slot);
        split_key(a, base < end ? base : ((end - 1) & ~15u), entry, slot0);
        rows.cache_lane = entry - cache.first_entry;
        const unsigned int block = __builtin_amdgcn_readlane(cache.blocks, rows.cache_lane);
        const bool known = block < a.physical_blocks;
        const unsigned int safe = known ? block : 0;
        rows.key_block = safe;
        rows.key_row = cache_row(safe, base + t < end ? slot0 + t : last_slot, a.block_size, a.kv_heads, kv_head);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const bool inside = base + 4 * g + i < end;
            rows.value_block[i] = safe;
            rows.value_row[i] = cache_row(safe, inside ? slot0 + 4 * g + i : last_slot, a.block_size, a.kv_heads, kv_head);
            if (inside && known) rows.live |= 1u << i;
        }
    } else {
        // Any block size: every lane looks up the table entry of its own keys.
        {
            unsigned int entry, slot;
            split_key(a, base + t < end ? base + t : end - 1, entry, slot);
            unsigned int block = table_row[entry];
            block = block < a.physical_blocks ? block : 0;
            rows.key_block = block;
            rows.key_row = cache_row(block, slot, a.block_size, a.kv_heads, kv_head);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const unsigned int wanted = base + 4 * g + i;
            const bool inside = wanted < end;
            unsigned int entry, slot;
            split_key(a, inside ? wanted : end - 1, entry, slot);
            unsigned int block = table_row[entry];
            const bool known = block < a.physical_blocks;
            block = known ? block : 0;
            rows.value_block[i] = block;
            rows.value_row[i] = cache_row(block, slot, a.block_size, a.kv_heads, kv_head);
            if (inside && known) rows.live |= 1u << i;
        }
    }
    return rows;
}

// Loads the 32 keys from `first` (a multiple of 32) of a sequence of `end` > first keys.
template <bool ALIGNED16, bool LEAN>
SINGE_DEVICE void load_tile(KeyTileBf16& tile, const DecodeArgs& a, const unsigned int* table_row, const EntryCache& cache,
                            unsigned int first, unsigned int end, unsigned int kv_head, unsigned int g,
                            unsigned int t) {
    tile.live = 0;
    const uint16_t* key_cache = static_cast<const uint16_t*>(a.key_cache);
    const uint16_t* value_cache = static_cast<const uint16_t*>(a.value_cache);
#pragma unroll
    for (int half = 0; half < 2; ++half) {
        const HalfRows rows = locate_half<ALIGNED16, LEAN>(a, table_row, cache, first + half * 16, end, kv_head, g, t);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            if (kDim == 128 || 8 * t < static_cast<unsigned int>(kDim)) {
                tile.k[half][i] = stream_load_16(key_cache + rows.value_row[i] + 8 * t);
                tile.v[half][i] = stream_load_16(value_cache + rows.value_row[i] + 8 * t);
            } else {
                tile.k[half][i] = make_uint4(0, 0, 0, 0);
                tile.v[half][i] = make_uint4(0, 0, 0, 0);
            }
        }
        tile.live |= rows.live << (half * 4);
    }
}

template <bool ALIGNED16, bool LEAN>
SINGE_DEVICE void load_tile(KeyTileFp8& tile, const DecodeArgs& a, const unsigned int* table_row, const EntryCache& cache,
                            unsigned int first, unsigned int end, unsigned int kv_head, unsigned int g,
                            unsigned int t) {
    tile.live = 0;
    const uint8_t* key_cache = static_cast<const uint8_t*>(a.key_cache);
    const uint8_t* value_cache = static_cast<const uint8_t*>(a.value_cache);
#pragma unroll
    for (int half = 0; half < 2; ++half) {
        const HalfRows rows = locate_half<ALIGNED16, LEAN>(a, table_row, cache, first + half * 16, end, kv_head, g, t);
        const uint8_t* kp = key_cache + rows.key_row + 32 * g;
        tile.k[half][0] = *reinterpret_cast<const uint4*>(kp);
        tile.k[half][1] = *reinterpret_cast<const uint4*>(kp + 16);
#pragma unroll
        for (int i = 0; i < 4; ++i) tile.v[half][i] = stream_load_8(value_cache + rows.value_row[i] + 8 * t);
        if constexpr (ALIGNED16) {
            // One block per half: its two scales come out of the entry cache.
            const float ks = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, cache.key_scales), rows.cache_lane));
            const float vs = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, cache.value_scales), rows.cache_lane));
            tile.key_scale[half] = ks;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                tile.row_key_scale[half][i] = ks;
                tile.row_value_scale[half][i] = vs;
            }
        } else {
            tile.key_scale[half] = a.key_scales[static_cast<size_t>(rows.key_block) * a.kv_heads + kv_head];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const size_t at = static_cast<size_t>(rows.value_block[i]) * a.kv_heads + kv_head;
                tile.row_key_scale[half][i] = a.key_scales[at];
                tile.row_value_scale[half][i] = a.value_scales[at];
            }
        }
        tile.live |= rows.live << (half * 4);
    }
}

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
typedef short i16x4_t __attribute__((ext_vector_type(4)));

SINGE_DEVICE unsigned int bf16_pair(float lo, float hi) {
    f32x2_t both = {lo, hi};
    return __builtin_bit_cast(unsigned int, __builtin_convertvector(both, bf16x2_t));
}

// bf16(value) in both halves of a dword (one v_cvt_pk_bf16_f32, round to nearest even).
SINGE_DEVICE unsigned int bf16_twice(float value) { return bf16_pair(value, value); }

// The same value rounded to the cache's 16-bit type in both halves of a dword, and the two MFMA shapes, for bf16
// (the default) or f16 operands.
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
typedef _Float16 f16x4_t __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));

template <bool F16>
SINGE_DEVICE unsigned int half_twice(float value) {
    if constexpr (F16) {
        const f32x2_t both = {value, value};
        return __builtin_bit_cast(unsigned int, __builtin_convertvector(both, f16x2_t));
    } else {
        return bf16_twice(value);
    }
}

// Two values rounded to the cache's 16-bit type, low half first.
template <bool F16>
SINGE_DEVICE unsigned int half_pair(float lo, float hi) {
    if constexpr (F16) {
        const f32x2_t both = {lo, hi};
        return __builtin_bit_cast(unsigned int, __builtin_convertvector(both, f16x2_t));
    } else {
        return bf16_pair(lo, hi);
    }
}

template <bool F16>
SINGE_DEVICE f32x4_t score_mma(uint4 keys, bf16x8_t query, f32x4_t acc) {
    if constexpr (F16)
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, keys), __builtin_bit_cast(f16x8_t, query), acc, 0, 0, 0);
    else
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, keys), query, acc, 0, 0, 0);
}

template <bool F16>
SINGE_DEVICE f32x4_t value_mma(uint2 values, uint2 weights, f32x4_t acc) {
    if constexpr (F16)
        return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(f16x4_t, values), __builtin_bit_cast(f16x4_t, weights), acc, 0, 0, 0);
    else
        return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(i16x4_t, values), __builtin_bit_cast(i16x4_t, weights), acc, 0, 0, 0);
}

// Eight fp8 e4m3 codes -> eight bf16 values.  EXACT: bf16_rne(value(code) * scale), the value the CPU path
// reads after dequantising the cache.  Otherwise the codes are widened as they are (every e4m3 value is a
// bf16 value), which v_cvt_scalef32_pk_bf16_fp8 does for two codes at a time; its scale operand only
// carries a power of two, so it cannot stand in for the multiply above.
template <bool EXACT>
SINGE_DEVICE uint4 widen_fp8x8(unsigned int low, unsigned int high, float scale) {
    if constexpr (EXACT) {
        const f32x2_t a = __builtin_amdgcn_cvt_pk_f32_fp8(low, false), b = __builtin_amdgcn_cvt_pk_f32_fp8(low, true);
        const f32x2_t c = __builtin_amdgcn_cvt_pk_f32_fp8(high, false), d = __builtin_amdgcn_cvt_pk_f32_fp8(high, true);
        return make_uint4(bf16_pair(a[0] * scale, a[1] * scale), bf16_pair(b[0] * scale, b[1] * scale),
                          bf16_pair(c[0] * scale, c[1] * scale), bf16_pair(d[0] * scale, d[1] * scale));
    } else {
        return make_uint4(__builtin_bit_cast(unsigned int, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(low, 1.0f, false)),
                          __builtin_bit_cast(unsigned int, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(low, 1.0f, true)),
                          __builtin_bit_cast(unsigned int, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(high, 1.0f, false)),
                          __builtin_bit_cast(unsigned int, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(high, 1.0f, true)));
    }
}

// Per-wave softmax state of one group of four query heads.
struct GroupState {
    f32x4_t acc[2];     // [dims 8t..8t+3 | 8t+4..8t+7]: C[t][(head, e)], lane (g, n) holds chunks t = 4g .. 4g+3
    float running_max;  // log2 units, equal in all lanes that hold the same head
    float running_sum;  // of this lane's keys only
};

// Rows of a wave's private V staging buffer in LDS (WIDE): 256 bytes of bf16 plus 16 bytes of padding, so
// the sixteen rows a transposing read touches fall into all banks twice over, which is the best 512
// bytes can do.
constexpr int kStagedRowBytes = 272;
constexpr int kStagedTileBytes = kTile * kStagedRowBytes;
// A wave's K staging buffer (bf16 / f16 caches): 32 rows of 256 bytes.
constexpr int kKeyStagingBytes = kTile * 256;

// GROUPS = groups of four query heads a wave carries (1 or 2: up to 8 query heads per kv head).
// WIDE (fp8 caches, and bf16 / f16 caches with more than four query heads per kv head): the query heads of the kv
// head sit in the sixteen columns of one MFMA, each once, and the values take the dense route: V rows (widened, for
// fp8) are staged in a private LDS buffer and read back transposed (ds_read_b64_tr_b16) as the A operand of
// v_mfma_f32_16x16x32, O^T[dim, head] += V^T . P^T.  That is a third of the matrix instructions and half the
// exponentials of the one-hot form with two groups, which matters where the byte rate of an fp8 cache leaves the vector
// and matrix units little time per byte, and where eight query heads share a kv head (the one-hot form with two
// groups runs out of registers there and reached 55 % of the HBM peak where one group reaches 74 %).  With bf16 / f16
// caches the wave's Q^T lives in LDS too (four kilobytes, read twice per tile): two 64-register tiles, the 32
// accumulators and Q^T would not fit the wave's registers together.
template <int GROUPS, bool ALIGNED16, bool FP8, bool EXACT, bool WIDE = false, bool F16 = false>
SINGE_DEVICE void paged_decode_body(const DecodeArgs& a, unsigned int* prefix, unsigned char* staging = nullptr) {
    static_assert((!FP8 || WIDE) && (!WIDE || GROUPS == 1), "fp8 caches take the wide form; the wide form carries one group");
    constexpr bool kQueryInLds = WIDE && !FP8;
    constexpr bool kLean = FP8 || (!WIDE && GROUPS == 1 && kDim == 128);  // see locate_half
    using Tile = typename std::conditional<FP8, KeyTileFp8, KeyTileBf16>::type;
    constexpr int DEPTH = FP8 ? 3 : 2;  // an fp8 tile is half the bytes, so one more is kept in flight
    const unsigned int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const unsigned int g = lane >> 4, t = lane & 15;
    const unsigned int reach = a.block_table_batch_stride * a.block_size;

    // Tiles per sequence, prefix-summed: prefix[b] = tiles of sequences before b; lengths[b] = its keys,
    // clamped to what its table row can address.
    unsigned int* lengths = prefix + a.batch + 1;
    unsigned int* starts = lengths + a.batch;  // rows of their own lengths: where each begins in the table (the launch then lends a third array)
    unsigned int* begins = starts + a.batch;   // and, under a window, how many of its first keys are hidden (a fourth)
    if (wave == 0) {
        unsigned int carry = 0;
        for (unsigned int base = 0; base < a.batch; base += 64) {
            unsigned int tiles = 0, len = 0;
            if (base + lane < a.batch) {
                const int raw = a.actual_seq_lens[base + lane];
                len = raw < 0 ? 0u : (static_cast<unsigned int>(raw) < reach ? static_cast<unsigned int>(raw) : reach);
                tiles = (len + kTile - 1) / kTile;
            }
            unsigned int scan = tiles;
#pragma unroll
            for (int step = 1; step < 64; step *= 2) {
                const unsigned int below = __shfl_up(scan, step, 64);
                if (lane >= static_cast<unsigned int>(step)) scan += below;
            }
            if (base + lane < a.batch) {
                prefix[base + lane + 1] = carry + scan;
                lengths[base + lane] = len;
                if (a.row_starts != nullptr) starts[base + lane] = a.row_starts[base + lane];
                if (a.row_begins != nullptr) begins[base + lane] = a.row_begins[base + lane];
            }
            carry += __shfl(scan, 63, 64);
        }
        if (lane == 0) prefix[0] = 0;
    }
    __syncthreads();
    const unsigned int total = prefix[a.batch];
    const unsigned int share = total == 0 ? 1u : (total + a.workers - 1) / a.workers;
    if (blockIdx.x == 0 && blockIdx.y == 0) {
        // What the combine kernel needs to find a sequence's slots.
        for (unsigned int i = threadIdx.x; i <= a.batch; i += blockDim.x) a.meta[2 + i] = prefix[i];
        if (threadIdx.x == 0) {
            a.meta[0] = share;
            a.meta[1] = total;
        }
    }

    const unsigned int lanes_of_work = a.kv_heads * a.head_groups;
    const unsigned int work = blockIdx.y * a.work_per_wg + wave % a.work_per_wg;
    const unsigned int sub = wave / a.work_per_wg;
    if (work >= lanes_of_work || sub >= a.workers_per_wg) return;
    const unsigned int worker = blockIdx.x * a.workers_per_wg + sub;
    const unsigned int range_first = worker * share;
    if (worker >= a.workers || range_first >= total) return;
    const unsigned int range_end = total < range_first + share ? total : range_first + share;

    const unsigned int group = a.heads / a.kv_heads;
    const unsigned int kv_head = work / a.head_groups;
    const unsigned int head_in_group = (work % a.head_groups) * a.heads_per_wave;  // first query head of this wave inside its group
    const unsigned int wave_heads = group - head_in_group < a.heads_per_wave ? group - head_in_group : a.heads_per_wave;
    const unsigned int slots = a.workers + a.batch;

    // The sequence that holds tile range_first: the last b with prefix[b] <= range_first.
    unsigned int seq = 0;
    {
        unsigned int low = 0, high = a.batch;  // prefix[low] <= range_first < prefix[high]
        while (high - low > 1) {
            const unsigned int mid = (low + high) / 2;
            if (prefix[mid] <= range_first) low = mid; else high = mid;
        }
        seq = low;
    }

    // One-hot placement of a probability: column n = lane % 16 carries head n / 4 at position n % 4.
    const unsigned int place0 = (t & 2) ? 0u : ((t & 1) ? 0xffff0000u : 0x0000ffffu);
    const unsigned int place1 = (t & 2) ? ((t & 1) ? 0xffff0000u : 0x0000ffffu) : 0u;
    // Dims a lane feeds into score MFMA c: bf16 rows are fetched as 32c + 8g (64 contiguous bytes
    // of each key per load), fp8 rows as 32g + 8c (32 contiguous bytes per lane).
    const unsigned int dim_lane = FP8 ? 32 * g : 8 * g, dim_step = FP8 ? 8 : 32;

    bf16x8_t q[GROUPS][4];
    GroupState state[GROUPS];
    // WIDE: column t of the score MFMAs is query head t of the wave; acc[db][r] is O^T[16 db + 4 g + r][head t].
    f32x4_t wide_acc[WIDE ? 8 : 1];
    float wide_max = -INFINITY, wide_sum = 0.0f;
    unsigned char* const staged = WIDE ? staging + wave * kStagedTileBytes : nullptr;
    // K's way into its operand layout (bf16 / f16 caches): behind the eight value buffers in the wide form, and the
    // waves' Q^T behind those.
    // (the wide form takes K through in two halves of sixteen keys, a buffer of half the size)
    unsigned char* const key_staging = WIDE ? staging + 8 * kStagedTileBytes + wave * (kKeyStagingBytes / 2) : staging + wave * kKeyStagingBytes;
    unsigned char* const query_slot = staging + 8 * (kStagedTileBytes + kKeyStagingBytes / 2) + wave * 4096 + 16 * lane;
    auto load_query = [&](unsigned int b) __attribute__((always_inline)) {
        if constexpr (WIDE) {
            const bool real = t < wave_heads;
            const uint16_t* qp = a.query + (static_cast<size_t>(b) * a.heads + kv_head * group + head_in_group + (real ? t : 0)) * kDim + dim_lane;
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                uint4 bits = *reinterpret_cast<const uint4*>(qp + dim_step * c);
                if (!real) bits = make_uint4(0, 0, 0, 0);
                if constexpr (kQueryInLds) *reinterpret_cast<uint4*>(query_slot + 1024 * c) = bits;  // a slot only this lane touches
                else q[0][c] = __builtin_bit_cast(bf16x8_t, bits);
            }
#pragma unroll
            for (int db = 0; db < 8; ++db) wide_acc[db] = {0.0f, 0.0f, 0.0f, 0.0f};
            wide_max = -INFINITY;
            wide_sum = 0.0f;
            return;
        }
#pragma unroll
        for (int hg = 0; hg < GROUPS; ++hg) {
            const unsigned int local = 4 * hg + (t >> 2);
            const bool real = local < wave_heads;
            const uint16_t* qp = a.query + (static_cast<size_t>(b) * a.heads + kv_head * group + head_in_group + (real ? local : 0)) * kDim;
#pragma unroll
            for (int c = 0; c < kDimSteps; ++c) {
                const bool within = kDim % 32 == 0 || dim_lane + dim_step * c < static_cast<unsigned int>(kDim);  // (half a last step)
                uint4 bits = *reinterpret_cast<const uint4*>(qp + (within ? dim_lane + dim_step * c : 0));
                if (!real || !within) bits = make_uint4(0, 0, 0, 0);
                q[hg][c] = __builtin_bit_cast(bf16x8_t, bits);
            }
            state[hg].acc[0] = {0.0f, 0.0f, 0.0f, 0.0f};
            state[hg].acc[1] = {0.0f, 0.0f, 0.0f, 0.0f};
            state[hg].running_max = -INFINITY;
            state[hg].running_sum = 0.0f;
        }
    };

    auto fold_wide = [&](const Tile& tile) __attribute__((always_inline)) {
        if constexpr (WIDE) {
            // Values first: widened rows go to the staging buffer while the scores are computed.  Lane (g, t)
            // holds key 16 half + 4 g + i, dims 8 t .. 8 t + 7.
#pragma unroll
            for (int half = 0; half < 2; ++half)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    uint4 row;
                    if constexpr (FP8) row = widen_fp8x8<EXACT>(tile.v[half][i].x, tile.v[half][i].y, EXACT ? tile.row_value_scale[half][i] : 1.0f);
                    else row = tile.v[half][i];
                    *reinterpret_cast<uint4*>(staged + (16 * half + 4 * g + i) * kStagedRowBytes + 16 * t) = row;
                }
            // Scores S^T[key 16 half + row][head]: row = lane % 16 of the A operand is key t of the half.
            // From here to the end of the tile the wave goes ahead of its SIMD's other wave: the scores, the softmax and
            // the value products are a dependent chain, the widening of the next tile's values above is not (fp8
            // split kernel 758 -> 731 us; the priority over the widening instead, or over the softmax alone, gains 1 %).
            __builtin_amdgcn_s_setprio(1);
            f32x4_t s0 = {0.0f, 0.0f, 0.0f, 0.0f}, s1 = {0.0f, 0.0f, 0.0f, 0.0f};
            if constexpr (FP8) {
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    const uint4 a0 = tile.k[0][c >> 1], a1 = tile.k[1][c >> 1];
                    const uint4 first = (c & 1) ? widen_fp8x8<EXACT>(a0.z, a0.w, EXACT ? tile.key_scale[0] : 1.0f)
                                                : widen_fp8x8<EXACT>(a0.x, a0.y, EXACT ? tile.key_scale[0] : 1.0f);
                    const uint4 second = (c & 1) ? widen_fp8x8<EXACT>(a1.z, a1.w, EXACT ? tile.key_scale[1] : 1.0f)
                                                 : widen_fp8x8<EXACT>(a1.x, a1.y, EXACT ? tile.key_scale[1] : 1.0f);
                    s0 = score_mma<F16>(first, q[0][c], s0);
                    s1 = score_mma<F16>(second, q[0][c], s1);
                }
            } else {
                // K rows go to the wave's other buffer as fetched and come back in the operand layout (as in `fold`),
                // sixteen keys at a time; LDS keeps a wave's accesses in order, so the second half may follow the
                // first half's reads into the same rows.
#pragma unroll
                for (int half = 0; half < 2; ++half) {
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        *reinterpret_cast<uint4*>(key_staging + (4 * g + i) * 256 + ((t ^ (4 * g + i)) << 4)) = tile.k[half][i];
                    f32x4_t scores = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        const uint4 keys = *reinterpret_cast<const uint4*>(key_staging + t * 256 + (((4 * c + g) ^ t) << 4));
                        const uint4 mine = *reinterpret_cast<const uint4*>(query_slot + 1024 * c);
                        scores = score_mma<F16>(keys, __builtin_bit_cast(bf16x8_t, mine), scores);
                    }
                    if (half == 0) s0 = scores; else s1 = scores;
                }
            }
            // Lane (g, t) now holds head t against keys 16 half + 4 g + i.
            float p[8];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                float first = s0[i] * a.scale_log2e, second = s1[i] * a.scale_log2e;
                if constexpr (!EXACT) {
                    first *= tile.row_key_scale[0][i];
                    second *= tile.row_key_scale[1][i];
                }
                p[i] = first;
                p[4 + i] = second;
            }
            // Dead keys (past the sequence's end, before its window, behind an entry that is no cache block) leave the
            // softmax: only a sequence's first and last tiles have any.  (kLean: the statement keeps this a branch that
            // the other tiles skip; as selects the tests run for every tile.)
            if (!kLean || __any(tile.live != 0xffu)) {
                if constexpr (kLean) asm volatile("");
#pragma unroll
                for (int i = 0; i < 8; ++i)
                    if (!((tile.live >> i) & 1u)) p[i] = -INFINITY;
            }
            float largest = fmaxf(fmaxf(fmaxf(p[0], p[1]), fmaxf(p[2], p[3])), fmaxf(fmaxf(p[4], p[5]), fmaxf(p[6], p[7])));
            largest = across_groups_max(largest);
            // The reference point of a head may lag its largest score by kReferenceLag doublings: the weights then
            // reach 2^kReferenceLag at most, and the 32 accumulator registers are rescaled on the few tiles where some
            // head's scores outgrow that, not on every tile.
            if (__any(largest > wide_max + kReferenceLag || (wide_max == -INFINITY && largest != -INFINITY))) {
                const float moved = fmaxf(wide_max, largest);
                const float rescale = fast_exp2(wide_max - (moved == -INFINITY ? 0.0f : moved));
                wide_sum *= rescale;
#pragma unroll
                for (int db = 0; db < 8; ++db)
#pragma unroll
                    for (int r = 0; r < 4; ++r) wide_acc[db][r] *= rescale;
                wide_max = moved;
            }
            const float base = wide_max == -INFINITY ? 0.0f : wide_max;
            float total = 0.0f;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                p[i] = fast_exp2(p[i] - base);
                total += p[i];
                if constexpr (!EXACT) p[i] *= tile.row_value_scale[i >> 2][i & 3];
            }
            wide_sum += total;
            const uint4 weights = make_uint4(half_pair<F16>(p[0], p[1]), half_pair<F16>(p[2], p[3]), half_pair<F16>(p[4], p[5]),
                                             half_pair<F16>(p[6], p[7]));
            // O^T[dim, head] += V^T . P^T: k-slots 8 g + j of the MFMA are keys 4 g + j (j < 4) and
            // 16 + 4 g + j - 4, which is how the two transposing reads of a 16-lane group deliver them.
            typedef short v4i16_t __attribute__((ext_vector_type(4)));
            typedef short v8i16_t __attribute__((ext_vector_type(8)));
            typedef v4i16_t __attribute__((address_space(3))) * lds_v4_t;
            const unsigned char* patch = staged + (4 * g + (t >> 2)) * kStagedRowBytes + 8 * (t & 3);
#pragma unroll
            for (int db = 0; db < 8; ++db) {
                const v4i16_t low = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4_t)(patch + 32 * db));
                const v4i16_t high = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4_t)(patch + 16 * kStagedRowBytes + 32 * db));
                const v8i16_t both = __builtin_shufflevector(low, high, 0, 1, 2, 3, 4, 5, 6, 7);
                wide_acc[db] = score_mma<F16>(__builtin_bit_cast(uint4, both), __builtin_bit_cast(bf16x8_t, weights), wide_acc[db]);
            }
        }
        if constexpr (WIDE) __builtin_amdgcn_s_setprio(0);
    };
    auto fold = [&](const Tile& tile) __attribute__((always_inline)) {
        if constexpr (WIDE) {
            fold_wide(tile);
            return;
        }
        // Scores of every head group.  fp8 operands are widened right where they are used, so only
        // one widened K chunk and one widened V row are alive at a time.
        f32x4_t s0[GROUPS], s1[GROUPS];
#pragma unroll
        for (int hg = 0; hg < GROUPS; ++hg) {
            s0[hg] = {0.0f, 0.0f, 0.0f, 0.0f};
            s1[hg] = {0.0f, 0.0f, 0.0f, 0.0f};
        }
        if constexpr (!FP8) {
            // K into its operand layout: rows go to the wave's LDS buffer as fetched (row = key, the sixteen 16-byte
            // chunks of a row permuted by the row's low bits so that the sixteen rows an operand read touches fall
            // in different banks) and come back as lane (g, t): key t, dims 32 c + 8 g .. + 8.
#pragma unroll
            for (int half = 0; half < 2; ++half)
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (kDim == 128 || 8 * t < static_cast<unsigned int>(kDim))
                        *reinterpret_cast<uint4*>(key_staging + (16 * half + 4 * g + i) * 256 + ((t ^ (4 * g + i)) << 4)) = tile.k[half][i];
        }
#pragma unroll
        for (int c = 0; c < kDimSteps; ++c) {
            uint4 first, second;
            if constexpr (!FP8) {
                const unsigned char* row = key_staging + t * 256 + (((4 * c + g) ^ t) << 4);
                first = *reinterpret_cast<const uint4*>(row);
                second = *reinterpret_cast<const uint4*>(row + 16 * 256);
                if (kDim % 32 != 0 && 8 * (4 * c + g) >= static_cast<unsigned int>(kDim))  // nobody wrote these chunks
                    first = second = make_uint4(0, 0, 0, 0);
            }
#pragma unroll
            for (int hg = 0; hg < GROUPS; ++hg) {
                s0[hg] = score_mma<F16>(first, q[hg][c], s0[hg]);
                s1[hg] = score_mma<F16>(second, q[hg][c], s1[hg]);
            }
        }
        float p[GROUPS][8];
#pragma unroll
        for (int hg = 0; hg < GROUPS; ++hg) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float first = s0[hg][i] * a.scale_log2e, second = s1[hg][i] * a.scale_log2e;
                p[hg][i] = first;
                p[hg][4 + i] = second;
            }
            // (dead keys leave the softmax: a branch that the tiles without any skip, as in the wide form)
            if (!kLean || __any(tile.live != 0xffu)) {
                if constexpr (kLean) asm volatile("");
#pragma unroll
                for (int i = 0; i < 8; ++i)
                    if (!((tile.live >> i) & 1u)) p[hg][i] = -INFINITY;
            }
            float largest = fmaxf(fmaxf(fmaxf(p[hg][0], p[hg][1]), fmaxf(p[hg][2], p[hg][3])),
                                  fmaxf(fmaxf(p[hg][4], p[hg][5]), fmaxf(p[hg][6], p[hg][7])));
            largest = fmaxf(across_groups_max(largest), state[hg].running_max);
            const float base = largest == -INFINITY ? 0.0f : largest;
            const float rescale = fast_exp2(state[hg].running_max - base);
            float total = 0.0f;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                p[hg][i] = fast_exp2(p[hg][i] - base);
                total += p[hg][i];
            }
            state[hg].running_sum = state[hg].running_sum * rescale + total;
            state[hg].running_max = largest;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                state[hg].acc[0][r] *= rescale;
                state[hg].acc[1][r] *= rescale;
            }
        }
#pragma unroll
        for (int half = 0; half < 2; ++half)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                uint4 row;
                if constexpr (!FP8) row = tile.v[half][i];
#pragma unroll
                for (int hg = 0; hg < GROUPS; ++hg) {
                    const unsigned int both = half_twice<F16>(p[hg][half * 4 + i]);
                    const uint2 hot = make_uint2(both & place0, both & place1);
                    state[hg].acc[0] = value_mma<F16>(make_uint2(row.x, row.y), hot, state[hg].acc[0]);
                    state[hg].acc[1] = value_mma<F16>(make_uint2(row.z, row.w), hot, state[hg].acc[1]);
                }
            }
    };

    // Writes the partial row of sequence b: O / sum per head, and the natural-log LSE.
    auto flush = [&](unsigned int b) __attribute__((always_inline)) {
        const size_t slot = static_cast<size_t>(work) * slots + worker + b;
        if constexpr (WIDE) {
            const float sum = across_groups_sum(wide_sum);
            const float inverse = sum > 0.0f ? 1.0f / sum : 0.0f;
            if (t < wave_heads) {
                float* row = a.partial_out + (slot * a.heads_per_wave + t) * kDim;
#pragma unroll
                for (int db = 0; db < 8; ++db)
                    *reinterpret_cast<float4*>(row + 16 * db + 4 * g) = make_float4(wide_acc[db][0] * inverse, wide_acc[db][1] * inverse,
                                                                                    wide_acc[db][2] * inverse, wide_acc[db][3] * inverse);
                if (g == 0) a.partial_lse[slot * a.heads_per_wave + t] = sum > 0.0f ? (wide_max + fast_log2(sum)) * kLn2 : -INFINITY;
            }
            return;
        }
#pragma unroll
        for (int hg = 0; hg < GROUPS; ++hg) {
            const float sum = across_groups_sum(state[hg].running_sum);
            const float inverse = sum > 0.0f ? 1.0f / sum : 0.0f;
            const unsigned int local = 4 * hg + (t >> 2);
            if (local < wave_heads) {
                float* row = a.partial_out + (slot * a.heads_per_wave + local) * kDim;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    if (kDim == 128 || 8 * (4 * g + r) < static_cast<unsigned int>(kDim)) {
                        row[8 * (4 * g + r) + (t & 3)] = state[hg].acc[0][r] * inverse;
                        row[8 * (4 * g + r) + 4 + (t & 3)] = state[hg].acc[1][r] * inverse;
                    }
                }
                if (g == 0 && (t & 3) == 0)
                    a.partial_lse[slot * a.heads_per_wave + local] =
                        sum > 0.0f ? (state[hg].running_max + fast_log2(sum)) * kLn2 : -INFINITY;
            }
        }
    };

    // Walk the range tile by tile with DEPTH tiles in registers: each buffer is refilled, with the tile
    // DEPTH ahead, right after it has been folded, so DEPTH - 1 tiles are always on their way.
    unsigned int at = range_first;                       // flat index of the tile being folded
    unsigned int load_at = range_first, load_seq = seq;  // and of the next tile to fetch
    EntryCache entries;
    auto issue = [&](Tile& buffer) __attribute__((always_inline)) {
        if (load_at >= range_end) return;
        // A tile's requests (table entries, address arithmetic, loads) go out ahead of the SIMD's other wave's folding:
        // the split kernel 51.95 -> 51.5 us, the fp8 one 778 -> 767 us (four rounds each way on one box).
        __builtin_amdgcn_s_setprio(2);
        while (prefix[load_seq + 1] <= load_at) ++load_seq;  // skips empty sequences
        const unsigned int first_key = (load_at - prefix[load_seq]) * kTile, end = lengths[load_seq];
        const size_t row_base = a.row_starts != nullptr ? starts[load_seq] : static_cast<size_t>(load_seq) * a.block_table_batch_stride;
        if constexpr (ALIGNED16) {
            // Entries this tile reads: those of its first key and of its last live key (a half past
            // the end re-reads the last key's entry).
            unsigned int low, high, slot;
            split_key(a, first_key, low, slot);
            split_key(a, (first_key + kTile <= end ? first_key + kTile : end) - 1, high, slot);
            if (entries.sequence != load_seq || low < entries.first_entry || high >= entries.first_entry + 64)
                fill_entries<FP8>(entries, a, load_seq, row_base, low, kv_head, lane);
        }
        load_tile<ALIGNED16, kLean>(buffer, a, a.block_table + row_base, entries, first_key, end, kv_head, g, t);
        if (a.row_begins != nullptr) {
            // Keys of the row before its window (bit half * 4 + i of `live` is key first_key + 16 half + 4 g + i).
            const unsigned int begin = begins[load_seq];
            if (begin > first_key) {
#pragma unroll
                for (int bit = 0; bit < 8; ++bit)
                    if (first_key + 16u * (bit >> 2) + 4u * g + (bit & 3) < begin) buffer.live &= ~(1u << bit);
            }
        }
        ++load_at;
        __builtin_amdgcn_s_setprio(0);
    };
    auto consume = [&](const Tile& buffer) __attribute__((always_inline)) {
        // Returns false when this was the last tile of the range.
        fold(buffer);
        const unsigned int next_at = at + 1;
        const bool more = next_at < range_end;
        unsigned int next_seq = seq;
        if (more)
            while (prefix[next_seq + 1] <= next_at) ++next_seq;
        if (!more || next_seq != seq) {
            flush(seq);
            if (more) load_query(next_seq);
        }
        at = next_at;
        seq = next_seq;
        return more;
    };
    load_query(seq);
    Tile first, second;
    issue(first);
    issue(second);
    if constexpr (DEPTH == 3) {
        Tile third;
        issue(third);
        while (true) {
            if (!consume(first)) break;
            issue(first);
            if (!consume(second)) break;
            issue(second);
            if (!consume(third)) break;
            issue(third);
        }
    } else {
        while (true) {
            if (!consume(first)) break;
            issue(first);
            if (!consume(second)) break;
            issue(second);
        }
    }
}

}  // namespace

// Names carry the head dimension of the build: singe_paged_decode_bf16_d128_g1_b16, ..._d64_g1_b16.
#define SINGE_PASTE4_(a, b, c, d) a##b##c##d
#define SINGE_PASTE4(a, b, c, d) SINGE_PASTE4_(a, b, c, d)
#define SINGE_DECODE_NAME(STEM, TAIL) SINGE_PASTE4(STEM, _d, SINGE_HEAD_DIM, TAIL)

#define SINGE_DECODE_KERNEL(NAME, GROUPS, ALIGNED, FP8, EXACT)                                  \
    extern "C" __global__ __launch_bounds__(512) void NAME(DecodeArgs args) {                    \
        extern __shared__ unsigned int prefix[];                                                \
        __shared__ __attribute__((aligned(16))) unsigned char staging[8 * kKeyStagingBytes];    \
        paged_decode_body<GROUPS, ALIGNED, FP8, EXACT>(args, prefix, staging);                  \
    }

SINGE_DECODE_KERNEL(SINGE_DECODE_NAME(singe_paged_decode_bf16, _g1_b16), 1, true, false, true)
SINGE_DECODE_KERNEL(SINGE_DECODE_NAME(singe_paged_decode_bf16, _g2_b16), 2, true, false, true)
SINGE_DECODE_KERNEL(SINGE_DECODE_NAME(singe_paged_decode_bf16, _g1_any), 1, false, false, true)
SINGE_DECODE_KERNEL(SINGE_DECODE_NAME(singe_paged_decode_bf16, _g2_any), 2, false, false, true)

// paged_kv_decode_attention_f16: the same kernels on f16 operands.
#define SINGE_DECODE_F16_KERNEL(NAME, GROUPS, ALIGNED)                                          \
    extern "C" __global__ __launch_bounds__(512) void NAME(DecodeArgs args) {                    \
        extern __shared__ unsigned int prefix[];                                                \
        __shared__ __attribute__((aligned(16))) unsigned char staging[8 * kKeyStagingBytes];    \
        paged_decode_body<GROUPS, ALIGNED, false, true, false, true>(args, prefix, staging);    \
    }

SINGE_DECODE_F16_KERNEL(SINGE_DECODE_NAME(singe_paged_decode_f16, _g1_b16), 1, true)
SINGE_DECODE_F16_KERNEL(SINGE_DECODE_NAME(singe_paged_decode_f16, _g2_b16), 2, true)
SINGE_DECODE_F16_KERNEL(SINGE_DECODE_NAME(singe_paged_decode_f16, _g1_any), 1, false)
SINGE_DECODE_F16_KERNEL(SINGE_DECODE_NAME(singe_paged_decode_f16, _g2_any), 2, false)

#if SINGE_HEAD_DIM == 128
// bf16 / f16 caches with five to sixteen query heads per kv head: the wide form; a value buffer, a key buffer and Q^T per wave.
#define SINGE_DECODE_WIDE_HALF_KERNEL(NAME, ALIGNED, F16)                                                               \
    extern "C" __global__ __launch_bounds__(512) void NAME(DecodeArgs args) {                                            \
        extern __shared__ unsigned int prefix[];                                                                        \
        __shared__ __attribute__((aligned(16))) unsigned char staging[8 * (kStagedTileBytes + kKeyStagingBytes / 2 + 4096)]; \
        paged_decode_body<1, ALIGNED, false, true, true, F16>(args, prefix, staging);                                   \
    }

SINGE_DECODE_WIDE_HALF_KERNEL(singe_paged_decode_bf16_wide_d128_b16, true, false)
SINGE_DECODE_WIDE_HALF_KERNEL(singe_paged_decode_bf16_wide_d128_any, false, false)
SINGE_DECODE_WIDE_HALF_KERNEL(singe_paged_decode_f16_wide_d128_b16, true, true)
SINGE_DECODE_WIDE_HALF_KERNEL(singe_paged_decode_f16_wide_d128_any, false, true)

#define SINGE_DECODE_WIDE_KERNEL(NAME, ALIGNED, EXACT)                                          \
    extern "C" __global__ __launch_bounds__(512) void NAME(DecodeArgs args) {                    \
        extern __shared__ unsigned int prefix[];                                                \
        __shared__ __attribute__((aligned(16))) unsigned char staging[8 * kStagedTileBytes];    \
        paged_decode_body<1, ALIGNED, true, EXACT, true>(args, prefix, staging);                \
    }

SINGE_DECODE_WIDE_KERNEL(singe_paged_decode_f8kv_wide_d128_b16, true, true)
SINGE_DECODE_WIDE_KERNEL(singe_paged_decode_f8kv_wide_d128_any, false, true)
SINGE_DECODE_WIDE_KERNEL(singe_paged_decode_f8kv_wide_relaxed_d128_b16, true, false)
SINGE_DECODE_WIDE_KERNEL(singe_paged_decode_f8kv_wide_relaxed_d128_any, false, false)
#endif

// Folds the partial rows of one (sequence, query head) into the bf16 output:
// out = sum_s exp(lse_s - max) * partial_s / sum_s exp(lse_s - max)
// (singe-kernel/src/cpu/attention.rs:2157-2193).  One wave per row.  The kernel is a chain of dependent
// memory round trips, so it is written to need few of them: lane s fetches the log-sum-exp of slot s
// (one trip for up to 64 slots), and the slots' rows are fetched FIRST (sixteen) at a time, two dims per lane.  When
// rows have one or two slots (more sequences than workers) the kernel's time is rounds of waves times its chain of
// round trips, and the sixteen rows' registers hold it to twelve waves a compute unit: the _few kernels fetch four.
template <bool F16, int FIRST = 16>
SINGE_DEVICE void paged_decode_combine_body(const CombineArgs& a) {
    const unsigned int lane = threadIdx.x & 63;
    const unsigned int row = blockIdx.x * 4 + (threadIdx.x >> 6);  // batch * heads + head
    if (row >= a.batch * a.heads) return;
    const unsigned int b = row / a.heads, head = row % a.heads;
    if (a.row_lengths != nullptr && a.row_lengths[b] < 0) return;
    const unsigned int group = a.heads / a.kv_heads;
    const unsigned int kv_head = head / group, in_group = head % group;
    const unsigned int work = kv_head * a.head_groups + in_group / a.heads_per_wave, local = in_group % a.heads_per_wave;
    const unsigned int share = a.meta[0];
    const unsigned int first_tile = a.meta[2 + b], end_tile = a.meta[3 + b];
    float low = 0.0f, high = 0.0f;  // a sequence with no keys keeps a zero row (cpu/attention.rs:1213-1215)
    float best = -INFINITY, total = 0.0f;
    const bool holds_values = 2 * lane < static_cast<unsigned int>(kDim);  // a lane takes two of the row's values
    if (end_tile > first_tile) {
        const unsigned int first_worker = first_tile / share, last_worker = (end_tile - 1) / share;
        const size_t base = (static_cast<size_t>(work) * (a.workers + a.batch) + first_worker + b) * a.heads_per_wave + local;
        const unsigned int count = last_worker - first_worker + 1;
        for (unsigned int chunk = 0; chunk < count; chunk += 64) {
            const unsigned int n = count - chunk < 64 ? count - chunk : 64;
            const size_t chunk_base = base + static_cast<size_t>(chunk) * a.heads_per_wave;
            const float mine = lane < n ? a.partial_lse[chunk_base + static_cast<size_t>(lane) * a.heads_per_wave] : -INFINITY;
            // The first FIRST rows are asked for together with the log-sum-exps, before anything waits for those: a
            // sequence rarely has more slots, and the kernel is a chain of memory round trips.
            float2 rows[FIRST];
            auto fetch = [&](unsigned int first) __attribute__((always_inline)) {
#pragma unroll
                for (int j = 0; j < FIRST; ++j) {
                    rows[j] = make_float2(0.0f, 0.0f);
                    if (first + j < n && holds_values)
                        rows[j] = *reinterpret_cast<const float2*>(a.partial_out + (chunk_base + static_cast<size_t>(first + j) * a.heads_per_wave) * kDim + 2 * lane);
                }
            };
            fetch(0);
            float largest = mine;
#pragma unroll
            for (int step = 32; step >= 1; step >>= 1) largest = fmaxf(largest, __shfl_xor(largest, step, 64));
            largest = fmaxf(largest, best);
            if (largest == -INFINITY) continue;  // nothing but empty slots so far
            const float rescale = __expf(best - largest);
            const float weight = __expf(mine - largest);  // 0 for lanes past n
            float weights = weight;
#pragma unroll
            for (int step = 32; step >= 1; step >>= 1) weights += __shfl_xor(weights, step, 64);
            total = total * rescale + weights;
            low *= rescale;
            high *= rescale;
            best = largest;
            for (unsigned int first = 0; first < n; first += FIRST) {
                if (first != 0) fetch(first);
#pragma unroll
                for (int j = 0; j < FIRST; ++j) {
                    const float w = __shfl(weight, static_cast<int>(first) + j, 64);
                    if (first + j < n) {
                        low = fmaf(w, rows[j].x, low);
                        high = fmaf(w, rows[j].y, high);
                    }
                }
            }
        }
        if (total > 0.0f) {
            low /= total;
            high /= total;
        }
    }
    unsigned int packed;
    if constexpr (F16) {
        const f32x2_t both = {low, high};
        packed = __builtin_bit_cast(unsigned int, __builtin_convertvector(both, f16x2_t));
    } else {
        packed = pack_bf16x2(low, high);
    }
    if (holds_values) *reinterpret_cast<unsigned int*>(a.out + static_cast<size_t>(row) * kDim + 2 * lane) = packed;
    // The row's log-sum-exp in base two, for the paged attention op (the slots hold natural logarithms).
    if (a.lse != nullptr && lane == 0) a.lse[row] = total > 0.0f ? (best + __logf(total)) * 1.4426950408889634074f : -INFINITY;
}

// The same fold for rows with many slots (few sequences, long contexts: a lone sequence has a slot per worker, 256 of
// them): a workgroup of eight waves per row, wave w folding the slots of the 16-slot groups w, w + 8, ..., and the first
// wave folding the eight results, which it finds in LDS.  One wave per row takes a round trip per sixteen slots, 21 us for
// 256 of them; this takes two.
constexpr int kCombineWaves = 8;

template <bool F16>
SINGE_DEVICE void paged_decode_combine_many_body(const CombineArgs& a) {
    __shared__ float wave_best[kCombineWaves], wave_total[kCombineWaves];
    __shared__ float2 wave_values[kCombineWaves][64];
    const unsigned int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const unsigned int row = blockIdx.x;  // batch * heads + head
    const unsigned int b = row / a.heads, head = row % a.heads;
    if (a.row_lengths != nullptr && a.row_lengths[b] < 0) return;  // (the whole workgroup: it is one row's)
    const unsigned int group = a.heads / a.kv_heads;
    const unsigned int kv_head = head / group, in_group = head % group;
    const unsigned int work = kv_head * a.head_groups + in_group / a.heads_per_wave, local = in_group % a.heads_per_wave;
    const unsigned int share = a.meta[0];
    const unsigned int first_tile = a.meta[2 + b], end_tile = a.meta[3 + b];
    const bool holds_values = 2 * lane < static_cast<unsigned int>(kDim);  // a lane takes two of the row's values
    float low = 0.0f, high = 0.0f, best = -INFINITY, total = 0.0f;
    if (end_tile > first_tile) {
        const unsigned int first_worker = first_tile / share, last_worker = (end_tile - 1) / share;
        const size_t base = (static_cast<size_t>(work) * (a.workers + a.batch) + first_worker + b) * a.heads_per_wave + local;
        const unsigned int count = last_worker - first_worker + 1;
        for (unsigned int first = 16 * wave; first < count; first += 16 * kCombineWaves) {
            const unsigned int n = count - first < 16 ? count - first : 16;
            const size_t group_base = base + static_cast<size_t>(first) * a.heads_per_wave;
            const float mine = lane < n ? a.partial_lse[group_base + static_cast<size_t>(lane) * a.heads_per_wave] : -INFINITY;
            float2 rows[16];
#pragma unroll
            for (int j = 0; j < 16; ++j) {
                rows[j] = make_float2(0.0f, 0.0f);
                if (static_cast<unsigned int>(j) < n && holds_values)
                    rows[j] = *reinterpret_cast<const float2*>(a.partial_out + (group_base + static_cast<size_t>(j) * a.heads_per_wave) * kDim + 2 * lane);
            }
            float largest = mine;
#pragma unroll
            for (int step = 32; step >= 1; step >>= 1) largest = fmaxf(largest, __shfl_xor(largest, step, 64));
            largest = fmaxf(largest, best);
            if (largest == -INFINITY) continue;  // nothing but empty slots so far
            const float rescale = __expf(best - largest);
            const float weight = __expf(mine - largest);  // 0 for lanes past n
            float weights = weight;
#pragma unroll
            for (int step = 32; step >= 1; step >>= 1) weights += __shfl_xor(weights, step, 64);
            total = total * rescale + weights;
            low *= rescale;
            high *= rescale;
            best = largest;
#pragma unroll
            for (int j = 0; j < 16; ++j) {
                const float w = __shfl(weight, j, 64);
                if (static_cast<unsigned int>(j) < n) {
                    low = fmaf(w, rows[j].x, low);
                    high = fmaf(w, rows[j].y, high);
                }
            }
        }
    }
    if (lane == 0) {
        wave_best[wave] = best;
        wave_total[wave] = total;
    }
    wave_values[wave][lane] = make_float2(low, high);
    __syncthreads();
    if (wave != 0) return;
    float largest = -INFINITY;
#pragma unroll
    for (int w = 0; w < kCombineWaves; ++w) largest = fmaxf(largest, wave_best[w]);
    low = 0.0f;
    high = 0.0f;
    total = 0.0f;
    if (largest != -INFINITY) {
#pragma unroll
        for (int w = 0; w < kCombineWaves; ++w) {
            const float factor = __expf(wave_best[w] - largest);  // 0 for a wave that saw nothing
            total = fmaf(factor, wave_total[w], total);
            low = fmaf(factor, wave_values[w][lane].x, low);
            high = fmaf(factor, wave_values[w][lane].y, high);
        }
        if (total > 0.0f) {
            low /= total;
            high /= total;
        }
    }
    unsigned int packed;
    if constexpr (F16) {
        const f32x2_t both = {low, high};
        packed = __builtin_bit_cast(unsigned int, __builtin_convertvector(both, f16x2_t));
    } else {
        packed = pack_bf16x2(low, high);
    }
    if (holds_values) *reinterpret_cast<unsigned int*>(a.out + static_cast<size_t>(row) * kDim + 2 * lane) = packed;
    if (a.lse != nullptr && lane == 0) a.lse[row] = total > 0.0f ? (largest + __logf(total)) * 1.4426950408889634074f : -INFINITY;
}

#if SINGE_HEAD_DIM == 128
extern "C" __global__ __launch_bounds__(512) void singe_paged_decode_combine_many_bf16(CombineArgs a) { paged_decode_combine_many_body<false>(a); }
extern "C" __global__ __launch_bounds__(512) void singe_paged_decode_combine_many_f16(CombineArgs a) { paged_decode_combine_many_body<true>(a); }
#else
extern "C" __global__ __launch_bounds__(512) void SINGE_DECODE_NAME(singe_paged_decode_combine_many_bf16, /**/)(CombineArgs a) { paged_decode_combine_many_body<false>(a); }
extern "C" __global__ __launch_bounds__(512) void SINGE_DECODE_NAME(singe_paged_decode_combine_many_f16, /**/)(CombineArgs a) { paged_decode_combine_many_body<true>(a); }
#endif

#if SINGE_HEAD_DIM == 128
extern "C" __global__ __launch_bounds__(256) void singe_paged_decode_combine_few_bf16(CombineArgs a) { paged_decode_combine_body<false, 4>(a); }
extern "C" __global__ __launch_bounds__(256) void singe_paged_decode_combine_few_f16(CombineArgs a) { paged_decode_combine_body<true, 4>(a); }
#else
extern "C" __global__ __launch_bounds__(256) void SINGE_DECODE_NAME(singe_paged_decode_combine_few_bf16, /**/)(CombineArgs a) { paged_decode_combine_body<false, 4>(a); }
extern "C" __global__ __launch_bounds__(256) void SINGE_DECODE_NAME(singe_paged_decode_combine_few_f16, /**/)(CombineArgs a) { paged_decode_combine_body<true, 4>(a); }
#endif

#if SINGE_HEAD_DIM == 128
extern "C" __global__ __launch_bounds__(256) void singe_paged_decode_combine_bf16(CombineArgs a) { paged_decode_combine_body<false>(a); }
extern "C" __global__ __launch_bounds__(256) void singe_paged_decode_combine_f16(CombineArgs a) { paged_decode_combine_body<true>(a); }
#else
extern "C" __global__ __launch_bounds__(256) void SINGE_DECODE_NAME(singe_paged_decode_combine_bf16, /**/)(CombineArgs a) { paged_decode_combine_body<false>(a); }
extern "C" __global__ __launch_bounds__(256) void SINGE_DECODE_NAME(singe_paged_decode_combine_f16, /**/)(CombineArgs a) { paged_decode_combine_body<true>(a); }
#endif
