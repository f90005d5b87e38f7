// Argument blocks shared by the host launcher and the gfx950 kernels.  Each kernel takes exactly one
// of these by value, so host and device agree on the layout by construction (plain fixed-width C
// types only; both sides include this header).
#pragma once

#include <stdint.h>

struct DecodeArgs {
    const uint16_t* query;          // [batch, heads, 128] bf16
    const void* key_cache;          // [blocks, block_size, kv_heads, 128] bf16, or fp8 e4m3 codes
    const void* value_cache;
    const float* key_scales;        // fp8 caches: [blocks, kv_heads] f32, else unused
    const float* value_scales;
    const int32_t* actual_seq_lens; // [batch]
    const uint32_t* block_table;    // [batch, stride]
    float* partial_out;             // [work, workers + batch, heads_per_wave, 128]
    float* partial_lse;             // [work, workers + batch, heads_per_wave], natural log
    uint32_t* meta;                 // [0] tiles per worker, [1] total tiles, [2 + b] tiles before sequence b
    uint32_t batch;
    uint32_t heads;
    uint32_t kv_heads;
    uint32_t block_size;
    int32_t block_shift;            // log2(block_size) when it is a power of two, else -1
    uint32_t physical_blocks;
    uint32_t block_table_batch_stride;
    uint32_t workers;               // equal ranges the flat tile list is cut into
    uint32_t workers_per_wg;        // ranges one workgroup walks (each by work_per_wg waves)
    uint32_t work_per_wg;           // (kv head, head group) pairs one workgroup covers
    uint32_t head_groups;           // waves a kv head's query heads are spread over: ceil(group / 8)
    uint32_t heads_per_wave;        // min(group, 8): partial rows per slot
    float scale_log2e;              // scale * log2(e)
    // Table rows of their own lengths (the paged attention op's page lists): row b starts at entry row_starts[b] of
    // block_table, which then holds block_table_batch_stride entries in all; null: rows are that stride apart.
    const uint32_t* row_starts = nullptr;
    // With row_starts: the first row_begins[b] keys of row b are hidden (a sliding window's keys before the page the
    // row starts in could be left out of the row; those inside that page are masked), or null.
    const uint32_t* row_begins = nullptr;
};

struct CombineArgs {
    uint16_t* out;                  // [batch, heads, 128] bf16
    const float* partial_out;
    const float* partial_lse;
    const uint32_t* meta;
    uint32_t batch;
    uint32_t heads;
    uint32_t kv_heads;
    uint32_t workers;
    uint32_t head_groups;
    uint32_t heads_per_wave;
    float* lse = nullptr;           // [batch, heads] base-two log-sum-exp of each row (-inf for a row without keys), or null
    const int32_t* row_lengths = nullptr;  // non-null: a row whose length is negative belongs to no sequence and is left as it is
};

// Waves of a dense prefill workgroup (singe_fmha_prefill_*_d128_*), 32 query rows each: host and kernel agree on
// it through this constant.  4 (two workgroups per compute unit) and 8 (one, whose K and V tiles serve 256 rows)
// both pass the tests and measure the same; 4 is what the committed profiles were taken with.
constexpr int kDensePrefillWaves = 4;

struct PrefillArgs {
    const uint16_t* query;          // [batch, query_len, heads, 128] bf16, element strides below
    const uint16_t* key;            // [batch, key_len, kv_heads, 128]
    const uint16_t* value;
    uint16_t* out;                  // like query
    float* lse;                     // [batch, heads, query_len] natural log, or null
    uint64_t query_batch_stride, query_sequence_stride, query_head_stride;
    uint64_t key_batch_stride, key_sequence_stride, key_head_stride;
    uint64_t value_batch_stride, value_sequence_stride, value_head_stride;
    uint64_t output_batch_stride, output_sequence_stride, output_head_stride;
    uint32_t batch;
    uint32_t query_len;
    uint32_t key_len;
    uint32_t heads;
    uint32_t kv_heads;
    uint32_t query_tiles;           // ceil(query_len / 128)
    float scale_log2e;
    // The two options of the dense op this kernel takes (null when absent): one logit per query head that joins
    // every row's softmax without a value, in the element type of the query; and the number of keys of each batch
    // entry that take part (the rest are hidden).
    const uint16_t* sinks = nullptr;
    const int32_t* key_lengths = nullptr;
    // The *_options kernels only: an additive mask in the element type of the query, read through element strides
    // over (batch, head, query, key) with 0 for a broadcast axis (null when absent); a window that hides
    // key + window <= query (negative when absent); a cap on the scaled scores, cap * tanh(score / cap)
    // (cap_scale = |scale / cap|, cap_log2e = |cap| * log2(e); both 0 when absent).
    const uint16_t* mask = nullptr;
    uint64_t mask_strides[4] = {0, 0, 0, 0};
    uint32_t mask_packed = 0;  // key stride 1, the other strides multiples of 4, the mask on an 8-byte boundary
    long long window = -1;
    float cap_scale = 0.0f, cap_log2e = 0.0f;
    // Key splits (splits > 1): the key tiles of a query tile are shared out over `splits` workgroups, each leaving its
    // rows normalised in partial_out [splits, batch * heads * query_len, head_dim] with a base-two log-sum-exp in
    // partial_lse [splits, batch * heads * query_len] (-inf and zeros for a share that saw nothing); a sink joins the
    // first share; singe_fmha_prefill_combine_* merges them into out and lse.
    uint32_t splits = 1;
    float* partial_out = nullptr;
    float* partial_lse = nullptr;
    // Few query rows under grouped heads (a decode step through the dense op, no causal mask): with packed_heads != 0
    // a workgroup takes a (batch, kv head) pair and its tile's row r is query r / group of head kv_head * group +
    // r % group (group = heads / kv_heads, query_len * group at most the tile's rows), so the kv head's keys and values
    // are fetched once for all of its query heads.
    uint32_t packed_heads = 0;
};

struct PrefillF32Args {
    const float* query;             // [batch, query_len, heads, dim] through the strides below
    const float* key;
    const float* value;
    float* out;
    float* lse;                     // [batch, heads, query_len] natural log, or null
    uint64_t query_batch_stride, query_sequence_stride, query_head_stride;
    uint64_t key_batch_stride, key_sequence_stride, key_head_stride;
    uint64_t value_batch_stride, value_sequence_stride, value_head_stride;
    uint64_t output_batch_stride, output_sequence_stride, output_head_stride;
    uint32_t batch;
    uint32_t query_len;
    uint32_t key_len;
    uint32_t heads;
    uint32_t kv_heads;
    uint32_t head_dim;
    uint32_t causal;
    uint32_t window_size;           // 0 = no window
    uint32_t has_soft_cap;
    float soft_cap;
    float scale;
    uint32_t aligned = 0;           // row kernels: every row of query, key and value starts on a 16-byte boundary
};

struct PagedAttentionArgs {
    const uint16_t* query_rows;     // [tokens, heads, 128] bf16
    const uint16_t* key_cache;      // [cache_pages, page_size, kv_heads, 128] bf16
    const uint16_t* value_cache;
    const void* query_offsets;      // [sequences + 1] i32 or i64; block-table form: [sequences] i32 starts
    const void* page_offsets;       // [sequences + 1]
    const void* pages;              // [page_table]
    const void* last_page_lengths;  // [sequences]; block-table form: the key lengths
    const void* query_lengths;      // block-table form only: [sequences] i32
    uint16_t* output;               // [tokens, heads, 128] bf16
    float* lse;                     // [tokens, heads] base two, or null
    uint32_t* status;               // first writer wins, may be null
    int64_t window;                 // keys a query sees before itself, itself included; -1 = no window
    uint32_t tokens;
    uint32_t heads;
    uint32_t kv_heads;
    uint32_t page_size;
    uint32_t sequences;
    uint32_t cache_pages;
    uint32_t page_table;            // entries of `pages`; block-table form: entries per table row
    uint32_t row_tiles;             // ceil(groups * tokens / 128): row tiles per (sequence, kv head); with `compact`,
                                    // a bound on the row tiles of all sequences together
    uint32_t compact = 0;           // workgroups find their (sequence, row tile) by a prefix sum over the sequences
    uint32_t longest_first = 0;     // with `compact` and at most 64 sequences: the list takes the sequences longest first
    uint32_t causal;
    int32_t page_shift;             // log2(page_size) when it is a power of two, else -1
    float scale_log2e;              // scale * log2(e)
    float softcap_scale;            // scale / cap
    float softcap_log2e;            // cap * log2(e)
    // Key splits (1 = none): workgroup (unit, row tile, split) folds its share of the tiles and leaves a
    // normalised f32 partial and its base-two log-sum-exp for singe_paged_attention_combine_bf16.
    uint32_t splits = 1;
    float* partial_out = nullptr;   // [splits, tokens * heads, 128]
    float* partial_lse = nullptr;   // [splits, tokens * heads]
    // Kernels that rotate their query themselves (rotary_paged_attention):
    const void* cos = nullptr;                // [tokens, 64] of table_type
    const void* sin = nullptr;
    const uint16_t* query_weight = nullptr;   // [128] bf16, or null
    uint32_t table_type = 0;                  // SingeElement of cos and sin
    uint32_t has_query_norm = 0;              // RMS norm over the head dimension before the rotation
    float query_eps = 0.0f;
};

// singe_mfma_ceiling_*: the register-only product loop.
struct MfmaCeilingArgs {
    const void* operands;   // operand_chunks 16-byte chunks of bf16 / f16 data
    float* out;             // one float per lane of the launch
    uint64_t operand_chunks;
    uint32_t iterations;
};

// singe_hbm_stream_read: the plain streaming read.
struct HbmStreamArgs {
    const void* data;       // chunks 16-byte chunks
    unsigned int* out;      // one word per lane of the launch
    uint64_t chunks;
};

// singe_splitk_reduce_f32: strides in elements.
struct SplitKReduceArgs {
    float* out;         // [batch, heads, dim]
    const float* attn;  // [batch, heads, splits, dim]
    const float* lse;   // [batch, heads, splits] natural log
    uint64_t attn_batch_stride, attn_head_stride, attn_split_stride;
    uint64_t lse_batch_stride, lse_head_stride;
    uint64_t output_batch_stride, output_head_stride;
    uint32_t batch, heads, splits, head_dim;
};

// singe_fmha_decode_splitk_f32_d*: one query per (batch, head) over a slice of the keys.
struct FmhaDecodeSplitKArgs {
    float* out;          // [batch, heads, splits, dim] through the strides below
    float* lse;          // [batch, heads, splits] natural log
    const float* query;  // [batch, heads, dim]
    const float* key;    // [batch, key_len, kv_heads, dim]
    const float* value;
    uint64_t query_batch_stride, key_batch_stride, value_batch_stride, output_batch_stride;
    uint64_t query_head_stride, key_sequence_stride, value_sequence_stride, output_head_stride, output_split_stride;
    uint64_t key_head_stride, value_head_stride, lse_batch_stride, lse_head_stride;
    uint32_t batch, key_len, heads, kv_heads, splits, kv_len_per_split;
    uint32_t aligned;    // every row of query, key and value starts on a 16-byte boundary
    float scale;
};

// singe_paged_kv_decode_splitk_f32_d* and singe_paged_kv_prefill_f32_d*: f32 rows over block-table caches
// [blocks, block_size, kv_heads, dim].
struct PagedRowsF32Args {
    float* out;                  // decode: partials [batch, heads, splits, dim]; prefill: [tokens, heads, dim]
    float* lse;                  // decode: [batch, heads, splits]; prefill: [tokens, heads]; natural log
    const float* query;          // decode: [batch, heads, dim]; prefill: [tokens, heads, dim]
    const float* key_cache;
    const float* value_cache;
    const int32_t* seq_lens_q;   // prefill only
    const int32_t* seq_lens_kv;
    const int32_t* seq_offsets;  // prefill only
    const uint32_t* block_table;
    uint32_t batch, heads, kv_heads, block_size, block_table_batch_stride, physical_blocks;
    uint32_t splits;             // decode only
    uint32_t causal;             // prefill only
    uint32_t aligned;            // every row of the query and the caches starts on a 16-byte boundary
    float scale;
};

// Element types of the general (any head dimension) kernels.
enum SingeElement : uint32_t { kElementF32 = 0, kElementBf16 = 1, kElementF16 = 2, kElementF64 = 3 };

// singe_attention_general_*: dense attention over [batch, heads, len, dim] tensors with every option
// of ScaledDotProductAttentionAttributes.
struct GeneralAttentionArgs {
    const void* query;              // [batch, heads, query_len, head_dim]
    const void* key;                // [batch, kv_heads, key_len, head_dim]
    const void* value;              // [batch, kv_heads, key_len, value_dim]
    const void* mask;               // additive, element type of the query, strides below; or null
    const void* sinks;              // [heads], element type of the query; or null
    const int32_t* key_lengths;     // [batch]; or null
    void* out;                      // [batch, heads, query_len, value_dim]
    float* lse;                     // [batch, heads, query_len] natural log, or null
    // Element strides over (batch, head, position) of the query, key, value and output; a row's dims are contiguous.
    uint64_t query_strides[3], key_strides[3], value_strides[3], out_strides[3];
    uint64_t mask_strides[4];       // over (batch, head, query, key); 0 broadcasts
    int64_t window;                 // -1 = none
    uint32_t batch, heads, kv_heads, query_len, key_len, head_dim, value_dim;
    uint32_t causal, has_softcap;
    float scale, softcap;
    double scale_wide;              // the scale for f64 tensors: the default 1 / sqrt(head_dim) is taken in f64 there
    // What the singe-kernel surface's dense family adds (all off by default).  Positions: query q sits at
    // query_start + q and key k at key_start + k; the causal mask, the window (key + window <= query hidden) and
    // `lookahead` (key > query + lookahead hidden; -1 = none) compare those.  The output is multiplied by
    // output_scale; a row that saw no key leaves `empty_lse` as its log-sum-exp.
    int64_t query_start = 0, key_start = 0, lookahead = -1;
    float output_scale = 1.0f, empty_lse = -__builtin_inff();
    // Keys behind a block table (block_table non-null): key k of batch b is slot k % block_size of block
    // block_table[b * table_stride + k / block_size], at block * key_block_stride (value_block_stride) + slot *
    // key_strides[2] + kv_head * key_strides[1]; a block id outside the cache hides the key.
    const uint32_t* block_table = nullptr;
    uint32_t block_size = 0, physical_blocks = 0, table_stride = 0;
    uint64_t key_block_stride = 0, value_block_stride = 0;
    // Ragged sequences (ragged != 0): rows are (token, head) pairs of `batch` sequences packed along the position
    // axis; sequence s owns query tokens sequence_offsets[s] .. + query_lengths[s] and keys sequence_offsets[s] .. +
    // kv_lengths[s] of the packed key / value tensors, clamped to total_kv_tokens; query_len is the total token
    // count, lse is [tokens, heads]; a token no sequence owns is left alone.
    uint32_t ragged = 0, total_kv_tokens = 0;
    const int32_t* query_lengths = nullptr;
    const int32_t* kv_lengths = nullptr;
    const int32_t* sequence_offsets = nullptr;
};

// singe_paged_attention_general_*: the paged ops for any element type and head dimension.  `form`: the FlashInfer
// form with i32 (0) or i64 (1) paging vectors (bottom-right causal, base-two lse, -inf for an empty row), or the
// block-table form of the singe-kernel surface (top-left causal, natural-log lse, -1e20 for an empty row): prefill (2:
// pages = the table, query_offsets / query_lengths / last_page_lengths = per-sequence i32 offsets, query counts and
// key counts) and decode (3: one query per sequence at row `sequence`, last_page_lengths = the key counts, clamped
// to what a table row addresses).
struct GeneralPagedArgs {
    const void* query_rows;         // [tokens, heads, head_dim]
    const void* key_cache;          // [cache_pages, page_size, kv_heads, head_dim]
    const void* value_cache;
    const void* query_offsets;
    const void* page_offsets;
    const void* pages;
    const void* last_page_lengths;
    const void* query_lengths;      // form 2 only
    void* output;                   // [tokens, heads, head_dim]
    float* lse;                     // [tokens, heads], or null
    uint32_t* status;
    int64_t window;
    uint32_t tokens, heads, kv_heads, head_dim, page_size, sequences, cache_pages, page_table;
    uint32_t row_blocks;            // workgroups (4 rows each) per sequence
    uint32_t causal, has_softcap, form;
    float scale, softcap;
    double scale_wide;              // the scale for f64 tensors: the default 1 / sqrt(head_dim) is taken in f64 there
};

// singe_paged_mla_attention_general_*: contiguous operands of one element type.
struct LatentAttentionArgs {
    const void* latent_queries;      // [tokens, heads, latent_dim]
    const void* positional_queries;  // [tokens, heads, position_dim]
    const void* latent_cache;        // [cache_pages, page_size, latent_dim]
    const void* positional_cache;    // [cache_pages, page_size, position_dim]
    const void* query_offsets;
    const void* page_offsets;
    const void* pages;
    const void* last_page_lengths;
    void* output;                    // [tokens, heads, latent_dim]
    float* lse;                      // [tokens, heads] base two, or null
    uint32_t* status;
    uint32_t tokens, heads, latent_dim, position_dim, page_size, sequences, cache_pages, page_table;
    uint32_t row_blocks;             // workgroups per sequence (4 rows each; 128 each on the matrix-core kernel)
    uint32_t causal, wide_index;
    float scale;
    // Matrix-core kernel with key splits (splits > 1): each of a row tile's `splits` workgroups leaves its rows
    // normalised in partial_out [splits, tokens, heads, latent_dim] with a base-two log-sum-exp in partial_lse
    // [splits, tokens, heads] (-inf and zeros for a share without keys); singe_paged_mla_attention_combine_* merges.
    uint32_t splits;
    int32_t page_shift;              // log2(page_size) when that is a power of two, else -1 (matrix-core kernel)
    float* partial_out;
    float* partial_lse;
    uint32_t unit_band;              // matrix-core kernel: neighbouring units (row tiles) that go to one XCD together
};

// singe_rotary_cache_write_*: contiguous operands of one element type; angles may be f32.
struct RotaryCacheArgs {
    const void* query;          // [tokens, query_heads, dim] or null when query_heads is 0
    const void* key;            // [tokens, cache_heads, dim]
    const void* value;          // [tokens, cache_heads, dim]
    const void* cos;            // [tokens, dim / 2]
    const void* sin;
    const void* pages;          // [tokens] i32 or i64
    const void* slots;
    const void* query_weight;   // [dim] or null
    const void* key_weight;
    void* query_out;            // [tokens, query_heads, dim]
    void* key_cache;            // [cache_pages, page_slots, cache_heads, dim]
    void* value_cache;
    uint32_t* status;
    uint32_t tokens, query_heads, cache_heads, head_dim, cache_pages, page_slots;
    uint32_t table_type;        // element type of cos / sin
    uint32_t wide_index;
    uint32_t has_query_norm, has_key_norm;
    float query_eps, key_eps;
    // The 16-byte kernels (singe_rotary_cache_write_chunks_*): a head's lanes that hold data, and the power of two of
    // neighbouring lanes it is dealt to.
    uint32_t head_lanes, group_lanes;
};

// singe_paged_decode_rows_{i32,i64}: a decode step given as FlashInfer CSR paging -> one row per token for the decode
// kernels: where the token's page list starts in `pages` and how many keys it sees.  The decode kernels read 32-bit
// page ids: i64 paging is copied into `pages32` on the way (an id outside the cache as 0xffffffff).
struct DecodeRowsArgs {
    const void* query_offsets;      // [sequences + 1]
    const void* page_offsets;       // [sequences + 1]
    const void* pages;              // [page_table]
    const void* last_page_lengths;  // [sequences]
    uint32_t* row_starts;           // [tokens]
    int32_t* lengths;               // [tokens]: -1 for a token no valid sequence owns
    uint32_t* pages32;              // [page_table] (i64 paging), else null
    uint32_t* row_begins;           // [tokens] (a window), else null: keys of the row's first page that lie before the window
    uint32_t* status;
    uint32_t tokens, sequences, page_table, page_size, cache_pages, causal;
    int32_t window;                 // a token sees the `window` keys up to its own position; -1: all of them
};

// singe_paging_indices_*: FlashInfer CSR paging -> block-table paging.
struct PagingIndicesArgs {
    const void* query_offsets;      // [sequences + 1]
    const void* page_offsets;       // [sequences + 1]
    const void* pages;              // [page_count]
    const void* last_page_lengths;  // [sequences]
    int32_t* packed_offsets;        // [sequences + 1]: first element of each sequence's queries
    int32_t* query_lengths;         // [sequences]
    int32_t* key_lengths;           // [sequences]
    int32_t* page_table;            // [sequences, width]
    uint32_t* status;
    uint32_t sequences, tokens, page_count, page_size, cache_pages, width;
    uint64_t row_elements;          // elements of one query token: heads * dim
};
