// Argument blocks shared by the host launcher and the gfx950 kernels.  Each kernel takes exactly one
// of these by value, so host and device agree on the layout by construction (plain fixed-width C
// types only; both sides include this header).
#pragma once

#include <stdint.h>

struct DecodeArgs {
    const uint16_t* query;          // [batch, heads, 128] bf16
    const uint16_t* key_cache;      // [blocks, block_size, kv_heads, 128] bf16
    const uint16_t* value_cache;
    const int32_t* actual_seq_lens; // [batch]
    const uint32_t* block_table;    // [batch, stride]
    float* partial_out;             // [batch, heads, splits, 128]
    float* partial_lse;             // [batch, heads, splits], natural log
    uint32_t heads;
    uint32_t kv_heads;
    uint32_t block_size;
    int32_t block_shift;            // log2(block_size) when it is a power of two, else -1
    uint32_t physical_blocks;
    uint32_t block_table_batch_stride;
    uint32_t splits;                // scratch rows per (batch, head)
    uint32_t keys_per_split;        // multiple of 32
    float scale_log2e;              // scale * log2(e)
};

struct CombineArgs {
    uint16_t* out;                  // [batch, heads, dim] bf16
    const float* partial_out;       // [batch, heads, splits, dim]
    const float* partial_lse;       // [batch, heads, splits]
    const int32_t* actual_seq_lens;
    uint32_t heads;
    uint32_t dim;
    uint32_t splits;
    uint32_t keys_per_split;
    uint32_t reach;                 // block_table_batch_stride * block_size
};
