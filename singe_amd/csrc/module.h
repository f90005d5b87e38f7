// Code-object handling: the gfx950 image, its per-device hipModule_t, and the kernel handles.
// Stands in for the reference's Context::load_module / Module::function pair
// (singe-cuda/src/context.rs:363-385, singe-cuda/src/module/mod.rs:387-410).
#pragma once

#include "hip_runtime_loader.h"

namespace singe_hip {

// Kernels of the code object, in the order of kKernelNames.
enum KernelId : int {
    // bf16 paged decode: index = 2 * (block size not a multiple of 16) + (two head groups per wave)
    kDecodeBf16 = 0,
    kDecodeCombine = 4,
    // f16 paged decode: the four bf16 forms in the same order, then their combine
    kDecodeF16, kDecodeF16Combine = kDecodeF16 + 4,
    // fp8 decode, dense form: + (block size not a multiple of 16) + 2 * relaxed
    kDecodeF8Wide, kDecodeF8WideAny, kDecodeF8WideRelaxed, kDecodeF8WideRelaxedAny,
    kPrefillCausal, kPrefillFull, kPrefillCausalF16, kPrefillFullF16,
    // the same four with the dense op's mask, window and cap
    kPrefillCausalOptions, kPrefillFullOptions, kPrefillCausalOptionsF16, kPrefillFullOptionsF16,
    kPrefillF32D32, kPrefillF32D64, kPrefillF32D128, kPrefillF32D256,
    // paged attention: + 4 when the page size is a power of two of at least 16 keys
    kPagedAttentionI32, kPagedAttentionI64, kPagedAttentionSoftcapI32, kPagedAttentionSoftcapI64,
    kPagedAttentionI32P16, kPagedAttentionI64P16, kPagedAttentionSoftcapI32P16, kPagedAttentionSoftcapI64P16,
    kPagedKvPrefill, kPagedKvPrefillP16, kPagedKvPrefillF16, kPagedKvPrefillF16P16,
    kPagedAttentionCombineI32, kPagedAttentionCombineI64, kPagedAttentionCombineF16I32, kPagedAttentionCombineF16I64,
    // f16 paged attention: same order as the eight bf16 kernels from kPagedAttentionI32
    kPagedAttentionF16,
    // fused query rotation: + (i64 indices) + 2 * (page size a power of two of at least 16 keys)
    kRotaryPagedAttention = kPagedAttentionF16 + 8, kRotaryPagedAttentionI64, kRotaryPagedAttentionP16, kRotaryPagedAttentionI64P16,
    kSplitKReduce,
    // dense f32 split-KV decode: + head dimension (4, 8, 16, 32, 64, 128, 256)
    kFmhaDecodeSplitK, kFmhaDecodeSplitKLast = kFmhaDecodeSplitK + 6,
    // f32 block-table decode (split over keys) and prefill, same seven head dimensions each
    kPagedKvDecodeSplitKF32, kPagedKvDecodeSplitKF32Last = kPagedKvDecodeSplitKF32 + 6,
    kPagedKvPrefillF32, kPagedKvPrefillF32Last = kPagedKvPrefillF32 + 6,
    kPrefillRowsF32, kPrefillRowsF32Last = kPrefillRowsF32 + 6,
    kRotaryCacheF32, kRotaryCacheBf16, kRotaryCacheF16,
    kPagingIndicesI32, kPagingIndicesI64,
    // latent (MLA) attention: + element (f32, bf16, f16)
    kLatentGeneral, kLatentGeneralBf16, kLatentGeneralF16,
    // the same at latent width 512, positional width 64 on the matrix cores
    kLatentTilesBf16, kLatentTilesF16, kLatentCombineBf16, kLatentCombineF16,
    // general kernels: index = base + 3 * element (f32, bf16, f16) + width (64, 128, 256)
    kDenseGeneral,
    kPagedGeneral = kDenseGeneral + 9,
    // the register-only product loop a prefill kernel is priced against
    kMfmaCeilingBf16 = kPagedGeneral + 9, kMfmaCeilingF16,
    // the matrix-core kernels built for head_dim 64, each bank in the order of its head_dim 128 forms: the ten
    // bf16 / f16 decode kernels from kDecodeBf16, the eight dense prefill kernels from kPrefillCausal, the paged
    // attention kernels from kPagedAttentionI32 up to kSplitKReduce
    kDecodeD64, kPrefillD64 = kDecodeD64 + 10, kPagedD64 = kPrefillD64 + 8,
    // the merge of the dense kernels' key splits: bf16, f16, then the same for head_dim 64
    kPrefillCombine = kPagedD64 + (kSplitKReduce - kPagedAttentionI32), kPrefillCombineF16, kPrefillCombineD64, kPrefillCombineF16D64,
    // the general kernels on f64 tensors: + width (64, 128, 256)
    kDenseGeneralF64, kPagedGeneralF64 = kDenseGeneralF64 + 3,
    // the plain streaming read a decode kernel is priced against
    kHbmStreamRead = kPagedGeneralF64 + 3,
    // the dense prefill and paged attention kernels built for the other multiples of 16 (32, 96, 16, 48, 80, 112, in
    // that order), each bank in the order of its head_dim 128 forms: eight dense kernels, their two merges, the
    // paged kernels up to kSplitKReduce
    kOtherHeadDims,
    // bf16 / f16 paged decode at head_dim 128 with five to eight query heads per kv head, dense form:
    // + (block size not a multiple of 16) + 2 * f16
    kDecodeWide = kOtherHeadDims + 6 * (10 + (kSplitKReduce - kPagedAttentionI32)),
    // the decode merge for rows with many slots: bf16, f16, then the same for head_dim 64
    kDecodeCombineMany = kDecodeWide + 4, kDecodeCombineManyF16, kDecodeCombineManyD64, kDecodeCombineManyF16D64,
    // rotate-and-append sixteen bytes at a time: f32, bf16, f16
    kRotaryCacheChunks, kRotaryCacheChunksBf16, kRotaryCacheChunksF16,
    // the decode merge for rows with one or two slots: bf16, f16, then the same for head_dim 64
    kDecodeCombineFew, kDecodeCombineFewF16, kDecodeCombineFewD64, kDecodeCombineFewF16D64,
    // a decode step in FlashInfer form -> one row per token for the decode kernels
    kPagedDecodeRows, kPagedDecodeRowsI64,
    // the fused query rotation beyond bf16 without a cap, twelve kernels per head dimension in the order 128, 64, then
    // the other multiples of 16 as in kOtherHeadDims: + 4 * (bf16 with a cap, f16, f16 with a cap) + (i64 indices)
    // + 2 * (page size a power of two of at least 16 keys)
    kRotaryPagedAttentionMore,
    // latent (MLA) attention on the matrix cores at the other widths (latent a multiple of 32 up to 512, positional a
    // multiple of 8 up to 64): bf16, f16, then their merges
    kLatentTilesAnyBf16 = kRotaryPagedAttentionMore + 8 * 12, kLatentTilesAnyF16, kLatentCombineAnyBf16, kLatentCombineAnyF16,
    // the bf16 / f16 decode kernels built for the other multiples of 16 (32, 16, 48, 80, 96, 112, in that order),
    // fourteen each: the ten from kDecodeBf16 in their order, then the merges for rows with many slots (bf16, f16)
    // and with one or two (bf16, f16)
    kDecodeOtherHeadDims,
    // the dense prefill that gives a wave two 32-row tiles (head_dim 128, no options): + (no causal mask) + 2 * f16
    // + 4 * (key_len not a multiple of 64)
    kPrefillPair = kDecodeOtherHeadDims + 6 * 14,
    // the paged attention op on the same two-tile loop (head_dim 128, page sizes that are powers of two from 16, no
    // options): + (i64 indices) + 2 * f16 + 4 * (the query's norm and rotation fused in)
    kPagedPair = kPrefillPair + 8,
    // the head_dim 64 builds of the two-tile dense prefill, in kPrefillPair's order
    kPrefillPairD64 = kPagedPair + 8,
    // the head_dim 64 builds of the two-tile paged attention, in kPagedPair's order
    kPagedPairD64 = kPrefillPairD64 + 8,
    // and the head_dim 96 builds of both
    kPrefillPairD96 = kPagedPairD64 + 8,
    kPagedPairD96 = kPrefillPairD96 + 8,
    // and those for 112, 80, 48, 32, 16: sixteen each, the dense eight first
    kPairOtherHeadDims = kPagedPairD96 + 8,
    kKernelCount = kPairOtherHeadDims + 5 * 16
};

// The two-tile kernels (fmha_prefill_pair.hip, paged_attention_pair.hip) have a build for every multiple of 16 up to 128.
inline bool has_pair_build(long long head_dim) { return head_dim >= 16 && head_dim <= 128 && head_dim % 16 == 0; }
// The first of the eight dense (or paged) two-tile kernels built for a head dimension.
inline int pair_kernels_at(long long head_dim, bool paged) {
    if (head_dim == 128) return paged ? kPagedPair : kPrefillPair;
    if (head_dim == 64) return paged ? kPagedPairD64 : kPrefillPairD64;
    if (head_dim == 96) return paged ? kPagedPairD96 : kPrefillPairD96;
    const int order = head_dim == 112 ? 0 : head_dim == 80 ? 1 : head_dim == 48 ? 2 : head_dim == 32 ? 3 : 4;
    return kPairOtherHeadDims + 16 * order + (paged ? 8 : 0);
}


// The head_dim 64 build of a matrix-core kernel named by its head_dim 128 id.
inline KernelId at_head_dim_64(KernelId kernel) {
    if (kernel < kDecodeF8Wide) return static_cast<KernelId>(kDecodeD64 + kernel);
    if (kernel >= kPrefillCausal && kernel < kPrefillF32D32) return static_cast<KernelId>(kPrefillD64 + (kernel - kPrefillCausal));
    return static_cast<KernelId>(kPagedD64 + (kernel - kPagedAttentionI32));
}

// Whether the bf16 / f16 decode kernels have a matrix-core build for a head dimension.
inline bool has_decode_build(long long head_dim) { return head_dim >= 16 && head_dim <= 128 && head_dim % 16 == 0; }

// The bank of the decode builds for a head dimension other than 128 and 64.
inline int other_decode_bank(long long head_dim) {
    const int order = head_dim == 32 ? 0 : head_dim == 16 ? 1 : head_dim == 48 ? 2 : head_dim == 80 ? 3 : head_dim == 96 ? 4 : 5;
    return kDecodeOtherHeadDims + 14 * order;
}

// That build of a bf16 / f16 decode kernel or of its one-wave merge, named by its head_dim 128 id below kDecodeF8Wide.
inline KernelId decode_at_head_dim(KernelId kernel, long long head_dim) {
    if (head_dim == 128) return kernel;
    return static_cast<KernelId>((head_dim == 64 ? static_cast<int>(kDecodeD64) : other_decode_bank(head_dim)) + kernel);
}

// The decode merges for rows with many slots (eight waves a row) and with one or two (four rows a fetch): + 1 for f16.
inline KernelId decode_combine_many_at(long long head_dim) {
    return head_dim == 128 ? kDecodeCombineMany : head_dim == 64 ? kDecodeCombineManyD64 : static_cast<KernelId>(other_decode_bank(head_dim) + 10);
}
inline KernelId decode_combine_few_at(long long head_dim) {
    return head_dim == 128 ? kDecodeCombineFew : head_dim == 64 ? kDecodeCombineFewD64 : static_cast<KernelId>(other_decode_bank(head_dim) + 12);
}

// Whether the dense prefill and paged attention kernels have a matrix-core build for a head dimension.
inline bool has_matrix_core_build(long long head_dim) { return head_dim >= 16 && head_dim <= 128 && head_dim % 16 == 0; }

// The bank of the builds for a head dimension other than 128 and 64.
inline int other_head_dim_bank(long long head_dim) {
    const int order = head_dim == 32 ? 0 : head_dim == 96 ? 1 : head_dim == 16 ? 2 : head_dim == 48 ? 3 : head_dim == 80 ? 4 : 5;
    return kOtherHeadDims + order * (10 + (kSplitKReduce - kPagedAttentionI32));
}

// That build of a dense prefill or paged attention kernel named by its head_dim 128 id (decode kernels: 64 only).
inline KernelId at_head_dim(KernelId kernel, long long head_dim) {
    if (head_dim == 128) return kernel;
    if (head_dim == 64) return at_head_dim_64(kernel);
    const bool dense = kernel >= kPrefillCausal && kernel < kPrefillF32D32;
    const int bank = other_head_dim_bank(head_dim);
    return static_cast<KernelId>(dense ? bank + (kernel - kPrefillCausal) : bank + 10 + (kernel - kPagedAttentionI32));
}

// The merge kernel of the dense kernels' key splits for a head dimension (+ 1 for f16).
inline KernelId prefill_combine_at(long long head_dim) {
    if (head_dim == 128) return kPrefillCombine;
    if (head_dim == 64) return kPrefillCombineD64;
    return static_cast<KernelId>(other_head_dim_bank(head_dim) + 8);
}

// The fused-rotation kernel for an element type, a cap and a head dimension, before the index / page form is added.
inline int rotary_paged_attention_base(bool f16, bool softcap, long long head_dim) {
    if (!f16 && !softcap) return at_head_dim(kRotaryPagedAttention, head_dim);
    const int order = head_dim == 128 ? 0 : head_dim == 64 ? 1 : 2 + (other_head_dim_bank(head_dim) - kOtherHeadDims) / (10 + (kSplitKReduce - kPagedAttentionI32));
    return kRotaryPagedAttentionMore + 12 * order + 4 * ((f16 ? 2 : 0) + (softcap ? 1 : 0) - 1);
}

extern const char* const kKernelNames[kKernelCount];

// Parts of the code object (one file each) and the part a kernel lives in.
constexpr int kPartCount = 52;
extern const char* const kPartNames[kPartCount];
int kernel_part(int kernel);

// Status of the thread's last failure (see singe_hip_last_error).
int32_t fail(int32_t status, const char* name = "", uint64_t minimum = 0, uint64_t actual = 0);
int32_t fail_hip(hipError_t error, const char* what);

// The handle of `kernel` on the current device, loading the module there on first use.
// Returns 0 and sets *function, or a status.
int32_t kernel_function(KernelId kernel, hipFunction_t* function);

// Compute units of the current device (256 when the runtime does not say).
unsigned compute_units();

// hipModuleLaunchKernel of a kernel that takes one argument block by value.
template <class Args>
int32_t launch(KernelId kernel, unsigned grid_x, unsigned grid_y, unsigned grid_z, unsigned threads,
               hipStream_t stream, Args& args, unsigned shared_bytes = 0) {
    hipFunction_t function = nullptr;
    if (int32_t status = kernel_function(kernel, &function)) return status;
    void* params[] = {&args};
    hipError_t error = hip_runtime()->hipModuleLaunchKernel(function, grid_x, grid_y, grid_z, threads, 1, 1,
                                                            shared_bytes, stream, params, nullptr);
    return error == hipSuccess ? 0 : fail_hip(error, kKernelNames[kernel]);
}

}  // namespace singe_hip
