/*
 * singe_hip_attention.h: C ABI of the MI355X (gfx950) attention kernels.
 *
 * This is the layer a `singe-kernel-sys`-style binding links against (the reference keeps that crate
 * as an empty placeholder: singe-kernel-sys/src/lib.rs:1-6).  Every entry point takes plain device
 * pointers, element counts and a #[repr(C)]-compatible config struct; nothing here allocates device
 * memory, synchronises, or owns a buffer.  Work is enqueued on the caller's HIP stream and completes
 * asynchronously, so every call is legal during stream capture
 * (raw kernel execution contract: singe-kernel/src/cuda/mod.rs:3-12).
 *
 * The kernels live in a gfx950 code object built in parts (singe_attention_gfx950.<part>.hsaco, hipcc --genco)
 * that this library loads with hipModuleLoadData and launches with hipModuleLaunchKernel, in place of
 * the reference's NVRTC -> cuModuleLoadData -> cuLaunchKernelEx path
 * (singe/src/backend/cuda/codegen/compile.rs:43-190, singe-cuda/src/module/mod.rs:2117-2132).
 * The HIP runtime's entry points are resolved with dlopen on first use, as the reference's sys crates do
 * (singe-loader/src/lib.rs:298-322), from the copy of libamdhip64 the process already holds: the library links that
 * runtime for the one hipcc-built unit that carries its fixed device scratch, and refuses to run on two copies.
 *
 * Return value of every int32_t function: 0 = success; a positive SingeHipStatus = a validation
 * failure found before launch (mirrors singe-kernel/src/error.rs:12-186); a negative value =
 * -(hipError_t) from the HIP runtime.
 */
#ifndef SINGE_HIP_ATTENTION_H
#define SINGE_HIP_ATTENTION_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SINGE_HIP_API __attribute__((visibility("default")))

typedef enum SingeHipStatus {
    SINGE_HIP_OK = 0,
    SINGE_HIP_INVALID_LENGTH = 1,        /* Error::InvalidLength: zero extent, heads % kv_heads != 0, non-finite scale */
    SINGE_HIP_LENGTH_TOO_SHORT = 2,      /* Error::LengthTooShort { name, minimum, actual } */
    SINGE_HIP_LENGTH_EXCEEDS_I32 = 3,    /* Error::LengthExceedsI32 */
    SINGE_HIP_SIZE_OVERFLOW = 4,         /* Error::SizeOverflow */
    SINGE_HIP_UNSUPPORTED_WIDTH = 5,     /* Error::UnsupportedWidth { op, width } */
    SINGE_HIP_NULL_POINTER = 6,          /* Error::NullPointer */
    SINGE_HIP_KERNEL_NOT_PREPARED = 7,   /* Error::KernelNotPrepared: code object missing or not loadable */
    SINGE_HIP_UNSUPPORTED_CONFIGURATION = 8, /* Error::UnsupportedConfiguration { op, reason } */
    SINGE_HIP_INVALID_ARGUMENT = 9,      /* singe::Error::InvalidArgument (shape / dtype rules of the singe op) */
    SINGE_HIP_RUNTIME_UNAVAILABLE = 10,  /* the HIP runtime library could not be opened */
    SINGE_HIP_TUNE_CACHE_MISS = 11,      /* Error::TuneCacheMiss { op }: TuningChoice::Cached without a cached entry */
    SINGE_HIP_AUTOTUNE_DURING_CAPTURE = 12, /* Error::AutotuneDuringCapture { op } */
    SINGE_HIP_NO_TUNE_CANDIDATES = 13,   /* Error::NoTuneCandidates { op } */
    SINGE_HIP_NO_SUCCESSFUL_TUNE_CANDIDATES = 14, /* Error::NoSuccessfulTuneCandidates { op } */
    SINGE_HIP_STALE_RECORD = 15          /* singe::Error::StaleRecord { key }: parameters the kernels do not take */
} SingeHipStatus;

/* Details of the last non-zero status returned on the calling thread. */
typedef struct SingeHipErrorDetail {
    int32_t status;
    const char* name;      /* buffer or parameter the failure is about; static string, never NULL */
    uint64_t minimum;      /* LengthTooShort: required element count; UnsupportedWidth: the width */
    uint64_t actual;       /* LengthTooShort: supplied element count */
} SingeHipErrorDetail;
SINGE_HIP_API void singe_hip_last_error(SingeHipErrorDetail* detail);
SINGE_HIP_API const char* singe_hip_status_string(int32_t status);

/* ---- code object management -------------------------------------------------------------------
 * Replaces Context::load_module / Module::function (singe-cuda/src/context.rs:363-385,
 * singe-cuda/src/module/mod.rs:387-410) and the kernel cache of CudaRuntime::kernel
 * (singe/src/backend/cuda/codegen/compile.rs:43-190).  The kernels are built as parts, one gfx950 code object per
 * kernel source and build (singe_hip_kernel lists which kernel lives in which part).  Loading is per process; a part's
 * module is instantiated lazily on each device that launches from it.  Without an explicit load the library looks for
 * singe_attention_gfx950.<part>.hsaco next to itself when a kernel of the part is first launched.  An embedding
 * caller hands the bytes over instead (they are copied):
 *   singe_hip_load_part(part, image, bytes)   one part's code object, by the part's name;
 *   singe_hip_load(image, bytes)              an archive of parts as the build writes it (singe_attention_gfx950.parts:
 *                                             16 bytes "SINGE_HIP_PARTS\0", u32 version = 1, u32 entries, then per
 *                                             entry char part[48], u64 offset, u64 bytes; little-endian, offsets from
 *                                             the archive's first byte), which replaces the parts it lists; any other
 *                                             image is taken as ONE code object (or clang offload bundle) that holds
 *                                             every kernel;
 *   singe_hip_load_file(path)                 the same from a file.
 * Parts no load has supplied are still looked for next to the library.  A malformed archive changes nothing and returns
 * SINGE_HIP_INVALID_LENGTH / SINGE_HIP_INVALID_ARGUMENT / SINGE_HIP_LENGTH_TOO_SHORT.  Launches read their kernel handle
 * without a lock once it has been resolved on their device (the first launch of a kernel there, or singe_hip_prepare,
 * takes a mutex); a load or unload drops the handles and modules it replaces, so it must not run while another thread
 * launches, as with cuModuleUnload. */
SINGE_HIP_API int32_t singe_hip_load(const void* image, size_t bytes);
SINGE_HIP_API int32_t singe_hip_load_part(const char* part, const void* image, size_t bytes);
SINGE_HIP_API int32_t singe_hip_load_file(const char* path);
SINGE_HIP_API void singe_hip_unload(void);
/* Resolves every kernel of the image on the current device; returns the number found through *count. */
SINGE_HIP_API int32_t singe_hip_prepare(int32_t* count);
/* The kernels the library launches, as profilers report them (the reference names its artifacts the same way,
 * singe/src/backend/cuda/kernel_plan/source/mod.rs:841-853), and the part of the code object each one is loaded from
 * (singe_attention_gfx950.<part>.hsaco).  index from 0; SINGE_HIP_INVALID_ARGUMENT past the last kernel. */
SINGE_HIP_API int32_t singe_hip_kernel(int32_t index, const char** name, const char** part);

/* ---- singe-kernel surface: paged decode ---------------------------------------------------------
 * Mirrors PagedKvDecodeAttentionConfig (singe-kernel/src/cuda/attention/mod.rs:76-90). */
typedef struct SingePagedKvDecodeAttentionConfig {
    size_t batch;
    size_t heads;
    size_t kv_heads;
    size_t head_dim;
    size_t block_size;
    size_t physical_blocks;
    size_t block_table_batch_stride;
    float scale;
} SingePagedKvDecodeAttentionConfig;

/* validate_paged_kv_decode_attention_config (mod.rs:2963-2985). */
SINGE_HIP_API int32_t singe_hip_paged_kv_decode_attention_config_validate(const SingePagedKvDecodeAttentionConfig* config);

/* Scratch the split-KV decode needs, in bytes: one normalised partial row (f32) and natural-log LSE
 * per (kv head, key range, sequence the range touches), plus the per-sequence tile prefix the reduce
 * step reads; caller-supplied like the reference's split-KV scratch (mod.rs:2456-2539).  Depends on
 * the device's compute-unit count.  0 on an invalid config. */
SINGE_HIP_API size_t singe_hip_paged_kv_decode_attention_workspace_bytes(const SingePagedKvDecodeAttentionConfig* config);

/* paged_kv_decode_attention_bf16 (singe-kernel/src/cuda/attention/paged.rs:210-249).
 * out/query [batch, heads, dim] bf16; caches [physical_blocks, block_size, kv_heads, dim] bf16;
 * actual_seq_lens [batch] i32; block_table [batch, stride] u32.  *_len are element counts and are
 * checked as PagedKvDecodeAttentionConfig::validate_lengths does (mod.rs:711-743).
 * workspace: device scratch of at least ..._workspace_bytes(config), 256-byte aligned; it carries no
 * state between calls. */
SINGE_HIP_API int32_t singe_hip_paged_kv_decode_attention_bf16(
    void* stream,
    uint16_t* out, size_t out_len,
    const uint16_t* query, size_t query_len,
    const uint16_t* key_cache, size_t key_cache_len,
    const uint16_t* value_cache, size_t value_cache_len,
    const int32_t* actual_seq_lens, size_t actual_seq_lens_len,
    const uint32_t* block_table, size_t block_table_len,
    void* workspace, size_t workspace_bytes,
    const SingePagedKvDecodeAttentionConfig* config);

/* paged_kv_decode_attention_f16 (paged.rs): the same kernels on f16 operands (v_mfma_f32_16x16x32_f16); same
 * workspace size and rules. */
SINGE_HIP_API int32_t singe_hip_paged_kv_decode_attention_f16(
    void* stream,
    uint16_t* out, size_t out_len,
    const uint16_t* query, size_t query_len,
    const uint16_t* key_cache, size_t key_cache_len,
    const uint16_t* value_cache, size_t value_cache_len,
    const int32_t* actual_seq_lens, size_t actual_seq_lens_len,
    const uint32_t* block_table, size_t block_table_len,
    void* workspace, size_t workspace_bytes,
    const SingePagedKvDecodeAttentionConfig* config);

/* The bf16 decode above for callers that cannot allocate (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc).  No counterpart in the reference: its split-KV scratch is always the
 * caller's.  Same kernels, same results bit for bit, but the scratch is a fixed array of
 * SINGE_HIP_STATIC_SCRATCH_BYTES in device memory that the library's device image carries (each GPU the library
 * runs on holds it until the process ends); the call allocates and frees nothing.  A config whose scratch
 * (..._workspace_bytes) exceeds that returns SINGE_HIP_LENGTH_TOO_SHORT naming "static scratch" (minimum = bytes
 * needed, actual = the fixed size).  The array's address is resolved on the first call on a device (or by
 * singe_hip_prepare), which must not run under stream capture.  All calls on a GPU share the one array, which keeps
 * the last call's contents (the kernels need none of it cleared): calls that overlap on one GPU race. */
#define SINGE_HIP_STATIC_SCRATCH_BYTES (16u << 20)
SINGE_HIP_API int32_t singe_hip_paged_kv_decode_attention_no_alloc_bf16(
    void* stream,
    uint16_t* out, size_t out_len,
    const uint16_t* query, size_t query_len,
    const uint16_t* key_cache, size_t key_cache_len,
    const uint16_t* value_cache, size_t value_cache_len,
    const int32_t* actual_seq_lens, size_t actual_seq_lens_len,
    const uint32_t* block_table, size_t block_table_len,
    const SingePagedKvDecodeAttentionConfig* config);

/* The same operation run phase by phase, as the reference exposes its split kernel and splitk_reduce
 * separately (singe-kernel/src/cuda/attention/fmha.rs:1038,1155): SPLIT fills the scratch with the
 * normalised partial rows and natural-log LSEs of every key range; REDUCE folds the scratch into
 * `out` (cpu/attention.rs:2157-2193).  Both bits = the call above. */
#define SINGE_HIP_DECODE_SPLIT 1u
#define SINGE_HIP_DECODE_REDUCE 2u
SINGE_HIP_API int32_t singe_hip_paged_kv_decode_attention_phases_bf16(
    void* stream,
    uint16_t* out, size_t out_len,
    const uint16_t* query, size_t query_len,
    const uint16_t* key_cache, size_t key_cache_len,
    const uint16_t* value_cache, size_t value_cache_len,
    const int32_t* actual_seq_lens, size_t actual_seq_lens_len,
    const uint32_t* block_table, size_t block_table_len,
    void* workspace, size_t workspace_bytes,
    const SingePagedKvDecodeAttentionConfig* config,
    uint32_t phases);

/* The same decode over an fp8 e4m3 KV cache: caches hold one code per element, key_scales and
 * value_scales [physical_blocks, kv_heads] f32 hold one scale per (block, kv head).  The kernel
 * widens the cache in registers: every element is read as bf16_rne(f8e4m3_value(code) * scale)
 * (singe-kernel/src/cpu/quantization.rs:245-280 for value * scale), i.e. exactly what the bf16 entry
 * point computes on the dequantised cache.  The reference has no entry point of this kind; the
 * argument order follows the bf16 one with the scales after the caches.  `phases` as above. */
SINGE_HIP_API int32_t singe_hip_paged_kv_decode_attention_f8e4m3kv_bf16(
    void* stream,
    uint16_t* out, size_t out_len,
    const uint16_t* query, size_t query_len,
    const uint8_t* key_cache, size_t key_cache_len,
    const uint8_t* value_cache, size_t value_cache_len,
    const float* key_scales, size_t key_scales_len,
    const float* value_scales, size_t value_scales_len,
    const int32_t* actual_seq_lens, size_t actual_seq_lens_len,
    const uint32_t* block_table, size_t block_table_len,
    void* workspace, size_t workspace_bytes,
    const SingePagedKvDecodeAttentionConfig* config,
    uint32_t phases);

/* Numerical policy, the counterpart of NumericalPolicy { precision: Full | Relaxed }
 * (singe/src/graph/numerics/mod.rs:6-49).  Full (0, the default): fp8 elements are rounded to bf16
 * after scaling, one by one.  Relaxed (non-zero): fp8 codes are widened exactly and the block scale is
 * applied once per key to its score / probability, which is cheaper and not bit-identical. */
SINGE_HIP_API void singe_hip_set_relaxed_numerics(int32_t relaxed);
SINGE_HIP_API int32_t singe_hip_relaxed_numerics(void);

/* Tuning knob of the split-KV decode: the number of equal key ranges each kv head's keys are cut
 * into (0 = one workgroup per compute unit).  The counterpart of
 * FmhaDecodeSplitKReduceConfig::max_splits / TuningChoice::Explicit
 * (singe-kernel/src/cuda/attention/mod.rs:2364-2380).  Changes what ..._workspace_bytes returns. */
SINGE_HIP_API void singe_hip_set_decode_workers(uint32_t workers);
SINGE_HIP_API uint32_t singe_hip_decode_workers(const SingePagedKvDecodeAttentionConfig* config);

/* The same choices for the calling thread alone.  The setters above and below (relaxed numerics, decode workers,
 * paged / MLA key splits, the installed SingeAttentionParameters) are process-wide defaults; the reference keeps its
 * numerical policy per thread (thread_local! NUMERICAL_POLICY, singe/src/graph/numerics/mod.rs:44-49) and carries
 * tuning choices in the call (TuningChoice::Explicit, singe-kernel/src/cuda/attention/mod.rs:2364-2380).  A thread
 * that installs options reads them in every size query (*_workspace_bytes, *_scratch_bytes, singe_hip_decode_workers)
 * and every launch it makes afterwards, whatever other threads set meanwhile, so the scratch a thread sized is the
 * scratch its launch expects.  A field at its "follow" value takes the process-wide setting.  NULL clears the thread's
 * options.  Returns SINGE_HIP_INVALID_ARGUMENT for relaxed_numerics outside -1 .. 1 or more than 64 splits. */
typedef struct SingeHipThreadOptions {
    int32_t relaxed_numerics;             /* -1 = follow; 0 = full; 1 = relaxed */
    uint32_t decode_workers;              /* 0 = follow; otherwise as singe_hip_set_decode_workers */
    uint32_t paged_attention_splits;      /* 0 = follow; 1 .. 64 as singe_hip_set_paged_attention_splits */
    uint32_t paged_mla_attention_splits;  /* 0 = follow; 1 .. 64 as singe_hip_set_paged_mla_attention_splits */
    uint8_t has_split_below_blocks;       /* 0 = follow the installed SingeAttentionParameters */
    uint64_t split_below_blocks;          /* AttentionParameters::split_below_blocks for this thread's calls */
} SingeHipThreadOptions;
SINGE_HIP_API int32_t singe_hip_set_thread_options(const SingeHipThreadOptions* options);
SINGE_HIP_API void singe_hip_thread_options(SingeHipThreadOptions* options);

/* ---- singe-kernel surface: paged prefill ----------------------------------------------------------
 * Mirrors PagedKvPrefillAttentionConfig (singe-kernel/src/cuda/attention/mod.rs:92-108). */
typedef struct SingePagedKvPrefillAttentionConfig {
    size_t batch;
    size_t total_query_tokens;
    size_t heads;
    size_t kv_heads;
    size_t head_dim;
    size_t block_size;
    size_t physical_blocks;
    size_t block_table_batch_stride;
    uint8_t causal;   /* Rust bool: 0 or 1 */
    float scale;
} SingePagedKvPrefillAttentionConfig;

/* validate_paged_kv_prefill_attention_config (mod.rs:2987-3011). */
SINGE_HIP_API int32_t singe_hip_paged_kv_prefill_attention_config_validate(const SingePagedKvPrefillAttentionConfig* config);

/* paged_kv_prefill_attention_bf16 (singe-kernel/src/cuda/attention/paged.rs:370-420; CPU form
 * cpu/attention.rs:1248-1341).  query/out [total_query_tokens, heads, dim] bf16, packed over the batch:
 * sequence b holds tokens actual_seq_offsets[b] .. + actual_seq_lens_q[b] and reads the first
 * actual_seq_lens_kv[b] keys of the blocks in row b of block_table [batch, stride] u32.  Causal hides
 * key index > query index (queries align with the FIRST keys).  lse [total_query_tokens, heads] f32,
 * natural log, -1e20 for a row that sees no key.  Rows of tokens no sequence covers are not written.
 * A sequence whose offsets or lengths would address outside the buffers is skipped.  Lengths are
 * checked as PagedKvPrefillAttentionConfig::validate_lengths does (mod.rs:786-818). */
SINGE_HIP_API int32_t singe_hip_paged_kv_prefill_attention_bf16(
    void* stream,
    uint16_t* out, size_t out_len,
    float* lse, size_t lse_len,
    const uint16_t* query, size_t query_len,
    const uint16_t* key_cache, size_t key_cache_len,
    const uint16_t* value_cache, size_t value_cache_len,
    const int32_t* actual_seq_lens_q, size_t actual_seq_lens_q_len,
    const int32_t* actual_seq_lens_kv, size_t actual_seq_lens_kv_len,
    const int32_t* actual_seq_offsets, size_t actual_seq_offsets_len,
    const uint32_t* block_table, size_t block_table_len,
    const SingePagedKvPrefillAttentionConfig* config);

/* paged_kv_prefill_attention_f16 (paged.rs): the same kernel on f16 operands (v_mfma_f32_32x32x16_f16). */
SINGE_HIP_API int32_t singe_hip_paged_kv_prefill_attention_f16(
    void* stream,
    uint16_t* out, size_t out_len,
    float* lse, size_t lse_len,
    const uint16_t* query, size_t query_len,
    const uint16_t* key_cache, size_t key_cache_len,
    const uint16_t* value_cache, size_t value_cache_len,
    const int32_t* actual_seq_lens_q, size_t actual_seq_lens_q_len,
    const int32_t* actual_seq_lens_kv, size_t actual_seq_lens_kv_len,
    const int32_t* actual_seq_offsets, size_t actual_seq_offsets_len,
    const uint32_t* block_table, size_t block_table_len,
    const SingePagedKvPrefillAttentionConfig* config);

/* ---- singe-kernel surface: dense prefill ---------------------------------------------------------
 * Mirrors FmhaPrefillConfig (singe-kernel/src/cuda/attention/mod.rs:253-274); strides in elements.
 * FmhaPrefillConfig::contiguous (mod.rs:1602-1632) fills them for packed [batch, len, heads, dim]. */
typedef struct SingeFmhaPrefillConfig {
    size_t batch;
    size_t query_len;
    size_t key_len;
    size_t heads;
    size_t kv_heads;
    size_t head_dim;
    size_t query_batch_stride;
    size_t key_batch_stride;
    size_t value_batch_stride;
    size_t output_batch_stride;
    size_t query_sequence_stride;
    size_t key_sequence_stride;
    size_t value_sequence_stride;
    size_t output_sequence_stride;
    size_t query_head_stride;
    size_t key_head_stride;
    size_t value_head_stride;
    size_t output_head_stride;
    float scale;
    uint8_t causal;   /* Rust bool: 0 or 1 */
} SingeFmhaPrefillConfig;

/* Tuning knob of the dense bf16 / f16 prefill at the multiples of 16 up to 128: the query rows a wave takes.  32: four waves share a
 * compute unit's SIMDs two by two, 128 rows a workgroup.  64: a wave has a SIMD to itself and folds every key block
 * into two 32-row tiles, 256 rows a workgroup; only calls without a mask, a window, a cap or key splits (sinks and
 * key lengths are taken) with a positive scale have this form, others keep 32.  0 (the default): 64 where the call has that form,
 * its 256-row tiles still fill the chip and the head dimension is one the form is faster at (64 and up; 48 without
 * the causal mask).  Results are the same up to the order in which a row's
 * reference point moves.  The counterpart of AttentionParameters::{warps, min_blocks}
 * (singe/src/backend/cuda/kernel_plan/source/parameters.rs:21-57). */
SINGE_HIP_API void singe_hip_set_dense_prefill_rows_per_wave(uint32_t rows);
/* What a bf16 / f16 call of this shape without options takes: 32 or 64 rows a wave, 0 when the head dimension has no
 * matrix-core build (the one-wave-per-row kernel). */
SINGE_HIP_API uint32_t singe_hip_dense_prefill_rows_per_wave(const SingeFmhaPrefillConfig* config);

/* validate_fmha_prefill_config (mod.rs:3369-3398). */
SINGE_HIP_API int32_t singe_hip_fmha_prefill_config_validate(const SingeFmhaPrefillConfig* config);

/* fmha_prefill_bf16 (singe-kernel/src/cuda/attention/fmha.rs:744-790): out = softmax(scale * Q K^T
 * [+ top-left causal mask]) V, query head h reading kv head h / (heads / kv_heads).
 * Lengths are checked as FmhaPrefillConfig::validate_output_lengths does (mod.rs:1704-1756). */
SINGE_HIP_API int32_t singe_hip_fmha_prefill_bf16(
    void* stream,
    uint16_t* out, size_t out_len,
    const uint16_t* query, size_t query_len,
    const uint16_t* key, size_t key_len,
    const uint16_t* value, size_t value_len,
    const SingeFmhaPrefillConfig* config);

/* fmha_prefill_lse_bf16 (fmha.rs:638-690): also writes lse [batch, heads, query_len], the natural-log
 * sum of exponentials of each row's scaled scores (cpu/attention.rs:1810-1811). */
SINGE_HIP_API int32_t singe_hip_fmha_prefill_lse_bf16(
    void* stream,
    uint16_t* out, size_t out_len,
    float* lse, size_t lse_len,
    const uint16_t* query, size_t query_len,
    const uint16_t* key, size_t key_len,
    const uint16_t* value, size_t value_len,
    const SingeFmhaPrefillConfig* config);

/* fmha_prefill_f16 / fmha_prefill_lse_f16 (fmha.rs, the f16 twins of the two calls above): the same kernels on
 * v_mfma_f32_32x32x16_f16; operands and outputs are IEEE half bit patterns. */
SINGE_HIP_API int32_t singe_hip_fmha_prefill_f16(
    void* stream,
    uint16_t* out, size_t out_len,
    const uint16_t* query, size_t query_len,
    const uint16_t* key, size_t key_len,
    const uint16_t* value, size_t value_len,
    const SingeFmhaPrefillConfig* config);
SINGE_HIP_API int32_t singe_hip_fmha_prefill_lse_f16(
    void* stream,
    uint16_t* out, size_t out_len,
    float* lse, size_t lse_len,
    const uint16_t* query, size_t query_len,
    const uint16_t* key, size_t key_len,
    const uint16_t* value, size_t value_len,
    const SingeFmhaPrefillConfig* config);

/* f32 forms for any head_dim up to 256 (fmha_prefill_f32 / fmha_prefill_lse_f32: fmha.rs:48-190).
 * The f32 correctness anchor: dense causal [1, 8, 512, 64] attention in [batch, heads, len, dim]
 * order is this call with batch stride heads*len*dim, head stride len*dim, sequence stride dim. */
SINGE_HIP_API int32_t singe_hip_fmha_prefill_f32(
    void* stream,
    float* out, size_t out_len,
    const float* query, size_t query_len,
    const float* key, size_t key_len,
    const float* value, size_t value_len,
    const SingeFmhaPrefillConfig* config);
SINGE_HIP_API int32_t singe_hip_fmha_prefill_lse_f32(
    void* stream,
    float* out, size_t out_len,
    float* lse, size_t lse_len,
    const float* query, size_t query_len,
    const float* key, size_t key_len,
    const float* value, size_t value_len,
    const SingeFmhaPrefillConfig* config);

/* Mirrors SoftcappedWindowAttentionConfig (mod.rs:292-296); Option<f32> soft_cap is the pair
 * (has_soft_cap, soft_cap).  window_size 0 = no window, otherwise keys more than window_size away
 * from the query on either side are hidden (cpu/attention.rs:1864-1869). */
typedef struct SingeSoftcappedWindowAttentionConfig {
    SingeFmhaPrefillConfig attention;
    size_t window_size;
    uint8_t has_soft_cap;
    float soft_cap;
} SingeSoftcappedWindowAttentionConfig;

/* softcapped_window_attention_f32 (fmha.rs:245-290; CPU form cpu/attention.rs:1835-1925). */
SINGE_HIP_API int32_t singe_hip_softcapped_window_attention_f32(
    void* stream,
    float* out, size_t out_len,
    const float* query, size_t query_len,
    const float* key, size_t key_len,
    const float* value, size_t value_len,
    const SingeSoftcappedWindowAttentionConfig* config);

/* ---- singe surface: paged attention in FlashInfer form ---------------------------------------------
 * Operation::PagedAttention (singe/src/tensor/neural.rs:409-457): ragged queries [tokens, heads, dim]
 * over caches [cache_pages, page_size, kv_heads, dim]; sequence b holds queries
 * query_offsets[b] .. query_offsets[b+1] and the keys of pages pages[page_offsets[b] .. page_offsets[b+1]],
 * all full but the last, which holds last_page_lengths[b].  Queries are a sequence's last tokens
 * (bottom-right causal).  The extents the reference bakes into the generated source are runtime values
 * here; the attributes are ScaledDotProductAttentionAttributes
 * (singe/src/backend/registry/attributes/mod.rs:288-303) with each Option as a (has_, value) pair. */
#define SINGE_HIP_INDEX_I32 0
#define SINGE_HIP_INDEX_I64 1
typedef struct SingePagedAttentionProblem {
    int64_t tokens;        /* query_rows.shape[0] */
    int64_t heads;
    int64_t kv_heads;
    int64_t head_dim;
    int64_t page_size;     /* cache.shape[1] */
    int64_t sequences;     /* last_page_lengths.len */
    int64_t cache_pages;   /* cache.shape[0] */
    int64_t page_table;    /* pages.len */
    int32_t index_type;    /* SINGE_HIP_INDEX_I32 or _I64, for all four index operands */
    uint8_t causal;
    uint8_t has_scale;     /* Option<f32> scale, default 1 / sqrt(head_dim) */
    uint8_t has_window;    /* Option<i64> window: key j is hidden from position i when j + window <= i */
    uint8_t has_softcap;   /* Option<f32> softcap: softcap * tanh(score / softcap) on the scaled scores */
    float scale;
    float softcap;
    int64_t window;
} SingePagedAttentionProblem;

/* The kernel artifact "singe_paged_attention" (kernel_plan/source/paged_attention.rs:544-868), with
 * its ABI order: inputs, outputs, status (paged_attention.rs:687-715).  output [tokens, heads, dim]
 * bf16; lse [tokens, heads] f32, base two, -inf for a row that sees no key (may be null: the fused
 * variants do not read it).  status: device u32, zeroed by the caller, set to 1
 * (STATUS_INDEX_OUT_OF_BOUNDS: singe/src/backend/kernel_lowering/mod.rs:40-61) by the first paging
 * value found outside its buffers; may be null (it is while a stream is being captured:
 * kernel_plan/mod.rs:176-197), and nothing is ever read through a bad value. */
SINGE_HIP_API int32_t singe_hip_paged_attention_bf16(
    void* stream,
    const uint16_t* query_rows,
    const uint16_t* key_cache,
    const uint16_t* value_cache,
    const void* query_offsets,
    const void* page_offsets,
    const void* pages,
    const void* last_page_lengths,
    uint16_t* output,
    float* lse,
    uint32_t* status,
    const SingePagedAttentionProblem* problem);

/* The same op with scratch for key splits.  With few query rows (decoding, short chunks) one workgroup per
 * (sequence, kv head, 128 packed rows) cannot fill the chip and the longest sequence sets the time; given
 * scratch, the keys of a row tile are shared out over several workgroups, each leaving a normalised f32
 * partial and its log-sum-exp, and a second kernel merges them (the scheme of the reference's own split
 * kernels, which declare such scratch in their plan: kernel_plan/source/mla.rs:232-241, 497-560).
 * singe_hip_paged_attention_scratch_bytes says how much this problem wants (0: it would not split);
 * with a null or smaller buffer the call runs unsplit, exactly as singe_hip_paged_attention_bf16.  The scratch
 * holds nothing between calls; calls that share it must not overlap.  Results equal the unsplit ones up to
 * the order of summation.  singe_hip_set_paged_attention_splits fixes the number of shares (0 = chosen by
 * problem size, the default), the counterpart of TuningChoice::Explicit
 * (singe-kernel/src/cuda/attention/mod.rs:2364-2380); it changes what ..._scratch_bytes returns.
 * A decode step (no more tokens than sequences, head_dim a multiple of 16 up to 128, no softcap, no window below 2048 keys) given
 * scratch on a 256-byte boundary runs on the block-table decode kernels instead, which cut the keys of all
 * sequences into equal ranges: a first kernel checks the paging vectors (same status word) and gives each token
 * its page list and key count, and the scratch then also holds those and the decode kernels' partial rows.  The
 * result is the same up to the order of summation; a fixed number of shares keeps such a call on the row-tile kernel. */
SINGE_HIP_API size_t singe_hip_paged_attention_scratch_bytes(const SingePagedAttentionProblem* problem);
SINGE_HIP_API void singe_hip_set_paged_attention_splits(uint32_t splits);
/* Packed rows a wave of the bf16 / f16 paged attention kernels takes, as singe_hip_set_dense_prefill_rows_per_wave: 32,
 * 64 (only calls at a head_dim that is a multiple of 16 up to 128 with a page size that is a power of two of at least 16 keys and a positive scale,
 * without a softcap, a window or key splits have that form, with or without the fused query rotation; others keep
 * 32), or 0 (the default): 64 where the call has that form and its 256-row tiles still fill the chip. */
SINGE_HIP_API void singe_hip_set_paged_attention_rows_per_wave(uint32_t rows);
/* What a bf16 / f16 call of this problem takes when it is given scratch: 32 or 64 rows a wave,
 * 0 when the head dimension has no matrix-core build. */
SINGE_HIP_API uint32_t singe_hip_paged_attention_rows_per_wave(const SingePagedAttentionProblem* problem);
SINGE_HIP_API int32_t singe_hip_paged_attention_scratch_bf16(
    void* stream,
    const uint16_t* query_rows,
    const uint16_t* key_cache,
    const uint16_t* value_cache,
    const void* query_offsets,
    const void* page_offsets,
    const void* pages,
    const void* last_page_lengths,
    uint16_t* output,
    float* lse,
    uint32_t* status,
    void* scratch,
    size_t scratch_bytes,
    const SingePagedAttentionProblem* problem);

SINGE_HIP_API int32_t singe_hip_paged_attention_scratch_f16(
    void* stream,
    const uint16_t* query_rows,
    const uint16_t* key_cache,
    const uint16_t* value_cache,
    const void* query_offsets,
    const void* page_offsets,
    const void* pages,
    const void* last_page_lengths,
    uint16_t* output,
    float* lse,
    uint32_t* status,
    void* scratch,
    size_t scratch_bytes,
    const SingePagedAttentionProblem* problem);

/* The same op over a query the kernel normalises and rotates itself, the counterpart of
 * KernelPlanner::rotary_paged_attention (singe/src/backend/cuda/kernel_plan/source/paged_attention.rs:533-542,
 * query stage :881-977; operand order :687-715: the attention's inputs, the output, then cos, sin and the
 * norm's weight, then the status word).  `query_rows` holds the query BEFORE its rotation; cos and sin are
 * [tokens, head_dim / 2] of `table_type` (the angles of each token, shared by its heads); pairs are half-split,
 * (p, p + head_dim / 2): first = a cos - b sin, second = b cos + a sin, after an optional RMS norm over the head
 * dimension (x * rsqrt(mean(x^2) + eps)) times an optional weight [head_dim] of the query's type; the rotated
 * query is rounded to the query's type before the products, as the reference rounds what it stages.
 * Fused wherever the reference fuses (paged_attention.rs:512-531 with takes_tensor_cores, tensor_core.rs:18-32): bf16
 * or f16 tensors at a head dimension that is a multiple of 16 up to 128, with or without a softcap, any window.  At odd
 * multiples of 16 a pair's two dims sit in the two lanes of a query row and change hands with one lane swap per word.
 * Other head dimensions return SINGE_HIP_UNSUPPORTED_WIDTH and take singe_hip_rotary_cache_write followed by
 * singe_hip_paged_attention_*, the two-step form the reference plans for them too.
 * `lse` may be null (the reference's fused kernel keeps it in scratch). */
typedef struct SingeQueryRotation {
    int32_t table_type;   /* SINGE_HIP_F32, SINGE_HIP_BF16 or SINGE_HIP_F16 */
    uint8_t has_norm;
    float eps;
} SingeQueryRotation;

SINGE_HIP_API int32_t singe_hip_rotary_paged_attention_bf16(
    void* stream,
    const uint16_t* query_rows,
    const uint16_t* key_cache,
    const uint16_t* value_cache,
    const void* query_offsets,
    const void* page_offsets,
    const void* pages,
    const void* last_page_lengths,
    const void* cos,
    const void* sin,
    const uint16_t* query_weight,
    uint16_t* output,
    float* lse,
    uint32_t* status,
    const SingePagedAttentionProblem* problem,
    const SingeQueryRotation* rotation);

/* The same for f16 tensors (query, caches, weight and output are f16 bit patterns). */
SINGE_HIP_API int32_t singe_hip_rotary_paged_attention_f16(
    void* stream,
    const uint16_t* query_rows,
    const uint16_t* key_cache,
    const uint16_t* value_cache,
    const void* query_offsets,
    const void* page_offsets,
    const void* pages,
    const void* last_page_lengths,
    const void* cos,
    const void* sin,
    const uint16_t* query_weight,
    uint16_t* output,
    float* lse,
    uint32_t* status,
    const SingePagedAttentionProblem* problem,
    const SingeQueryRotation* rotation);

/* The same op for f32 and f16 tensors, and (through the bf16 entry point above) for bf16 at head
 * dimensions other than 128, up to 256: the general kernel, one wave per (token, head) row, f32
 * arithmetic whatever the storage type (kernel_plan/source/paged_general.rs:73-247; CPU form
 * singe/src/backend/cpu/normalization/attention.rs:297-330, 424-538). */
SINGE_HIP_API int32_t singe_hip_paged_attention_f32(
    void* stream,
    const float* query_rows,
    const float* key_cache,
    const float* value_cache,
    const void* query_offsets,
    const void* page_offsets,
    const void* pages,
    const void* last_page_lengths,
    float* output,
    float* lse,
    uint32_t* status,
    const SingePagedAttentionProblem* problem);
/* f64 tensors, computed in f64 as the CPU path and the reference's general kernel do (paged_general.rs:91-99); the
 * log-sum-exp stays f32. */
SINGE_HIP_API int32_t singe_hip_paged_attention_f64(
    void* stream,
    const double* query_rows,
    const double* key_cache,
    const double* value_cache,
    const void* query_offsets,
    const void* page_offsets,
    const void* pages,
    const void* last_page_lengths,
    double* output,
    float* lse,
    uint32_t* status,
    const SingePagedAttentionProblem* problem);
SINGE_HIP_API int32_t singe_hip_paged_attention_f16(
    void* stream,
    const uint16_t* query_rows,
    const uint16_t* key_cache,
    const uint16_t* value_cache,
    const void* query_offsets,
    const void* page_offsets,
    const void* pages,
    const void* last_page_lengths,
    uint16_t* output,
    float* lse,
    uint32_t* status,
    const SingePagedAttentionProblem* problem);

/* ---- singe surface: dense scaled-dot-product attention ----------------------------------------------
 * Operation::ScaledDotProductAttention (singe/src/tensor/neural.rs:92-190; CPU form
 * singe/src/backend/cpu/normalization/attention.rs:191-276; shape rules spec/neural/attention.rs:209-290):
 * query [batch, heads, query_len, head_dim], key [batch, kv_heads, key_len, head_dim], value
 * [batch, kv_heads, key_len, value_dim], output [batch, heads, query_len, value_dim], all contiguous and
 * of one element type; query head h reads kv head h / (heads / kv_heads).  Causal hides key > query
 * (top-left), window hides key + window <= query, softcap caps the scaled scores, then `mask` (element
 * type of the query, read through mask_strides over (batch, head, query, key), 0 = broadcast) adds to
 * them; `sinks` [heads] joins each row's softmax without weighing a value; `key_lengths` [batch] i32
 * hides the keys past each batch's count (a count of zero gives zeros).  mask, sinks and key_lengths may
 * be null.  head_dim and value_dim up to 256.  bf16 and f16 at head_dim = value_dim = 128 run on the matrix-core
 * flash kernel of fmha_prefill_* with every option (a mask, a window or a cap take its block-by-block masked path);
 * other widths and f32 on the vector-unit kernel.  A row whose every key is hidden gives zeros (the CPU form
 * divides zero by zero there). */
#define SINGE_HIP_F32 0
#define SINGE_HIP_BF16 1
#define SINGE_HIP_F16 2
#define SINGE_HIP_F64 3   /* the vector-unit kernels only, with f64 arithmetic (attention.rs:63-69; paged_general.rs:91-99) */
typedef struct SingeAttentionProblem {
    int64_t batch;
    int64_t heads;
    int64_t kv_heads;
    int64_t query_len;
    int64_t key_len;
    int64_t head_dim;
    int64_t value_dim;
    int64_t mask_strides[4];
    int32_t data_type;     /* SINGE_HIP_F32, _BF16, _F16 or _F64 */
    uint8_t causal;
    uint8_t has_scale;
    uint8_t has_window;
    uint8_t has_softcap;
    float scale;
    float softcap;
    int64_t window;
} SingeAttentionProblem;

SINGE_HIP_API int32_t singe_hip_scaled_dot_product_attention(
    void* stream,
    const void* query,
    const void* key,
    const void* value,
    const void* mask,
    const void* sinks,
    const int32_t* key_lengths,
    void* output,
    const SingeAttentionProblem* problem);

/* The same op with scratch for key splits (the reference's fused_attention plans the same: few blocks and many keys
 * split the keys into chunks attended separately and combined after, singe/src/backend/cuda/kernel_plan/source/
 * attention.rs:283-292, 420-452, 588-654).  A decode-shaped call (few query rows, many keys) has one workgroup per
 * (batch, head) and cannot fill the chip; given scratch, bf16 / f16 calls at a head_dim that is a multiple of 16 up to
 * 128 share the keys of a
 * query tile out over several workgroups, each leaving a normalised f32 partial and its base-two log-sum-exp, and a
 * second kernel merges them (sinks join the first share).  ..._scratch_bytes says how much the problem wants (0: it
 * would not split, by SingeAttentionParameters.split_below_blocks and the key count); with a null or smaller buffer,
 * and for every other type and width, the call is singe_hip_scaled_dot_product_attention.  The scratch holds nothing
 * between calls; calls that share it must not overlap. */
SINGE_HIP_API size_t singe_hip_scaled_dot_product_attention_scratch_bytes(const SingeAttentionProblem* problem);
SINGE_HIP_API int32_t singe_hip_scaled_dot_product_attention_scratch(
    void* stream,
    const void* query,
    const void* key,
    const void* value,
    const void* mask,
    const void* sinks,
    const int32_t* key_lengths,
    void* output,
    void* scratch,
    size_t scratch_bytes,
    const SingeAttentionProblem* problem);

/* ---- singe surface: the choices the attention kernels leave open ----------------------------------------
 * AttentionParameters (singe/src/backend/cuda/kernel_plan/source/parameters.rs:21-57), field for field.  On gfx950:
 *   warps               4: a workgroup is four waves of 32 query rows; nothing else is built
 *   key_tile            64: keys per LDS stage; nothing else is built
 *   stages              1 or 2: both name the one pipeline the kernels have (LDS always holds the tiles to come:
 *                       three stages of K, two of V), so a record tuned to either runs the same code
 *   split_below_blocks  a launch of fewer workgroups than this splits its keys, into
 *                       min(ceil(2 * split_below_blocks / workgroups), ceil(keys / (4 * key_tile)), 16) shares
 *                       (attention.rs:283-292), given scratch; 0 never splits.  Default: twice the compute units
 *   min_blocks          none, or 2: the kernels are built with two workgroups per compute unit
 * ..._candidates lists what the kernels take on the current device, the default first, as attention_candidates does
 * (attention.rs:113-160); ..._set installs one of them for the paged op and the dense op of this process (null: the
 * default) and returns SINGE_HIP_STALE_RECORD for anything else, as the reference refuses a record whose parameters
 * its kernel no longer takes (parameters.rs:245-250) instead of quietly running the default. */
typedef struct SingeAttentionParameters {
    size_t warps;
    size_t key_tile;
    size_t stages;
    size_t split_below_blocks;
    uint8_t has_min_blocks;   /* Option<u32> min_blocks */
    uint32_t min_blocks;
} SingeAttentionParameters;
SINGE_HIP_API void singe_hip_attention_parameters_default(SingeAttentionParameters* parameters);
SINGE_HIP_API int32_t singe_hip_attention_candidates(SingeAttentionParameters* candidates, size_t capacity, size_t* count);
SINGE_HIP_API int32_t singe_hip_set_attention_parameters(const SingeAttentionParameters* parameters);
SINGE_HIP_API void singe_hip_attention_parameters(SingeAttentionParameters* parameters);
/* parameter_key (parameters.rs:221-230): the key a tuning record of the op is stored under,
 * "kernel|<label>|<numerical policy>|<attributes>" followed by " <type><dimensions><strides>+<offset % 8>" per
 * operand, spelled as Rust's Debug spells them, for contiguous operands at offset 0: label "paged_attention" with
 * its seven operands, or "attention" with query, key, value (a mask, sinks and key lengths are flags of the
 * attributes).  Writes at most capacity bytes, NUL included, and returns the length the whole key needs without it
 * (0 on a null problem). */
SINGE_HIP_API size_t singe_hip_paged_attention_parameter_key(const SingePagedAttentionProblem* problem, int32_t data_type,
                                                             char* buffer, size_t capacity);
SINGE_HIP_API size_t singe_hip_attention_parameter_key(const SingeAttentionProblem* problem, int32_t masked, int32_t sinks,
                                                       int32_t key_lengths, char* buffer, size_t capacity);

/* ---- singe-kernel surface: split-KV reduce -----------------------------------------------------------
 * Mirrors SplitKReduceConfig (singe-kernel/src/cuda/attention/mod.rs:385-398); strides in elements.
 * SplitKReduceConfig::contiguous (mod.rs:2312-2328) fills them for attn [batch, heads, splits, dim],
 * lse [batch, heads, splits], out [batch, heads, dim]. */
typedef struct SingeSplitKReduceConfig {
    size_t batch;
    size_t heads;
    size_t splits;
    size_t head_dim;
    size_t attn_batch_stride;
    size_t attn_head_stride;
    size_t attn_split_stride;
    size_t lse_batch_stride;
    size_t lse_head_stride;
    size_t output_batch_stride;
    size_t output_head_stride;
} SingeSplitKReduceConfig;

/* splitk_reduce_f32 (singe-kernel/src/cuda/attention/fmha.rs:1038-1067; CPU form
 * cpu/attention.rs:2157-2193): out = sum_s exp(lse_s - max) * attn_s / sum_s exp(lse_s - max), natural
 * log.  Lengths are checked as SplitKReduceConfig::validate_lengths does (mod.rs:2330-2361). */
SINGE_HIP_API int32_t singe_hip_splitk_reduce_f32(
    void* stream,
    float* out, size_t out_len,
    const float* attn_splitk, size_t attn_splitk_len,
    const float* lse_splitk, size_t lse_splitk_len,
    const SingeSplitKReduceConfig* config);

/* ---- f32 forms of the two block-table ops -------------------------------------------------------------
 * paged_kv_decode_attention_f32 and paged_kv_prefill_attention_f32 (singe-kernel/src/cuda/attention/paged.rs; CPU
 * forms singe-kernel/src/cpu/attention.rs:1172-1246, 1248-1341), same operands, config structs and length checks
 * as the bf16 entry points above, f32 throughout.  head_dim 4, 8, 16, 32, 64 (the reference's set for these
 * kernels, cutile/attention/paged.rs:799-810) and 128, 256.  Vector-unit kernels: accuracy anchors at 1e-4, HBM
 * bound for decode, not the matrix-core path.  A sequence length beyond what its table row can name is cut
 * there and a table entry beyond the cache is read as the last block (the reference checks neither).
 * Decode splits the keys of each (sequence, kv head) over workgroups and combines with the split-KV reduce;
 * its scratch is caller-supplied: ..._f32_workspace_bytes(config), 16-byte aligned, no state between calls.
 * Prefill writes every token row: zeros and an LSE of 0 for a token no sequence covers (what the CPU form's
 * zero-filled outputs hold there), zeros and -1e20 for a covered row without visible keys. */
SINGE_HIP_API size_t singe_hip_paged_kv_decode_attention_f32_workspace_bytes(const SingePagedKvDecodeAttentionConfig* config);

SINGE_HIP_API int32_t singe_hip_paged_kv_decode_attention_f32(
    void* stream,
    float* out, size_t out_len,
    const float* query, size_t query_len,
    const float* key_cache, size_t key_cache_len,
    const float* value_cache, size_t value_cache_len,
    const int32_t* actual_seq_lens, size_t actual_seq_lens_len,
    const uint32_t* block_table, size_t block_table_len,
    void* workspace, size_t workspace_bytes,
    const SingePagedKvDecodeAttentionConfig* config);

SINGE_HIP_API int32_t singe_hip_paged_kv_prefill_attention_f32(
    void* stream,
    float* out, size_t out_len,
    float* lse, size_t lse_len,
    const float* query, size_t query_len,
    const float* key_cache, size_t key_cache_len,
    const float* value_cache, size_t value_cache_len,
    const int32_t* actual_seq_lens_q, size_t actual_seq_lens_q_len,
    const int32_t* actual_seq_lens_kv, size_t actual_seq_lens_kv_len,
    const int32_t* actual_seq_offsets, size_t actual_seq_offsets_len,
    const uint32_t* block_table, size_t block_table_len,
    const SingePagedKvPrefillAttentionConfig* config);

/* ---- dense f32 decode with split keys -----------------------------------------------------------------
 * The reference's split-KV convention (singe-kernel/src/cuda/attention/fmha.rs:1074-1250): a split kernel
 * writes one normalised partial output and one natural-log LSE per (batch, head, split) into scratch the
 * caller supplies, and splitk_reduce_f32 (above) combines them.  query / out [batch, heads, dim], key / value
 * [batch, key_len, kv_heads, dim], all f32, through element strides.  head_dim 4, 8, 16, 32, 64 (the reference's
 * set, cutile/attention/splitk.rs:124-139) and 128, 256; other widths give SINGE_HIP_UNSUPPORTED_WIDTH. */

/* Mirrors FmhaDecodeConfig (mod.rs:366-383); FmhaDecodeConfig::contiguous (mod.rs:2233-2261) fills the strides. */
typedef struct SingeFmhaDecodeConfig {
    size_t batch;
    size_t key_len;
    size_t heads;
    size_t kv_heads;
    size_t head_dim;
    size_t query_batch_stride;
    size_t key_batch_stride;
    size_t value_batch_stride;
    size_t output_batch_stride;
    size_t query_head_stride;
    size_t key_sequence_stride;
    size_t value_sequence_stride;
    size_t output_head_stride;
    size_t key_head_stride;
    size_t value_head_stride;
    float scale;
} SingeFmhaDecodeConfig;

/* Mirrors FmhaDecodeSplitKConfig (mod.rs:401-423; contiguous form mod.rs:2662-2697): split s covers keys
 * s * kv_len_per_split .. + kv_len_per_split, clipped to key_len. */
typedef struct SingeFmhaDecodeSplitKConfig {
    size_t batch;
    size_t key_len;
    size_t heads;
    size_t kv_heads;
    size_t splits;
    size_t kv_len_per_split;
    size_t head_dim;
    size_t query_batch_stride;
    size_t key_batch_stride;
    size_t value_batch_stride;
    size_t output_batch_stride;
    size_t query_head_stride;
    size_t key_sequence_stride;
    size_t value_sequence_stride;
    size_t output_head_stride;
    size_t output_split_stride;
    size_t key_head_stride;
    size_t value_head_stride;
    size_t lse_batch_stride;
    size_t lse_head_stride;
    float scale;
} SingeFmhaDecodeSplitKConfig;

/* fmha_decode_splitk_f32 (fmha.rs:1074-1118; kernel cutile/kernel/attention/local.rs:6127-6272): out[b, h, s, :]
 * is the softmax-weighted mean of the slice's values (zeros for an empty slice), lse[b, h, s] = max + ln(sum)
 * (-1e20 for an empty slice).  Lengths are checked as FmhaDecodeSplitKConfig::validate_lengths does
 * (mod.rs:2699-2760). */
SINGE_HIP_API int32_t singe_hip_fmha_decode_splitk_f32(
    void* stream,
    float* out, size_t out_len,
    float* lse, size_t lse_len,
    const float* query, size_t query_len,
    const float* key, size_t key_len,
    const float* value, size_t value_len,
    const SingeFmhaDecodeSplitKConfig* config);

/* TuningChoice<AttentionSplitKTuning> (singe-kernel/src/cuda/autotune.rs:77-89) and TuneOptions (:34-71,
 * defaults warmup 1, repeats 5, no candidate limit; zero repeats count as one). */
typedef enum SingeHipTuningChoice {
    SINGE_HIP_TUNING_DEFAULT = 0,  /* min(max_splits, key_len) splits */
    SINGE_HIP_TUNING_EXPLICIT = 1, /* explicit_splits; must be 1 .. min(max_splits, key_len) */
    SINGE_HIP_TUNING_CACHED = 2,   /* the cached winner, SINGE_HIP_TUNE_CACHE_MISS without one */
    SINGE_HIP_TUNING_TUNE = 3,     /* time the candidates on a cache miss, store and use the winner */
    SINGE_HIP_TUNING_RETUNE = 4    /* always time again */
} SingeHipTuningChoice;

typedef struct SingeHipTuneOptions {
    size_t warmup;
    size_t repeats;
    size_t max_candidates;
} SingeHipTuneOptions;

/* Mirrors FmhaDecodeSplitKReduceConfig (mod.rs:452-458). */
typedef struct SingeFmhaDecodeSplitKReduceConfig {
    SingeFmhaDecodeConfig decode;
    size_t max_splits;
    int32_t tuning;                /* SingeHipTuningChoice */
    size_t explicit_splits;        /* SINGE_HIP_TUNING_EXPLICIT */
    SingeHipTuneOptions options;   /* SINGE_HIP_TUNING_TUNE / RETUNE */
} SingeFmhaDecodeSplitKReduceConfig;

/* fmha_decode_splitk_reduce_f32 (fmha.rs:1155-1250): the split kernel into the caller's scratch, then the
 * reduce.  attn_scratch holds at least batch * heads * min(max_splits, key_len) * head_dim elements laid out
 * [batch, heads, splits, dim] for the split count in use, lse_scratch batch * heads * min(max_splits, key_len)
 * laid out [batch, heads, splits] (mod.rs:2456-2539).  Timing candidates synchronises the stream's events and is
 * refused while the stream is being captured (SINGE_HIP_AUTOTUNE_DURING_CAPTURE), also when the cache would
 * have answered, as in the reference (fmha.rs:1203-1207); winners are cached per process and device, keyed
 * by the extents, max_splits and the strides (TuneProblemKey::AttentionSplitK, mod.rs:2394-2413), and the winner is launched once more so `out`
 * holds its result. */
SINGE_HIP_API int32_t singe_hip_fmha_decode_splitk_reduce_f32(
    void* stream,
    float* out, size_t out_len,
    float* attn_scratch, size_t attn_scratch_len,
    float* lse_scratch, size_t lse_scratch_len,
    const float* query, size_t query_len,
    const float* key, size_t key_len,
    const float* value, size_t value_len,
    const SingeFmhaDecodeSplitKReduceConfig* config);

/* attention_splitk_candidates (mod.rs:2364-2380): {1, 2, 4, 8, 16, 32, 64} up to min(max_splits, key_len), and
 * that bound itself.  Writes at most `capacity` of them to `splits` (which may be NULL) and their number to
 * `count`. */
SINGE_HIP_API int32_t singe_hip_attention_splitk_candidates(
    const SingeFmhaDecodeSplitKReduceConfig* config, size_t* splits, size_t capacity, size_t* count);

/* The cached winner for this problem on the current device, 0 when there is none (autotune::cache().get,
 * mod.rs:2432-2441); and MemoryTuneCache::clear. */
SINGE_HIP_API int32_t singe_hip_fmha_decode_splitk_reduce_tuned_splits(
    const SingeFmhaDecodeSplitKReduceConfig* config, size_t* splits);
SINGE_HIP_API void singe_hip_clear_tune_cache(void);

/* ---- latent (MLA) attention over paged caches --------------------------------------------------------
 * Tensor::paged_mla_attention / Operation::PagedMlaAttention (singe/src/backend/spec/neural/attention.rs:453-497;
 * CPU singe/src/backend/cpu/normalization/attention.rs:540-679; kernel plan
 * singe/src/backend/cuda/kernel_plan/source/mla.rs, operands in its ABI order :219-230, status word :260).
 * Every head of a token attends over one shared latent cache [cache_pages, page_size, latent_dim], whose rows
 * are the keys, with a positional part [cache_pages, page_size, position_dim] beside them, and the values:
 * score = (q_latent . c_latent + q_positional . c_positional) * scale, scale = 1 / sqrt(latent_dim +
 * position_dim) unless given; output [tokens, heads, latent_dim] of the operands' type; lse [tokens, heads] f32
 * base two, -inf for a row without keys (may be null).  Paging, causal alignment and the status word are those
 * of singe_hip_paged_attention_*.  All operands contiguous, one element type; latent_dim <= 512 and
 * position_dim <= 128 (SINGE_HIP_UNSUPPORTED_WIDTH beyond).  bf16 and f16 at latent_dim 512 with position_dim 64
 * run on the matrix cores, 128 (token, head) rows of a sequence to a workgroup that share every cache tile; every
 * other shape on a vector-unit kernel, one wave per (token, head) row. */
typedef struct SingePagedMlaAttentionProblem {
    int64_t tokens;
    int64_t heads;
    int64_t latent_dim;
    int64_t position_dim;
    int64_t page_size;
    int64_t sequences;
    int64_t cache_pages;
    int64_t page_table;    /* entries of `pages` */
    int32_t data_type;     /* SINGE_HIP_F32, _BF16 or _F16 */
    int32_t index_type;    /* SINGE_HIP_INDEX_I32 or _I64 */
    uint8_t causal;
    uint8_t has_scale;
    float scale;
} SingePagedMlaAttentionProblem;

SINGE_HIP_API int32_t singe_hip_paged_mla_attention(
    void* stream,
    const void* latent_queries,
    const void* positional_queries,
    const void* latent_cache,
    const void* positional_cache,
    const void* query_offsets,
    const void* page_offsets,
    const void* pages,
    const void* last_page_lengths,
    void* output,
    float* lse,
    uint32_t* status,
    const SingePagedMlaAttentionProblem* problem);

/* The same op with scratch for key splits, for the shapes on the matrix cores.  A decode step or a short chunk has
 * one workgroup per 128 rows of a sequence, too few to fill the chip; given scratch, the keys of a row tile are
 * shared out over several workgroups, each leaving a normalised f32 partial and its base-two log-sum-exp, and a
 * second kernel merges them (the reference's plan declares such scratch and merges the same way:
 * kernel_plan/source/mla.rs:232-241, 497-560).  singe_hip_paged_mla_attention_scratch_bytes says how much this
 * problem wants (0: it would not split); with a null or smaller buffer the call runs unsplit, exactly as
 * singe_hip_paged_mla_attention.  The scratch, 16-byte aligned, holds nothing between calls; calls that share it
 * must not overlap.  Results equal the unsplit ones up to the order of summation.
 * singe_hip_set_paged_mla_attention_splits fixes the number of shares (0 = chosen by problem size, the default; at
 * most 64); it changes what ..._scratch_bytes returns. */
SINGE_HIP_API size_t singe_hip_paged_mla_attention_scratch_bytes(const SingePagedMlaAttentionProblem* problem);
SINGE_HIP_API void singe_hip_set_paged_mla_attention_splits(uint32_t splits);
SINGE_HIP_API int32_t singe_hip_paged_mla_attention_scratch(
    void* stream,
    const void* latent_queries,
    const void* positional_queries,
    const void* latent_cache,
    const void* positional_cache,
    const void* query_offsets,
    const void* page_offsets,
    const void* pages,
    const void* last_page_lengths,
    void* output,
    float* lse,
    uint32_t* status,
    void* scratch,
    size_t scratch_bytes,
    const SingePagedMlaAttentionProblem* problem);

/* ---- singe surface: the steps either side of paged attention ------------------------------------------
 * The fused rotate-and-append kernel "rotary_cache_write"
 * (singe/src/backend/cuda/kernel_plan/source/rotary_cache.rs:249-427): rotates query [tokens, query_heads,
 * dim] into query_out, rotates key [tokens, cache_heads, dim] into key_cache[page_index[t], slot_index[t]]
 * and copies value [tokens, cache_heads, dim] into value_cache at the same cell; caches are
 * [cache_pages, page_slots, cache_heads, dim] and only the selected cells are written.  Half-split pairs
 * (p, p + dim / 2) turn by the angles cos / sin [tokens, dim / 2] (of table_type): first = a cos - b sin,
 * second = b cos + a sin, after an optional RMS normalisation (scale = rsqrt(mean(x^2) + eps), times an
 * optional weight [dim]; rotary_cache.rs:92-185).  A negative page or slot counts from the end; one still
 * outside its extent sets *status to 1 and leaves the caches alone for that token (rotary_cache.rs:376-385).
 * Operands in the order of the reference kernel's ABI (rotary_cache.rs:52-66, 268-293); query, query_out
 * and the weights may be null (query_heads 0 when attention rotates its own query). */
typedef struct SingeRotaryCacheProblem {
    int64_t tokens;
    int64_t query_heads;
    int64_t cache_heads;
    int64_t head_dim;
    int64_t cache_pages;
    int64_t page_slots;
    int32_t data_type;    /* SINGE_HIP_F32, _BF16 or _F16: queries, keys, values, weights, caches */
    int32_t table_type;   /* cos and sin */
    int32_t index_type;   /* SINGE_HIP_INDEX_I32 or _I64: page_index and slot_index */
    uint8_t has_query_norm;
    uint8_t has_key_norm;
    float query_eps;
    float key_eps;
} SingeRotaryCacheProblem;

SINGE_HIP_API int32_t singe_hip_rotary_cache_write(
    void* stream,
    const void* query,
    const void* key,
    const void* value,
    const void* cos,
    const void* sin,
    const void* page_index,
    const void* slot_index,
    const void* query_weight,
    const void* key_weight,
    void* query_out,
    void* key_cache,
    void* value_cache,
    uint32_t* status,
    const SingeRotaryCacheProblem* problem);

/* The kernel "paged_cudnn_indices" (kernel_plan/source/paged_attention.rs:325-398): FlashInfer CSR paging
 * -> block-table paging.  Writes packed_offsets [sequences + 1] (first element of each sequence's queries:
 * token offset * row_elements), query_lengths and key_lengths [sequences], and page_table
 * [sequences, width] (a sequence's pages, zero-padded; width is the widest row the caller allows, pages past
 * it are dropped).  Offsets are clamped into [0, tokens] and made monotone, so everything written stays
 * inside its buffer whatever the input holds; a sequence or page id that the attention kernels would refuse
 * sets *status to 1 and gets zero keys / a zero entry. */
typedef struct SingePagingIndicesProblem {
    int64_t sequences;
    int64_t tokens;
    int64_t page_count;     /* pages.len */
    int64_t page_size;
    int64_t cache_pages;
    int64_t width;          /* page_table row length */
    int64_t row_elements;   /* elements of one query token: heads * dim */
    int32_t index_type;
} SingePagingIndicesProblem;

SINGE_HIP_API int32_t singe_hip_paging_indices(
    void* stream,
    const void* query_offsets,
    const void* page_offsets,
    const void* pages,
    const void* last_page_lengths,
    int32_t* packed_offsets,
    int32_t* query_lengths,
    int32_t* key_lengths,
    int32_t* page_table,
    uint32_t* status,
    const SingePagingIndicesProblem* problem);

/* A measurement aid with no counterpart in the reference: `iterations` rounds of 32 register-only
 * v_mfma_f32_32x32x16 products per wave (bf16, or f16 when `f16` is set), `workgroups` workgroups of four waves, on
 * operands read once from `operands` (16-byte chunks, taken modulo the buffer).  No LDS, no softmax, no memory traffic
 * inside the loop: the rate it reaches is the matrix cores' own ceiling on that data (the clock under such a loop is
 * set by power, and power by the operands' bits), which the prefill kernels are priced against beside the published
 * peak.  Flop per launch = workgroups * 4 * iterations * 32 * 32768.  `out` takes one float per lane. */
/* The same kind of aid for the memory-bound kernels: `workgroups` workgroups of 512 lanes stream `bytes` of `data`
 * once with 16-byte non-temporal loads, eight in flight per lane, and do nothing else; bytes / time is the streaming
 * read rate the decode kernels are priced against beside the published HBM peak.  `out` takes one word per lane. */
SINGE_HIP_API int32_t singe_hip_hbm_stream_read(void* stream, const void* data, size_t bytes, uint32_t* out, size_t out_len,
                                                uint32_t workgroups);
SINGE_HIP_API int32_t singe_hip_mfma_ceiling(void* stream, const void* operands, size_t operand_bytes, float* out,
                                             size_t out_len, uint32_t workgroups, uint32_t iterations, int32_t f16);

/* Seeded benchmark inputs made on the host, the same for every caller whatever its language (no counterpart among the
 * reference's attention launchers; the stream is the splitmix64 sequence of its plan search,
 * singe/src/backend/cuda/tuning/plan.rs:527-543, read as a counter).  Word i of a stream is
 * mix(seed + (i + 1) * 0x9E3779B97F4A7C15).  Normal values: word i gives elements 2 i and 2 i + 1 by Box-Muller on
 * u1 = ((word >> 40) + 1) / 2^24 and u2 = ((word >> 16) & 0xFFFFFF) / 2^24, computed in double and rounded to float.
 * Integers: low + ((word >> 32) * span >> 32), span < 2^32.  Permutation: Fisher-Yates from the back, step k drawing
 * from [0, count - 1 - k] with word k.  A tensor's seed is base_seed ^ FNV-1a-64(name).  Host memory only. */
SINGE_HIP_API uint64_t singe_hip_synthetic_seed(uint64_t base_seed, const char* tensor_name);
SINGE_HIP_API uint64_t singe_hip_synthetic_word(uint64_t seed, uint64_t index);
SINGE_HIP_API void singe_hip_synthetic_normal_f32(uint64_t seed, uint64_t first_element, float* out, size_t count, uint32_t threads);
SINGE_HIP_API void singe_hip_synthetic_integers(uint64_t seed, uint64_t first_index, int64_t low, uint64_t span, int64_t* out,
                                                size_t count);
SINGE_HIP_API void singe_hip_synthetic_permutation(uint64_t seed, int64_t* out, size_t count);

/* ---- singe-kernel surface: the rest of the dense attention family ---------------------------------------
 * The launchers of singe-kernel/src/cuda/attention/fmha.rs:193-1036 and paged.rs:36-116, 427-576 that the entry points
 * above do not cover.  Every one checks its config and lengths in the order of the reference's `validate_lengths` and
 * then runs on a kernel of this library: the matrix-core prefill kernels where the call is one of their shapes (bf16 /
 * f16, a head dimension that is a multiple of 16 up to 128, strides in multiples of eight elements, 16-byte aligned
 * buffers), otherwise the one-wave-per-row kernel that reads every operand through element strides, in f32 arithmetic
 * whatever the storage type, head dimensions up to 256 (SINGE_HIP_UNSUPPORTED_WIDTH beyond). */

/* softcapped_window_attention_f16 / _bf16 (fmha.rs:295-393; CPU form cpu/attention.rs:1835-1925): the 16-bit forms
 * of singe_hip_softcapped_window_attention_f32.  A soft cap must be finite and positive (mod.rs:3418-3430). */
SINGE_HIP_API int32_t singe_hip_softcapped_window_attention_bf16(
    void* stream, uint16_t* out, size_t out_len, const uint16_t* query, size_t query_len, const uint16_t* key, size_t key_len,
    const uint16_t* value, size_t value_len, const SingeSoftcappedWindowAttentionConfig* config);
SINGE_HIP_API int32_t singe_hip_softcapped_window_attention_f16(
    void* stream, uint16_t* out, size_t out_len, const uint16_t* query, size_t query_len, const uint16_t* key, size_t key_len,
    const uint16_t* value, size_t value_len, const SingeSoftcappedWindowAttentionConfig* config);

/* Mirrors AttentionSinkPrefillConfig (mod.rs:299-304).  Query q sits at position start_q + q; under the causal mask
 * later keys are hidden; window w > 0 hides keys before position - (w - 1); every row's softmax also holds its head's
 * sink logit, which weighs no value (CPU form cpu/attention.rs:2073-2155). */
typedef struct SingeAttentionSinkPrefillConfig {
    SingeFmhaPrefillConfig attention;
    size_t start_q;
    size_t window;
} SingeAttentionSinkPrefillConfig;

/* attention_sink_prefill_f32 / _f16 / _bf16 (fmha.rs:193-243, 796-898).  sinks [heads] in the tensors' type. */
SINGE_HIP_API int32_t singe_hip_attention_sink_prefill_f32(
    void* stream, float* out, size_t out_len, const float* query, size_t query_len, const float* key, size_t key_len,
    const float* value, size_t value_len, const float* sinks, size_t sinks_len, const SingeAttentionSinkPrefillConfig* config);
SINGE_HIP_API int32_t singe_hip_attention_sink_prefill_bf16(
    void* stream, uint16_t* out, size_t out_len, const uint16_t* query, size_t query_len, const uint16_t* key, size_t key_len,
    const uint16_t* value, size_t value_len, const uint16_t* sinks, size_t sinks_len, const SingeAttentionSinkPrefillConfig* config);
SINGE_HIP_API int32_t singe_hip_attention_sink_prefill_f16(
    void* stream, uint16_t* out, size_t out_len, const uint16_t* query, size_t query_len, const uint16_t* key, size_t key_len,
    const uint16_t* value, size_t value_len, const uint16_t* sinks, size_t sinks_len, const SingeAttentionSinkPrefillConfig* config);

/* fmha_decode_lse_f32 / _f16 / _bf16 (fmha.rs:395-438, 900-1036): one query per batch item over key_len keys through
 * the strides of SingeFmhaDecodeConfig; lse [batch, heads] is the natural log-sum-exp of each row's scaled scores
 * (FmhaDecodeConfig::validate_lengths, mod.rs:2262-2308). */
SINGE_HIP_API int32_t singe_hip_fmha_decode_lse_f32(
    void* stream, float* out, size_t out_len, float* lse, size_t lse_len, const float* query, size_t query_len, const float* key,
    size_t key_len, const float* value, size_t value_len, const SingeFmhaDecodeConfig* config);
SINGE_HIP_API int32_t singe_hip_fmha_decode_lse_bf16(
    void* stream, uint16_t* out, size_t out_len, float* lse, size_t lse_len, const uint16_t* query, size_t query_len,
    const uint16_t* key, size_t key_len, const uint16_t* value, size_t value_len, const SingeFmhaDecodeConfig* config);
SINGE_HIP_API int32_t singe_hip_fmha_decode_lse_f16(
    void* stream, uint16_t* out, size_t out_len, float* lse, size_t lse_len, const uint16_t* query, size_t query_len,
    const uint16_t* key, size_t key_len, const uint16_t* value, size_t value_len, const SingeFmhaDecodeConfig* config);

/* Mirrors SoftcappedWindowDecodeConfig (mod.rs:307-311); soft_cap: Option<f32> as (has_soft_cap, soft_cap).  The query
 * sits at position key_len - 1; window_size w > 0 hides keys with key + w < that position
 * (CPU form cpu/attention.rs:1927-1998). */
typedef struct SingeSoftcappedWindowDecodeConfig {
    SingeFmhaDecodeConfig decode;
    size_t window_size;
    uint8_t has_soft_cap;
    float soft_cap;
} SingeSoftcappedWindowDecodeConfig;

/* softcapped_window_decode_lse_f32 / _f16 / _bf16 (fmha.rs:440-582). */
SINGE_HIP_API int32_t singe_hip_softcapped_window_decode_lse_f32(
    void* stream, float* out, size_t out_len, float* lse, size_t lse_len, const float* query, size_t query_len, const float* key,
    size_t key_len, const float* value, size_t value_len, const SingeSoftcappedWindowDecodeConfig* config);
SINGE_HIP_API int32_t singe_hip_softcapped_window_decode_lse_bf16(
    void* stream, uint16_t* out, size_t out_len, float* lse, size_t lse_len, const uint16_t* query, size_t query_len,
    const uint16_t* key, size_t key_len, const uint16_t* value, size_t value_len, const SingeSoftcappedWindowDecodeConfig* config);
SINGE_HIP_API int32_t singe_hip_softcapped_window_decode_lse_f16(
    void* stream, uint16_t* out, size_t out_len, float* lse, size_t lse_len, const uint16_t* query, size_t query_len,
    const uint16_t* key, size_t key_len, const uint16_t* value, size_t value_len, const SingeSoftcappedWindowDecodeConfig* config);

/* Mirrors RaggedKvPrefillAttentionConfig (mod.rs:110-123): query [total_query_tokens, heads, dim] and key / value
 * [total_kv_tokens, kv_heads, dim] packed by sequence; sequence b owns query tokens actual_seq_offsets[b] .. +
 * actual_seq_lens_q[b] and keys actual_seq_offsets[b] .. + actual_seq_lens_kv[b]; top-left causal inside a sequence;
 * lse [total_query_tokens, heads] natural log, -1e20 for a token that sees no key (CPU form
 * cpu/attention.rs:1343-1420).  Tokens no sequence owns are left as they are; keys past total_kv_tokens are not read. */
typedef struct SingeRaggedKvPrefillAttentionConfig {
    size_t batch;
    size_t total_query_tokens;
    size_t total_kv_tokens;
    size_t heads;
    size_t kv_heads;
    size_t head_dim;
    uint8_t causal;
    float scale;
} SingeRaggedKvPrefillAttentionConfig;

/* ragged_kv_prefill_attention_f32 / _f16 / _bf16 (paged.rs:427-576). */
SINGE_HIP_API int32_t singe_hip_ragged_kv_prefill_attention_f32(
    void* stream, float* out, size_t out_len, float* lse, size_t lse_len, const float* query, size_t query_len, const float* key,
    size_t key_len, const float* value, size_t value_len, const int32_t* actual_seq_lens_q, size_t actual_seq_lens_q_len,
    const int32_t* actual_seq_lens_kv, size_t actual_seq_lens_kv_len, const int32_t* actual_seq_offsets,
    size_t actual_seq_offsets_len, const SingeRaggedKvPrefillAttentionConfig* config);
SINGE_HIP_API int32_t singe_hip_ragged_kv_prefill_attention_bf16(
    void* stream, uint16_t* out, size_t out_len, float* lse, size_t lse_len, const uint16_t* query, size_t query_len,
    const uint16_t* key, size_t key_len, const uint16_t* value, size_t value_len, const int32_t* actual_seq_lens_q,
    size_t actual_seq_lens_q_len, const int32_t* actual_seq_lens_kv, size_t actual_seq_lens_kv_len,
    const int32_t* actual_seq_offsets, size_t actual_seq_offsets_len, const SingeRaggedKvPrefillAttentionConfig* config);
SINGE_HIP_API int32_t singe_hip_ragged_kv_prefill_attention_f16(
    void* stream, uint16_t* out, size_t out_len, float* lse, size_t lse_len, const uint16_t* query, size_t query_len,
    const uint16_t* key, size_t key_len, const uint16_t* value, size_t value_len, const int32_t* actual_seq_lens_q,
    size_t actual_seq_lens_q_len, const int32_t* actual_seq_lens_kv, size_t actual_seq_lens_kv_len,
    const int32_t* actual_seq_offsets, size_t actual_seq_offsets_len, const SingeRaggedKvPrefillAttentionConfig* config);

/* Mirrors SlidingWindowAttentionConfig (mod.rs:32-56): query q at position query_start + q, key k at key_start + k; a
 * key is kept when its position is at most the query's and position + window is beyond it; the output is multiplied
 * by output_scale; a row that sees no key is zero (CPU form cpu/attention.rs:1089-1170).  window 0 is InvalidLength
 * (mod.rs:3037-3060). */
typedef struct SingeSlidingWindowAttentionConfig {
    size_t batch;
    size_t query_len;
    size_t key_len;
    size_t heads;
    size_t kv_heads;
    size_t head_dim;
    size_t query_start;
    size_t key_start;
    size_t window;
    size_t query_batch_stride;
    size_t key_batch_stride;
    size_t value_batch_stride;
    size_t output_batch_stride;
    size_t query_sequence_stride;
    size_t key_sequence_stride;
    size_t value_sequence_stride;
    size_t output_sequence_stride;
    size_t query_head_stride;
    size_t key_head_stride;
    size_t value_head_stride;
    size_t output_head_stride;
    float scale;
    float output_scale;
} SingeSlidingWindowAttentionConfig;

/* Mirrors PackedQkvAttentionConfig (mod.rs:59-64): query, key and value are views of one buffer from these offsets on. */
typedef struct SingePackedQkvAttentionConfig {
    SingeSlidingWindowAttentionConfig attention;
    size_t query_offset;
    size_t key_offset;
    size_t value_offset;
} SingePackedQkvAttentionConfig;

/* Mirrors PagedKvAttentionConfig (mod.rs:67-74): key k of batch item b is slot k % block_size of block
 * block_table[b * block_table_batch_stride + k / block_size], at block * key_cache_block_stride + slot *
 * key_sequence_stride + kv_head * key_head_stride (the value cache alike); a block id outside the cache hides its keys
 * (cutile/kernel/attention/local.rs:9150-9330).  The batch strides of key and value are not used. */
typedef struct SingePagedKvAttentionConfig {
    SingeSlidingWindowAttentionConfig attention;
    size_t block_size;
    size_t physical_blocks;
    size_t block_table_batch_stride;
    size_t key_cache_block_stride;
    size_t value_cache_block_stride;
} SingePagedKvAttentionConfig;

/* sliding_window_attention_f32 (mod.rs:2812-2855), sliding_window_attention_packed_qkv_f32
 * (paged.rs:36-50; an offset past the buffer is LengthMismatch there and SINGE_HIP_LENGTH_TOO_SHORT naming "qkv" here)
 * and sliding_window_attention_paged_kv_f32 (paged.rs:56-116). */
SINGE_HIP_API int32_t singe_hip_sliding_window_attention_f32(
    void* stream, float* out, size_t out_len, const float* query, size_t query_len, const float* key, size_t key_len,
    const float* value, size_t value_len, const SingeSlidingWindowAttentionConfig* config);
SINGE_HIP_API int32_t singe_hip_sliding_window_attention_packed_qkv_f32(
    void* stream, float* out, size_t out_len, const float* qkv, size_t qkv_len, const SingePackedQkvAttentionConfig* config);
SINGE_HIP_API int32_t singe_hip_sliding_window_attention_paged_kv_f32(
    void* stream, float* out, size_t out_len, const float* query, size_t query_len, const float* key_cache, size_t key_cache_len,
    const float* value_cache, size_t value_cache_len, const uint32_t* block_table, size_t block_table_len,
    const SingePagedKvAttentionConfig* config);

#ifdef __cplusplus
}
#endif

#endif /* SINGE_HIP_ATTENTION_H */
