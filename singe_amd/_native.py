"""ctypes binding of libsinge_hip_attention.so.  There is no fallback: if the library or its code
object is missing the import of any op fails loudly."""
from __future__ import annotations

import ctypes
import os

from . import error

_HERE = os.path.dirname(os.path.abspath(__file__))
LIBRARY_PATH = os.path.join(_HERE, "libsinge_hip_attention.so")
CODE_OBJECT_PARTS = ("paged_decode", "fmha_prefill", "fmha_prefill_f32", "paged_attention", "splitk_reduce",
                     "attention_rows_f32", "cache_ops", "latent_attention", "latent_attention_mfma",
                     "general_attention_f32", "general_attention_bf16", "general_attention_f16", "mfma_ceiling",
                     "paged_decode_d64", "fmha_prefill_d64", "paged_attention_d64", "general_attention_f64", "hbm_stream",
                     "fmha_prefill_d32", "paged_attention_d32", "fmha_prefill_d96", "paged_attention_d96",
                     "fmha_prefill_d16", "paged_attention_d16", "fmha_prefill_d48", "paged_attention_d48",
                     "fmha_prefill_d80", "paged_attention_d80", "fmha_prefill_d112", "paged_attention_d112",
                     "paged_decode_d32", "paged_decode_d16", "paged_decode_d48", "paged_decode_d80", "paged_decode_d96",
                     "paged_decode_d112", "fmha_prefill_pair", "paged_attention_pair", "fmha_prefill_pair_d64", "paged_attention_pair_d64", "fmha_prefill_pair_d96",
                     "paged_attention_pair_d96") + tuple(
    f"{source}_pair_d{dim}" for dim in (112, 80, 48, 32, 16) for source in ("fmha_prefill", "paged_attention"))
CODE_OBJECT_PATHS = [os.path.join(_HERE, f"singe_attention_gfx950.{part}.hsaco") for part in CODE_OBJECT_PARTS]

c_size = ctypes.c_size_t
c_void = ctypes.c_void_p


class ErrorDetail(ctypes.Structure):
    _fields_ = [("status", ctypes.c_int32), ("name", ctypes.c_char_p), ("minimum", ctypes.c_uint64),
                ("actual", ctypes.c_uint64)]


class PagedKvDecodeAttentionConfigC(ctypes.Structure):
    _fields_ = [("batch", c_size), ("heads", c_size), ("kv_heads", c_size), ("head_dim", c_size),
                ("block_size", c_size), ("physical_blocks", c_size), ("block_table_batch_stride", c_size),
                ("scale", ctypes.c_float)]


class PagedKvPrefillAttentionConfigC(ctypes.Structure):
    _fields_ = [("batch", c_size), ("total_query_tokens", c_size), ("heads", c_size), ("kv_heads", c_size),
                ("head_dim", c_size), ("block_size", c_size), ("physical_blocks", c_size),
                ("block_table_batch_stride", c_size), ("causal", ctypes.c_uint8), ("scale", ctypes.c_float)]


class FmhaPrefillConfigC(ctypes.Structure):
    _fields_ = [(name, c_size) for name in (
        "batch", "query_len", "key_len", "heads", "kv_heads", "head_dim", "query_batch_stride",
        "key_batch_stride", "value_batch_stride", "output_batch_stride", "query_sequence_stride",
        "key_sequence_stride", "value_sequence_stride", "output_sequence_stride", "query_head_stride",
        "key_head_stride", "value_head_stride", "output_head_stride")] + [("scale", ctypes.c_float),
                                                                        ("causal", ctypes.c_uint8)]


class SoftcappedWindowAttentionConfigC(ctypes.Structure):
    _fields_ = [("attention", FmhaPrefillConfigC), ("window_size", c_size), ("has_soft_cap", ctypes.c_uint8),
                ("soft_cap", ctypes.c_float)]


class AttentionSinkPrefillConfigC(ctypes.Structure):
    _fields_ = [("attention", FmhaPrefillConfigC), ("start_q", c_size), ("window", c_size)]


class RaggedKvPrefillAttentionConfigC(ctypes.Structure):
    _fields_ = [("batch", c_size), ("total_query_tokens", c_size), ("total_kv_tokens", c_size), ("heads", c_size),
                ("kv_heads", c_size), ("head_dim", c_size), ("causal", ctypes.c_uint8), ("scale", ctypes.c_float)]


_SLIDING_FIELDS = ("batch", "query_len", "key_len", "heads", "kv_heads", "head_dim", "query_start", "key_start", "window",
                   "query_batch_stride", "key_batch_stride", "value_batch_stride", "output_batch_stride",
                   "query_sequence_stride", "key_sequence_stride", "value_sequence_stride", "output_sequence_stride",
                   "query_head_stride", "key_head_stride", "value_head_stride", "output_head_stride")


class SlidingWindowAttentionConfigC(ctypes.Structure):
    _fields_ = [(name, c_size) for name in _SLIDING_FIELDS] + [("scale", ctypes.c_float), ("output_scale", ctypes.c_float)]


class PackedQkvAttentionConfigC(ctypes.Structure):
    _fields_ = [("attention", SlidingWindowAttentionConfigC), ("query_offset", c_size), ("key_offset", c_size),
                ("value_offset", c_size)]


class PagedKvAttentionConfigC(ctypes.Structure):
    _fields_ = [("attention", SlidingWindowAttentionConfigC), ("block_size", c_size), ("physical_blocks", c_size),
                ("block_table_batch_stride", c_size), ("key_cache_block_stride", c_size), ("value_cache_block_stride", c_size)]


class PagedAttentionProblemC(ctypes.Structure):
    _fields_ = [("tokens", ctypes.c_int64), ("heads", ctypes.c_int64), ("kv_heads", ctypes.c_int64),
                ("head_dim", ctypes.c_int64), ("page_size", ctypes.c_int64), ("sequences", ctypes.c_int64),
                ("cache_pages", ctypes.c_int64), ("page_table", ctypes.c_int64), ("index_type", ctypes.c_int32),
                ("causal", ctypes.c_uint8), ("has_scale", ctypes.c_uint8), ("has_window", ctypes.c_uint8),
                ("has_softcap", ctypes.c_uint8), ("scale", ctypes.c_float), ("softcap", ctypes.c_float),
                ("window", ctypes.c_int64)]


class AttentionProblemC(ctypes.Structure):
    _fields_ = [("batch", ctypes.c_int64), ("heads", ctypes.c_int64), ("kv_heads", ctypes.c_int64),
                ("query_len", ctypes.c_int64), ("key_len", ctypes.c_int64), ("head_dim", ctypes.c_int64),
                ("value_dim", ctypes.c_int64), ("mask_strides", ctypes.c_int64 * 4), ("data_type", ctypes.c_int32),
                ("causal", ctypes.c_uint8), ("has_scale", ctypes.c_uint8), ("has_window", ctypes.c_uint8),
                ("has_softcap", ctypes.c_uint8), ("scale", ctypes.c_float), ("softcap", ctypes.c_float),
                ("window", ctypes.c_int64)]


class SplitKReduceConfigC(ctypes.Structure):
    _fields_ = [(name, c_size) for name in (
        "batch", "heads", "splits", "head_dim", "attn_batch_stride", "attn_head_stride", "attn_split_stride",
        "lse_batch_stride", "lse_head_stride", "output_batch_stride", "output_head_stride")]


_DECODE_FIELDS = ("batch", "key_len", "heads", "kv_heads", "head_dim", "query_batch_stride", "key_batch_stride",
                  "value_batch_stride", "output_batch_stride", "query_head_stride", "key_sequence_stride",
                  "value_sequence_stride", "output_head_stride", "key_head_stride", "value_head_stride")


class FmhaDecodeConfigC(ctypes.Structure):
    _fields_ = [(name, c_size) for name in _DECODE_FIELDS] + [("scale", ctypes.c_float)]


class FmhaDecodeSplitKConfigC(ctypes.Structure):
    _fields_ = [(name, c_size) for name in (
        "batch", "key_len", "heads", "kv_heads", "splits", "kv_len_per_split", "head_dim", "query_batch_stride",
        "key_batch_stride", "value_batch_stride", "output_batch_stride", "query_head_stride", "key_sequence_stride",
        "value_sequence_stride", "output_head_stride", "output_split_stride", "key_head_stride", "value_head_stride",
        "lse_batch_stride", "lse_head_stride")] + [("scale", ctypes.c_float)]


class SoftcappedWindowDecodeConfigC(ctypes.Structure):
    _fields_ = [("decode", FmhaDecodeConfigC), ("window_size", c_size), ("has_soft_cap", ctypes.c_uint8),
                ("soft_cap", ctypes.c_float)]


class TuneOptionsC(ctypes.Structure):
    _fields_ = [("warmup", c_size), ("repeats", c_size), ("max_candidates", c_size)]


class FmhaDecodeSplitKReduceConfigC(ctypes.Structure):
    _fields_ = [("decode", FmhaDecodeConfigC), ("max_splits", c_size), ("tuning", ctypes.c_int32),
                ("explicit_splits", c_size), ("options", TuneOptionsC)]


class PagedMlaAttentionProblemC(ctypes.Structure):
    _fields_ = [("tokens", ctypes.c_int64), ("heads", ctypes.c_int64), ("latent_dim", ctypes.c_int64),
                ("position_dim", ctypes.c_int64), ("page_size", ctypes.c_int64), ("sequences", ctypes.c_int64),
                ("cache_pages", ctypes.c_int64), ("page_table", ctypes.c_int64), ("data_type", ctypes.c_int32),
                ("index_type", ctypes.c_int32), ("causal", ctypes.c_uint8), ("has_scale", ctypes.c_uint8),
                ("scale", ctypes.c_float)]


class AttentionParametersC(ctypes.Structure):
    _fields_ = [("warps", c_size), ("key_tile", c_size), ("stages", c_size), ("split_below_blocks", c_size),
                ("has_min_blocks", ctypes.c_uint8), ("min_blocks", ctypes.c_uint32)]


class ThreadOptionsC(ctypes.Structure):
    _fields_ = [("relaxed_numerics", ctypes.c_int32), ("decode_workers", ctypes.c_uint32),
                ("paged_attention_splits", ctypes.c_uint32), ("paged_mla_attention_splits", ctypes.c_uint32),
                ("has_split_below_blocks", ctypes.c_uint8), ("split_below_blocks", ctypes.c_uint64)]


class QueryRotationC(ctypes.Structure):
    _fields_ = [("table_type", ctypes.c_int32), ("has_norm", ctypes.c_uint8), ("eps", ctypes.c_float)]


class RotaryCacheProblemC(ctypes.Structure):
    _fields_ = [("tokens", ctypes.c_int64), ("query_heads", ctypes.c_int64), ("cache_heads", ctypes.c_int64),
                ("head_dim", ctypes.c_int64), ("cache_pages", ctypes.c_int64), ("page_slots", ctypes.c_int64),
                ("data_type", ctypes.c_int32), ("table_type", ctypes.c_int32), ("index_type", ctypes.c_int32),
                ("has_query_norm", ctypes.c_uint8), ("has_key_norm", ctypes.c_uint8), ("query_eps", ctypes.c_float),
                ("key_eps", ctypes.c_float)]


class PagingIndicesProblemC(ctypes.Structure):
    _fields_ = [("sequences", ctypes.c_int64), ("tokens", ctypes.c_int64), ("page_count", ctypes.c_int64),
                ("page_size", ctypes.c_int64), ("cache_pages", ctypes.c_int64), ("width", ctypes.c_int64),
                ("row_elements", ctypes.c_int64), ("index_type", ctypes.c_int32)]


DATA_TYPE_F32, DATA_TYPE_BF16, DATA_TYPE_F16, DATA_TYPE_F64 = 0, 1, 2, 3

_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        _lib = bind(LIBRARY_PATH)
    return _lib


def bind(path: str) -> ctypes.CDLL:
    """Opens the C-ABI library at `path` and declares every entry point's argument and result types.  `lib()` is this
    for the library next to the package; a copy elsewhere (one that finds no code object beside itself and is handed
    the kernels as bytes, say) binds the same way."""
    if not os.path.exists(path):
        raise error.KernelNotPrepared(
            f"{path} is missing: build it with `python -m singe_amd.build` (there is no fallback path)")
    handle = ctypes.CDLL(path)
    i32 = ctypes.c_int32
    handle.singe_hip_last_error.argtypes = [ctypes.POINTER(ErrorDetail)]
    handle.singe_hip_last_error.restype = None
    handle.singe_hip_status_string.argtypes = [i32]
    handle.singe_hip_status_string.restype = ctypes.c_char_p
    handle.singe_hip_load.argtypes = [c_void, c_size]
    handle.singe_hip_load.restype = i32
    handle.singe_hip_set_thread_options.argtypes = [ctypes.POINTER(ThreadOptionsC)]
    handle.singe_hip_set_thread_options.restype = i32
    handle.singe_hip_thread_options.argtypes = [ctypes.POINTER(ThreadOptionsC)]
    handle.singe_hip_thread_options.restype = None
    handle.singe_hip_load_part.argtypes = [ctypes.c_char_p, c_void, c_size]
    handle.singe_hip_load_part.restype = i32
    handle.singe_hip_load_file.argtypes = [ctypes.c_char_p]
    handle.singe_hip_load_file.restype = i32
    handle.singe_hip_unload.argtypes = []
    handle.singe_hip_unload.restype = None
    handle.singe_hip_kernel.argtypes = [i32, ctypes.POINTER(ctypes.c_char_p), ctypes.POINTER(ctypes.c_char_p)]
    handle.singe_hip_kernel.restype = i32
    parameters = ctypes.POINTER(AttentionParametersC)
    handle.singe_hip_attention_parameters_default.argtypes = [parameters]
    handle.singe_hip_attention_parameters_default.restype = None
    handle.singe_hip_attention_parameters.argtypes = [parameters]
    handle.singe_hip_attention_parameters.restype = None
    handle.singe_hip_attention_candidates.argtypes = [parameters, c_size, ctypes.POINTER(c_size)]
    handle.singe_hip_attention_candidates.restype = i32
    handle.singe_hip_set_attention_parameters.argtypes = [parameters]
    handle.singe_hip_set_attention_parameters.restype = i32
    handle.singe_hip_paged_attention_parameter_key.argtypes = [ctypes.POINTER(PagedAttentionProblemC), i32, ctypes.c_char_p, c_size]
    handle.singe_hip_paged_attention_parameter_key.restype = c_size
    handle.singe_hip_attention_parameter_key.argtypes = [ctypes.POINTER(AttentionProblemC), i32, i32, i32, ctypes.c_char_p, c_size]
    handle.singe_hip_attention_parameter_key.restype = c_size
    handle.singe_hip_scaled_dot_product_attention_scratch_bytes.argtypes = [ctypes.POINTER(AttentionProblemC)]
    handle.singe_hip_scaled_dot_product_attention_scratch_bytes.restype = c_size
    handle.singe_hip_scaled_dot_product_attention_scratch.argtypes = [c_void] * 8 + [c_void, c_size, ctypes.POINTER(AttentionProblemC)]
    handle.singe_hip_scaled_dot_product_attention_scratch.restype = i32
    handle.singe_hip_hbm_stream_read.argtypes = [c_void, c_void, c_size, c_void, c_size, ctypes.c_uint32]
    handle.singe_hip_hbm_stream_read.restype = i32
    handle.singe_hip_mfma_ceiling.argtypes = [c_void, c_void, c_size, c_void, c_size, ctypes.c_uint32, ctypes.c_uint32, i32]
    handle.singe_hip_mfma_ceiling.restype = i32
    u64 = ctypes.c_uint64
    handle.singe_hip_synthetic_seed.argtypes = [u64, ctypes.c_char_p]
    handle.singe_hip_synthetic_seed.restype = u64
    handle.singe_hip_synthetic_word.argtypes = [u64, u64]
    handle.singe_hip_synthetic_word.restype = u64
    handle.singe_hip_synthetic_normal_f32.argtypes = [u64, u64, c_void, c_size, ctypes.c_uint32]
    handle.singe_hip_synthetic_normal_f32.restype = None
    handle.singe_hip_synthetic_integers.argtypes = [u64, u64, ctypes.c_int64, u64, c_void, c_size]
    handle.singe_hip_synthetic_integers.restype = None
    handle.singe_hip_synthetic_permutation.argtypes = [u64, c_void, c_size]
    handle.singe_hip_synthetic_permutation.restype = None
    handle.singe_hip_prepare.argtypes = [ctypes.POINTER(i32)]
    handle.singe_hip_prepare.restype = i32
    cfg = ctypes.POINTER(PagedKvDecodeAttentionConfigC)
    handle.singe_hip_paged_kv_decode_attention_config_validate.argtypes = [cfg]
    handle.singe_hip_paged_kv_decode_attention_config_validate.restype = i32
    handle.singe_hip_paged_kv_decode_attention_workspace_bytes.argtypes = [cfg]
    handle.singe_hip_paged_kv_decode_attention_workspace_bytes.restype = c_size
    handle.singe_hip_paged_kv_decode_attention_bf16.argtypes = [
        c_void, c_void, c_size, c_void, c_size, c_void, c_size, c_void, c_size, c_void, c_size, c_void, c_size,
        c_void, c_size, cfg]
    handle.singe_hip_paged_kv_decode_attention_bf16.restype = i32
    handle.singe_hip_paged_kv_decode_attention_no_alloc_bf16.argtypes = [
        c_void, c_void, c_size, c_void, c_size, c_void, c_size, c_void, c_size, c_void, c_size, c_void, c_size, cfg]
    handle.singe_hip_paged_kv_decode_attention_no_alloc_bf16.restype = i32
    handle.singe_hip_paged_kv_decode_attention_f16.argtypes = handle.singe_hip_paged_kv_decode_attention_bf16.argtypes
    handle.singe_hip_paged_kv_decode_attention_f16.restype = i32
    handle.singe_hip_paged_kv_decode_attention_phases_bf16.argtypes = [
        c_void, c_void, c_size, c_void, c_size, c_void, c_size, c_void, c_size, c_void, c_size, c_void, c_size,
        c_void, c_size, cfg, ctypes.c_uint32]
    handle.singe_hip_paged_kv_decode_attention_phases_bf16.restype = i32
    handle.singe_hip_paged_kv_decode_attention_f8e4m3kv_bf16.argtypes = [
        c_void, c_void, c_size, c_void, c_size, c_void, c_size, c_void, c_size, c_void, c_size, c_void, c_size,
        c_void, c_size, c_void, c_size, c_void, c_size, cfg, ctypes.c_uint32]
    handle.singe_hip_paged_kv_decode_attention_f8e4m3kv_bf16.restype = i32
    handle.singe_hip_set_relaxed_numerics.argtypes = [i32]
    handle.singe_hip_set_relaxed_numerics.restype = None
    handle.singe_hip_relaxed_numerics.argtypes = []
    handle.singe_hip_relaxed_numerics.restype = i32
    handle.singe_hip_set_paged_attention_rows_per_wave.argtypes = [ctypes.c_uint32]
    handle.singe_hip_set_paged_attention_rows_per_wave.restype = None
    handle.singe_hip_paged_attention_rows_per_wave.argtypes = [ctypes.c_void_p]
    handle.singe_hip_paged_attention_rows_per_wave.restype = ctypes.c_uint32
    handle.singe_hip_set_dense_prefill_rows_per_wave.argtypes = [ctypes.c_uint32]
    handle.singe_hip_set_dense_prefill_rows_per_wave.restype = None
    handle.singe_hip_dense_prefill_rows_per_wave.argtypes = [ctypes.c_void_p]
    handle.singe_hip_dense_prefill_rows_per_wave.restype = ctypes.c_uint32
    handle.singe_hip_set_decode_workers.argtypes = [ctypes.c_uint32]
    handle.singe_hip_set_decode_workers.restype = None
    handle.singe_hip_decode_workers.argtypes = [cfg]
    handle.singe_hip_decode_workers.restype = ctypes.c_uint32
    paged_prefill = ctypes.POINTER(PagedKvPrefillAttentionConfigC)
    handle.singe_hip_paged_kv_prefill_attention_config_validate.argtypes = [paged_prefill]
    handle.singe_hip_paged_kv_prefill_attention_config_validate.restype = i32
    handle.singe_hip_paged_kv_prefill_attention_bf16.argtypes = [c_void] + [c_void, c_size] * 9 + [paged_prefill]
    handle.singe_hip_paged_kv_prefill_attention_bf16.restype = i32
    handle.singe_hip_paged_kv_prefill_attention_f16.argtypes = [c_void] + [c_void, c_size] * 9 + [paged_prefill]
    handle.singe_hip_paged_kv_prefill_attention_f16.restype = i32
    fmha = ctypes.POINTER(FmhaPrefillConfigC)
    handle.singe_hip_fmha_prefill_config_validate.argtypes = [fmha]
    handle.singe_hip_fmha_prefill_config_validate.restype = i32
    handle.singe_hip_fmha_prefill_bf16.argtypes = [c_void, c_void, c_size, c_void, c_size, c_void, c_size, c_void,
                                                   c_size, fmha]
    handle.singe_hip_fmha_prefill_bf16.restype = i32
    handle.singe_hip_fmha_prefill_lse_bf16.argtypes = [c_void, c_void, c_size, c_void, c_size, c_void, c_size, c_void,
                                                       c_size, c_void, c_size, fmha]
    handle.singe_hip_fmha_prefill_lse_bf16.restype = i32
    handle.singe_hip_fmha_prefill_f16.argtypes = handle.singe_hip_fmha_prefill_bf16.argtypes
    handle.singe_hip_fmha_prefill_f16.restype = i32
    handle.singe_hip_fmha_prefill_lse_f16.argtypes = handle.singe_hip_fmha_prefill_lse_bf16.argtypes
    handle.singe_hip_fmha_prefill_lse_f16.restype = i32
    handle.singe_hip_paged_attention_scratch_f16.argtypes = [c_void] * 12 + [ctypes.c_size_t, ctypes.POINTER(PagedAttentionProblemC)]
    handle.singe_hip_paged_attention_scratch_f16.restype = i32
    handle.singe_hip_fmha_prefill_f32.argtypes = [c_void, c_void, c_size, c_void, c_size, c_void, c_size, c_void,
                                                  c_size, fmha]
    handle.singe_hip_fmha_prefill_f32.restype = i32
    handle.singe_hip_fmha_prefill_lse_f32.argtypes = [c_void, c_void, c_size, c_void, c_size, c_void, c_size, c_void,
                                                      c_size, c_void, c_size, fmha]
    handle.singe_hip_fmha_prefill_lse_f32.restype = i32
    handle.singe_hip_softcapped_window_attention_f32.argtypes = [
        c_void, c_void, c_size, c_void, c_size, c_void, c_size, c_void, c_size,
        ctypes.POINTER(SoftcappedWindowAttentionConfigC)]
    handle.singe_hip_softcapped_window_attention_f32.restype = i32
    handle.singe_hip_paged_attention_bf16.argtypes = [c_void] * 11 + [ctypes.POINTER(PagedAttentionProblemC)]
    handle.singe_hip_paged_attention_bf16.restype = i32
    handle.singe_hip_rotary_paged_attention_bf16.argtypes = [c_void] * 14 + [ctypes.POINTER(PagedAttentionProblemC),
                                                                             ctypes.POINTER(QueryRotationC)]
    handle.singe_hip_rotary_paged_attention_bf16.restype = i32
    handle.singe_hip_rotary_paged_attention_f16.argtypes = handle.singe_hip_rotary_paged_attention_bf16.argtypes
    handle.singe_hip_rotary_paged_attention_f16.restype = i32
    handle.singe_hip_paged_attention_scratch_bf16.argtypes = [c_void] * 12 + [ctypes.c_size_t, ctypes.POINTER(PagedAttentionProblemC)]
    handle.singe_hip_paged_attention_scratch_bf16.restype = i32
    handle.singe_hip_paged_attention_scratch_bytes.argtypes = [ctypes.POINTER(PagedAttentionProblemC)]
    handle.singe_hip_paged_attention_scratch_bytes.restype = ctypes.c_size_t
    handle.singe_hip_set_paged_attention_splits.argtypes = [ctypes.c_uint32]
    handle.singe_hip_set_paged_attention_splits.restype = None
    handle.singe_hip_paged_mla_attention.argtypes = [c_void] * 12 + [ctypes.POINTER(PagedMlaAttentionProblemC)]
    handle.singe_hip_paged_mla_attention.restype = i32
    handle.singe_hip_paged_mla_attention_scratch.argtypes = [c_void] * 13 + [c_size, ctypes.POINTER(PagedMlaAttentionProblemC)]
    handle.singe_hip_paged_mla_attention_scratch.restype = i32
    handle.singe_hip_paged_mla_attention_scratch_bytes.argtypes = [ctypes.POINTER(PagedMlaAttentionProblemC)]
    handle.singe_hip_paged_mla_attention_scratch_bytes.restype = ctypes.c_size_t
    handle.singe_hip_set_paged_mla_attention_splits.argtypes = [ctypes.c_uint32]
    handle.singe_hip_set_paged_mla_attention_splits.restype = None
    handle.singe_hip_paged_attention_f32.argtypes = [c_void] * 11 + [ctypes.POINTER(PagedAttentionProblemC)]
    handle.singe_hip_paged_attention_f32.restype = i32
    handle.singe_hip_paged_attention_f64.argtypes = [c_void] * 11 + [ctypes.POINTER(PagedAttentionProblemC)]
    handle.singe_hip_paged_attention_f64.restype = i32
    handle.singe_hip_paged_attention_f16.argtypes = [c_void] * 11 + [ctypes.POINTER(PagedAttentionProblemC)]
    handle.singe_hip_paged_attention_f16.restype = i32
    handle.singe_hip_scaled_dot_product_attention.argtypes = [c_void] * 8 + [ctypes.POINTER(AttentionProblemC)]
    handle.singe_hip_scaled_dot_product_attention.restype = i32
    handle.singe_hip_splitk_reduce_f32.argtypes = [c_void, c_void, c_size, c_void, c_size, c_void, c_size,
                                                   ctypes.POINTER(SplitKReduceConfigC)]
    handle.singe_hip_splitk_reduce_f32.restype = i32
    handle.singe_hip_paged_kv_decode_attention_f32_workspace_bytes.argtypes = [cfg]
    handle.singe_hip_paged_kv_decode_attention_f32_workspace_bytes.restype = ctypes.c_size_t
    handle.singe_hip_paged_kv_decode_attention_f32.argtypes = [c_void] + [c_void, c_size] * 7 + [cfg]
    handle.singe_hip_paged_kv_decode_attention_f32.restype = i32
    handle.singe_hip_paged_kv_prefill_attention_f32.argtypes = [c_void] + [c_void, c_size] * 9 + [paged_prefill]
    handle.singe_hip_paged_kv_prefill_attention_f32.restype = i32
    split = ctypes.POINTER(FmhaDecodeSplitKConfigC)
    split_reduce = ctypes.POINTER(FmhaDecodeSplitKReduceConfigC)
    handle.singe_hip_fmha_decode_splitk_f32.argtypes = [c_void] + [c_void, c_size] * 5 + [split]
    handle.singe_hip_fmha_decode_splitk_f32.restype = i32
    handle.singe_hip_fmha_decode_splitk_reduce_f32.argtypes = [c_void] + [c_void, c_size] * 6 + [split_reduce]
    handle.singe_hip_fmha_decode_splitk_reduce_f32.restype = i32
    handle.singe_hip_attention_splitk_candidates.argtypes = [split_reduce, ctypes.POINTER(c_size), c_size,
                                                             ctypes.POINTER(c_size)]
    handle.singe_hip_attention_splitk_candidates.restype = i32
    handle.singe_hip_fmha_decode_splitk_reduce_tuned_splits.argtypes = [split_reduce, ctypes.POINTER(c_size)]
    handle.singe_hip_fmha_decode_splitk_reduce_tuned_splits.restype = i32
    handle.singe_hip_clear_tune_cache.argtypes = []
    handle.singe_hip_clear_tune_cache.restype = None
    pairs4, pairs5 = [c_void, c_size] * 4, [c_void, c_size] * 5
    for element in ("bf16", "f16"):
        entry = getattr(handle, f"singe_hip_softcapped_window_attention_{element}")
        entry.argtypes, entry.restype = [c_void] + pairs4 + [ctypes.POINTER(SoftcappedWindowAttentionConfigC)], i32
    for element in ("f32", "bf16", "f16"):
        entry = getattr(handle, f"singe_hip_attention_sink_prefill_{element}")
        entry.argtypes, entry.restype = [c_void] + pairs5 + [ctypes.POINTER(AttentionSinkPrefillConfigC)], i32
        entry = getattr(handle, f"singe_hip_fmha_decode_lse_{element}")
        entry.argtypes, entry.restype = [c_void] + pairs5 + [ctypes.POINTER(FmhaDecodeConfigC)], i32
        entry = getattr(handle, f"singe_hip_softcapped_window_decode_lse_{element}")
        entry.argtypes, entry.restype = [c_void] + pairs5 + [ctypes.POINTER(SoftcappedWindowDecodeConfigC)], i32
        entry = getattr(handle, f"singe_hip_ragged_kv_prefill_attention_{element}")
        entry.argtypes, entry.restype = [c_void] + [c_void, c_size] * 8 + [ctypes.POINTER(RaggedKvPrefillAttentionConfigC)], i32
    handle.singe_hip_sliding_window_attention_f32.argtypes = [c_void] + pairs4 + [ctypes.POINTER(SlidingWindowAttentionConfigC)]
    handle.singe_hip_sliding_window_attention_f32.restype = i32
    handle.singe_hip_sliding_window_attention_packed_qkv_f32.argtypes = [c_void] + [c_void, c_size] * 2 + [ctypes.POINTER(PackedQkvAttentionConfigC)]
    handle.singe_hip_sliding_window_attention_packed_qkv_f32.restype = i32
    handle.singe_hip_sliding_window_attention_paged_kv_f32.argtypes = [c_void] + pairs5 + [ctypes.POINTER(PagedKvAttentionConfigC)]
    handle.singe_hip_sliding_window_attention_paged_kv_f32.restype = i32
    handle.singe_hip_rotary_cache_write.argtypes = [c_void] * 14 + [ctypes.POINTER(RotaryCacheProblemC)]
    handle.singe_hip_rotary_cache_write.restype = i32
    handle.singe_hip_paging_indices.argtypes = [c_void] * 10 + [ctypes.POINTER(PagingIndicesProblemC)]
    handle.singe_hip_paging_indices.restype = i32
    return handle


def check(status: int, op: str = "") -> None:
    """Turns a C status into the matching exception (the `try_ffi!` of this layer)."""
    if status == 0:
        return
    detail = ErrorDetail()
    lib().singe_hip_last_error(ctypes.byref(detail))
    name = (detail.name or b"").decode()
    if status < 0:
        message = (lib().singe_hip_status_string(status) or b"").decode()
        raise error.Hip(-status, message, name or op)
    table = {
        1: lambda: error.InvalidLength("invalid length"),
        2: lambda: error.LengthTooShort(name, int(detail.minimum), int(detail.actual)),
        3: lambda: error.LengthExceedsI32("length exceeds i32"),
        4: lambda: error.SizeOverflow("size overflow"),
        5: lambda: error.UnsupportedWidth(name or op, int(detail.minimum)),
        6: lambda: error.NullPointer(f"null pointer: {name}"),
        7: lambda: error.KernelNotPrepared(f"kernel specialization has not been prepared: {name}"),
        8: lambda: error.UnsupportedConfiguration(f"unsupported configuration for {op}: {name}"),
        9: lambda: error.InvalidArgument(f"{op} {name}"),
        10: lambda: error.KernelNotPrepared("the HIP runtime library could not be opened"),
        11: lambda: error.TuneCacheMiss(f"tune cache miss for {name or op}"),
        12: lambda: error.AutotuneDuringCapture(f"autotune during stream capture for {name or op}"),
        13: lambda: error.NoTuneCandidates(f"no tune candidates for {name or op}"),
        14: lambda: error.NoTuneCandidates(f"no tune candidate completed for {name or op}"),
        15: lambda: error.StaleRecord(f"stale record: {name or op}"),
    }
    raise table.get(status, lambda: error.Error(f"status {status}"))()
