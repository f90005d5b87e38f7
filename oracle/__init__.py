"""CPU oracle for the attention hot path: test infrastructure only.

numpy-facing wrappers over ``libsinge_oracle.so`` (built from ``singe_oracle.c``
by ``make -C oracle``).  Each wrapper names the reference function it restates.
Only the tests, the smoke check and the benchmark's CPU-baseline leg import
this package; the shipped library never does.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libsinge_oracle.so")

_c_size = ctypes.c_size_t
_c_float = ctypes.c_float
_c_int = ctypes.c_int
_c_i64 = ctypes.c_int64


def build(force: bool = False) -> str:
    """Compiles the oracle with gcc and returns the library path."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.run(["make", "-C", _HERE, "-B" if force else "-s", "all"], check=True)
    return _LIB_PATH


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.oracle_bf16_to_f32.restype = _c_float
        _lib.oracle_bf16_to_f32.argtypes = [ctypes.c_uint16]
        _lib.oracle_f32_to_bf16.restype = ctypes.c_uint16
        _lib.oracle_f32_to_bf16.argtypes = [_c_float]
        _lib.oracle_f8e4m3_value.restype = _c_float
        _lib.oracle_f8e4m3_value.argtypes = [ctypes.c_uint8]
        _lib.oracle_f8e4m3_encode.restype = ctypes.c_uint8
        _lib.oracle_f8e4m3_encode.argtypes = [ctypes.c_double]
        _lib.oracle_check_paged_values.restype = _c_int
        _lib.oracle_paged_attention_f32.restype = _c_int
        _lib.oracle_paged_mla_attention.restype = _c_int
        _lib.oracle_paged_slots.restype = _c_size
        _lib.oracle_max_threads.restype = _c_int
    return _lib


def _f32(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.float32)


def _ptr(a: np.ndarray | None):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def max_threads() -> int:
    return int(lib().oracle_max_threads())


# ---- codecs -------------------------------------------------------------------

def bf16_to_f32(bits) -> np.ndarray:
    """prelude.rs:91-93 load_bfloat."""
    bits = np.asarray(bits, dtype=np.uint16)
    return (bits.astype(np.uint32) << 16).view(np.float32)


def f32_to_bf16(values) -> np.ndarray:
    """prelude.rs:94-106 store_bfloat (round to nearest even), vectorised; the scalar C form is
    oracle_f32_to_bf16 and a test shows the two agree on every exponent/rounding case."""
    bits = _f32(values).view(np.uint32)
    nan = (bits & 0x7FFFFFFF) > 0x7F800000
    rounded = ((bits.astype(np.uint64) + 0x7FFF + ((bits >> 16) & 1)) >> 16).astype(np.uint16)
    return np.where(nan, ((bits >> 16) | 0x0040).astype(np.uint16), rounded)


def round_bf16(values) -> np.ndarray:
    """f32 values rounded to bf16 and widened back."""
    return bf16_to_f32(f32_to_bf16(values))


def f8e4m3_value(code: int) -> float:
    """singe-kernel/src/cpu/quantization.rs:265-280."""
    return float(lib().oracle_f8e4m3_value(int(code) & 0xFF))


def f8e4m3_encode(value: float) -> int:
    """singe-codegen/src/interpret/minifloat.rs:97-151 (finite e4m3)."""
    return int(lib().oracle_f8e4m3_encode(float(value)))


def f8e4m3_table() -> np.ndarray:
    return np.array([f8e4m3_value(c) for c in range(256)], dtype=np.float32)


def f8e4m3_encode_array(values) -> np.ndarray:
    flat = np.asarray(values, dtype=np.float64).ravel()
    out = np.empty(flat.shape, dtype=np.uint8)
    encode = lib().oracle_f8e4m3_encode
    for i, v in enumerate(flat):
        out[i] = encode(float(v))
    return out.reshape(np.shape(values))


def dequantize_f8e4m3_cache(codes, scales) -> np.ndarray:
    """codes [blocks, block_size, kv_heads, dim] u8, scales [blocks, kv_heads] f32
    -> bf16_rne(value * scale) widened to f32."""
    codes = np.ascontiguousarray(codes, dtype=np.uint8)
    scales = _f32(scales)
    blocks, block_size, kv_heads, dim = codes.shape
    out = np.empty(codes.shape, dtype=np.float32)
    lib().oracle_dequantize_f8e4m3_cache(_ptr(out), _ptr(codes), _ptr(scales), _c_size(blocks),
                                         _c_size(block_size), _c_size(kv_heads), _c_size(dim))
    return out


# ---- singe-kernel surface -----------------------------------------------------

def paged_kv_decode_attention_f32(query, key_cache, value_cache, actual_seq_lens, block_table, *,
                                  batch, heads, kv_heads, head_dim, block_size,
                                  block_table_batch_stride, scale, threads=1, literal=False):
    """singe-kernel/src/cpu/attention.rs:1172-1246."""
    query, key_cache, value_cache = _f32(query), _f32(key_cache), _f32(value_cache)
    lens = np.ascontiguousarray(actual_seq_lens, dtype=np.int32)
    table = np.ascontiguousarray(block_table, dtype=np.uint32)
    out = np.empty(batch * heads * head_dim, dtype=np.float32)
    args = [_ptr(out), _ptr(query), _ptr(key_cache), _ptr(value_cache), _ptr(lens), _ptr(table),
            _c_size(batch), _c_size(heads), _c_size(kv_heads), _c_size(head_dim), _c_size(block_size),
            _c_size(block_table_batch_stride), _c_float(scale)]
    if literal:
        lib().oracle_paged_kv_decode_attention_f32_literal(*args)
    else:
        lib().oracle_paged_kv_decode_attention_f32(*args, _c_int(threads))
    return out.reshape(batch, heads, head_dim)


def paged_gather_offsets(actual_seq_lens, block_table, *, kv_heads, head_dim, block_size,
                         block_table_batch_stride, kv_head=0):
    """Element offset of every key's row in the cache (cpu/attention.rs:1196-1206)."""
    lens = np.ascontiguousarray(actual_seq_lens, dtype=np.int32)
    table = np.ascontiguousarray(block_table, dtype=np.uint32)
    out = np.empty(int(lens.astype(np.int64).sum()), dtype=np.uint64)
    lib().oracle_paged_gather_offsets(_ptr(out), _ptr(lens), _ptr(table), _c_size(len(lens)),
                                      _c_size(kv_heads), _c_size(head_dim), _c_size(block_size),
                                      _c_size(block_table_batch_stride), _c_size(kv_head))
    return out


def paged_kv_prefill_attention_f32(query, key_cache, value_cache, actual_seq_lens_q,
                                   actual_seq_lens_kv, actual_seq_offsets, block_table, *, batch,
                                   total_query_tokens, heads, kv_heads, head_dim, block_size,
                                   block_table_batch_stride, causal, scale, threads=1):
    """singe-kernel/src/cpu/attention.rs:1248-1341 -> (out [T,H,D], lse [T,H])."""
    query, key_cache, value_cache = _f32(query), _f32(key_cache), _f32(value_cache)
    lq = np.ascontiguousarray(actual_seq_lens_q, dtype=np.int32)
    lk = np.ascontiguousarray(actual_seq_lens_kv, dtype=np.int32)
    off = np.ascontiguousarray(actual_seq_offsets, dtype=np.int32)
    table = np.ascontiguousarray(block_table, dtype=np.uint32)
    out = np.empty(total_query_tokens * heads * head_dim, dtype=np.float32)
    lse = np.empty(total_query_tokens * heads, dtype=np.float32)
    lib().oracle_paged_kv_prefill_attention_f32(
        _ptr(out), _ptr(lse), _ptr(query), _ptr(key_cache), _ptr(value_cache), _ptr(lq), _ptr(lk),
        _ptr(off), _ptr(table), _c_size(batch), _c_size(total_query_tokens), _c_size(heads),
        _c_size(kv_heads), _c_size(head_dim), _c_size(block_size), _c_size(block_table_batch_stride),
        _c_int(bool(causal)), _c_float(scale), _c_int(threads))
    return out.reshape(total_query_tokens, heads, head_dim), lse.reshape(total_query_tokens, heads)


def fmha_prefill_lse_f32(query, key, value, *, batch, query_len, key_len, heads, kv_heads, head_dim,
                         scale, causal, threads=1):
    """singe-kernel/src/cpu/attention.rs:1758-1833 (BSHD) -> (out, lse [B,H,L])."""
    query, key, value = _f32(query), _f32(key), _f32(value)
    out = np.empty(batch * query_len * heads * head_dim, dtype=np.float32)
    lse = np.empty(batch * heads * query_len, dtype=np.float32)
    lib().oracle_fmha_prefill_lse_f32(_ptr(out), _ptr(lse), _ptr(query), _ptr(key), _ptr(value),
                                      _c_size(batch), _c_size(query_len), _c_size(key_len),
                                      _c_size(heads), _c_size(kv_heads), _c_size(head_dim),
                                      _c_float(scale), _c_int(bool(causal)), _c_int(threads))
    return out.reshape(batch, query_len, heads, head_dim), lse.reshape(batch, heads, query_len)


def fmha_prefill_lse_f32_literal(query, key, value, *, batch, query_len, key_len, heads, kv_heads, head_dim,
                                 scale, causal, row_first=0, row_count=None):
    """fmha_prefill_lse_f32 with the reference's loop shape kept literally (cpu/attention.rs:1776-1830), on query rows
    [row_first, row_first + row_count) of every (batch, head); the other rows stay zero."""
    query, key, value = _f32(query), _f32(key), _f32(value)
    out = np.empty(batch * query_len * heads * head_dim, dtype=np.float32)
    lse = np.empty(batch * heads * query_len, dtype=np.float32)
    count = query_len - row_first if row_count is None else row_count
    lib().oracle_fmha_prefill_lse_f32_literal(_ptr(out), _ptr(lse), _ptr(query), _ptr(key), _ptr(value),
                                              _c_size(batch), _c_size(query_len), _c_size(key_len),
                                              _c_size(heads), _c_size(kv_heads), _c_size(head_dim),
                                              _c_float(scale), _c_int(bool(causal)), _c_size(row_first), _c_size(count))
    return out.reshape(batch, query_len, heads, head_dim), lse.reshape(batch, heads, query_len)


def softcapped_window_attention_f32(query, key, value, *, batch, query_len, key_len, heads, kv_heads,
                                    head_dim, scale, causal, window_size=0, soft_cap=None, threads=1):
    """singe-kernel/src/cpu/attention.rs:1835-1925 (BHSD)."""
    query, key, value = _f32(query), _f32(key), _f32(value)
    out = np.empty(batch * heads * query_len * head_dim, dtype=np.float32)
    lib().oracle_softcapped_window_attention_f32(
        _ptr(out), _ptr(query), _ptr(key), _ptr(value), _c_size(batch), _c_size(query_len),
        _c_size(key_len), _c_size(heads), _c_size(kv_heads), _c_size(head_dim), _c_float(scale),
        _c_int(bool(causal)), _c_size(window_size), _c_int(soft_cap is not None),
        _c_float(soft_cap if soft_cap is not None else 0.0), _c_int(threads))
    return out.reshape(batch, heads, query_len, head_dim)


def sliding_window_attention_f32(query, key, value, *, batch, query_len, key_len, heads, kv_heads,
                                 head_dim, query_start, key_start, window, scale, output_scale):
    """singe-kernel/src/cpu/attention.rs:1089-1170 (BSHD, causal left window)."""
    query, key, value = _f32(query), _f32(key), _f32(value)
    out = np.empty(batch * query_len * heads * head_dim, dtype=np.float32)
    lib().oracle_sliding_window_attention_f32(
        _ptr(out), _ptr(query), _ptr(key), _ptr(value), _c_size(batch), _c_size(query_len),
        _c_size(key_len), _c_size(heads), _c_size(kv_heads), _c_size(head_dim), _c_size(query_start),
        _c_size(key_start), _c_size(window), _c_float(scale), _c_float(output_scale))
    return out


def ragged_kv_prefill_attention_f32(query, key, value, lens_q, lens_kv, offsets, *, causal, scale):
    """singe-kernel/src/cpu/attention.rs:1343-1420: query [T, H, D], key / value [S, G, D] packed by sequence ->
    (out [T, H, D], lse [T, H] natural log, -1e20 where a token sees no key)."""
    query, key, value = _f32(query), _f32(key), _f32(value)
    tokens, heads, head_dim = query.shape
    kv_heads = key.shape[1]
    lens_q, lens_kv, offsets = (np.ascontiguousarray(a, dtype=np.int32) for a in (lens_q, lens_kv, offsets))
    out = np.empty(query.shape, dtype=np.float32)
    lse = np.empty((tokens, heads), dtype=np.float32)
    i32 = ctypes.POINTER(ctypes.c_int32)
    lib().oracle_ragged_kv_prefill_attention_f32(
        _ptr(out), _ptr(lse), _ptr(query), _ptr(key), _ptr(value), lens_q.ctypes.data_as(i32), lens_kv.ctypes.data_as(i32),
        offsets.ctypes.data_as(i32), _c_size(len(lens_q)), _c_size(tokens), _c_size(heads), _c_size(kv_heads), _c_size(head_dim),
        _c_int(bool(causal)), _c_float(scale))
    return out, lse


def softcapped_window_decode_lse_f32(query, key, value, *, scale, window_size=0, soft_cap=None):
    """singe-kernel/src/cpu/attention.rs:1927-1998: query [B, H, D], key / value [B, G, S, D] -> (out [B, H, D], lse [B, H])."""
    query, key, value = _f32(query), _f32(key), _f32(value)
    batch, heads, head_dim = query.shape
    kv_heads, key_len = key.shape[1], key.shape[2]
    out = np.empty(query.shape, dtype=np.float32)
    lse = np.empty((batch, heads), dtype=np.float32)
    lib().oracle_softcapped_window_decode_lse_f32(
        _ptr(out), _ptr(lse), _ptr(query), _ptr(key), _ptr(value), _c_size(batch), _c_size(key_len), _c_size(heads), _c_size(kv_heads),
        _c_size(head_dim), _c_float(scale), _c_size(window_size), _c_int(soft_cap is not None),
        _c_float(soft_cap if soft_cap is not None else 0.0))
    return out, lse


def attention_sink_prefill_f32(query, key, value, sinks, *, start_q=0, window=0, scale, causal):
    """singe-kernel/src/cpu/attention.rs:2073-2155: query [B, L, H, D], key / value [B, S, G, D], sinks [H] -> out [B, L, H, D]."""
    query, key, value, sinks = _f32(query), _f32(key), _f32(value), _f32(sinks)
    batch, query_len, heads, head_dim = query.shape
    key_len, kv_heads = key.shape[1], key.shape[2]
    out = np.empty(query.shape, dtype=np.float32)
    lib().oracle_attention_sink_prefill_f32(
        _ptr(out), _ptr(query), _ptr(key), _ptr(value), _ptr(sinks), _c_size(batch), _c_size(query_len), _c_size(key_len), _c_size(heads),
        _c_size(kv_heads), _c_size(head_dim), _c_size(start_q), _c_size(window), _c_float(scale), _c_int(bool(causal)))
    return out


def sliding_window_attention_paged_kv_f32(query, key_cache, value_cache, block_table, *, key_len, query_start, key_start, window,
                                          scale, output_scale=1.0):
    """The reference's sliding_window_attention_paged_kv_f32 kernel (cutile/kernel/attention/local.rs:9150-9330):
    query [B, L, H, D], caches [P, block, G, D], block_table [B, stride] u32 -> out [B, L, H, D]."""
    query, key_cache, value_cache = _f32(query), _f32(key_cache), _f32(value_cache)
    batch, query_len, heads, head_dim = query.shape
    physical_blocks, block_size, kv_heads, _ = key_cache.shape
    table = np.ascontiguousarray(block_table, dtype=np.uint32)
    out = np.empty(query.shape, dtype=np.float32)
    lib().oracle_sliding_window_attention_paged_kv_f32(
        _ptr(out), _ptr(query), _ptr(key_cache), _ptr(value_cache), table.ctypes.data_as(ctypes.POINTER(ctypes.c_uint32)), _c_size(batch),
        _c_size(query_len), _c_size(key_len), _c_size(heads), _c_size(kv_heads), _c_size(head_dim), _c_size(query_start),
        _c_size(key_start), _c_size(window), _c_size(block_size), _c_size(physical_blocks), _c_size(table.shape[1]), _c_float(scale),
        _c_float(output_scale))
    return out


def splitk_reduce_f32(attn, lse, *, batch, heads, splits, head_dim):
    """singe-kernel/src/cpu/attention.rs:2157-2193."""
    attn, lse = _f32(attn), _f32(lse)
    out = np.empty(batch * heads * head_dim, dtype=np.float32)
    lib().oracle_splitk_reduce_f32(_ptr(out), _ptr(attn), _ptr(lse), _c_size(batch), _c_size(heads),
                                   _c_size(splits), _c_size(head_dim))
    return out.reshape(batch, heads, head_dim)


def fmha_decode_splitk_f32(query, key, value, *, splits, kv_len_per_split, scale):
    """singe-kernel/src/cuda/cutile/kernel/attention/local.rs:6127-6272.  query [B,H,D], key / value [B,S,G,D];
    returns (out [B,H,splits,D], lse [B,H,splits] natural log)."""
    query, key, value = _f32(query), _f32(key), _f32(value)
    batch, heads, head_dim = query.shape
    _, key_len, kv_heads, _ = key.shape
    out = np.empty((batch, heads, splits, head_dim), dtype=np.float32)
    lse = np.empty((batch, heads, splits), dtype=np.float32)
    lib().oracle_fmha_decode_splitk_f32(_ptr(out), _ptr(lse), _ptr(query), _ptr(key), _ptr(value), _c_size(batch),
                                        _c_size(key_len), _c_size(heads), _c_size(kv_heads), _c_size(splits),
                                        _c_size(kv_len_per_split), _c_size(head_dim), ctypes.c_float(scale))
    return out, lse


# ---- singe surface --------------------------------------------------------------

def scaled_dot_product_attention_f32(query, key, value, *, scale=None, causal=False, window=None,
                                     softcap=None, mask=None, sinks=None, key_lengths=None, threads=1):
    """singe/src/backend/cpu/normalization/attention.rs:20-130,191-276 (BHSD, f32).
    query [B,H,L,D], key [B,G,S,D], value [B,G,S,Dv]."""
    query, key, value = _f32(query), _f32(key), _f32(value)
    batch, heads, query_len, head_dim = query.shape
    _, kv_heads, key_len, _ = key.shape
    value_dim = value.shape[3]
    if scale is None:
        scale = float(np.float32(1.0) / np.sqrt(np.float32(head_dim)))
    mask_full = None
    if mask is not None:
        mask_full = np.ascontiguousarray(np.broadcast_to(_f32(mask), (batch, heads, query_len, key_len)))
    sinks_a = None if sinks is None else _f32(sinks)
    lens_a = None if key_lengths is None else np.ascontiguousarray(key_lengths, dtype=np.int32)
    out = np.empty((batch, heads, query_len, value_dim), dtype=np.float32)
    lib().oracle_scaled_dot_product_attention_f32(
        _ptr(out), _ptr(query), _ptr(key), _ptr(value), _ptr(mask_full), _ptr(sinks_a), _ptr(lens_a),
        _c_size(batch), _c_size(heads), _c_size(kv_heads), _c_size(query_len), _c_size(key_len),
        _c_size(head_dim), _c_size(value_dim), _c_float(scale), _c_int(bool(causal)),
        _c_i64(-1 if window is None else int(window)), _c_int(softcap is not None),
        _c_float(softcap if softcap is not None else 0.0), _c_int(threads))
    return out


def check_paged_values(query_offsets, page_offsets, pages, last_page_lengths, *, tokens, cache_pages,
                       page_size) -> int:
    """singe/src/backend/spec/neural/attention.rs:372-406; 0 = ok, 1 = index out of bounds."""
    qo = np.ascontiguousarray(query_offsets, dtype=np.int64)
    po = np.ascontiguousarray(page_offsets, dtype=np.int64)
    pg = np.ascontiguousarray(pages, dtype=np.int64)
    lp = np.ascontiguousarray(last_page_lengths, dtype=np.int64)
    return int(lib().oracle_check_paged_values(_ptr(qo), _ptr(po), _ptr(pg), _ptr(lp), _c_size(len(lp)),
                                               _c_i64(len(pg)), _c_i64(tokens), _c_i64(cache_pages),
                                               _c_i64(page_size)))


def paged_attention_f32(query, key_cache, value_cache, query_offsets, page_offsets, pages,
                        last_page_lengths, *, scale=None, causal=False, window=None, softcap=None,
                        threads=1):
    """singe/src/backend/cpu/normalization/attention.rs:297-538 (f32 compute).
    Returns (status, out [T,H,D], lse [T,H] base two); status 1 = index out of bounds."""
    query, key_cache, value_cache = _f32(query), _f32(key_cache), _f32(value_cache)
    tokens, heads, head_dim = query.shape
    cache_pages, page_size, kv_heads, _ = key_cache.shape
    qo = np.ascontiguousarray(query_offsets, dtype=np.int64)
    po = np.ascontiguousarray(page_offsets, dtype=np.int64)
    pg = np.ascontiguousarray(pages, dtype=np.int64)
    lp = np.ascontiguousarray(last_page_lengths, dtype=np.int64)
    if scale is None:
        scale = float(np.float32(1.0) / np.sqrt(np.float32(head_dim)))
    out = np.zeros((tokens, heads, head_dim), dtype=np.float32)
    lse = np.full((tokens, heads), -np.inf, dtype=np.float32)
    status = lib().oracle_paged_attention_f32(
        _ptr(out), _ptr(lse), _ptr(query), _ptr(key_cache), _ptr(value_cache), _ptr(qo), _ptr(po),
        _ptr(pg), _ptr(lp), _c_size(len(lp)), _c_size(len(pg)), _c_size(tokens), _c_size(heads),
        _c_size(kv_heads), _c_size(head_dim), _c_size(page_size), _c_size(cache_pages), _c_float(scale),
        _c_int(bool(causal)), _c_i64(-1 if window is None else int(window)),
        _c_int(softcap is not None), _c_float(softcap if softcap is not None else 0.0), _c_int(threads))
    return int(status), out, lse


def paged_mla_attention(query, query_positions, latent_cache, position_cache, query_offsets, page_offsets, pages,
                        last_page_lengths, *, scale=None, causal=False, threads=1):
    """singe/src/backend/cpu/normalization/attention.rs:540-679 (f64 compute).  query [T, H, L], query_positions
    [T, H, R], latent_cache [P, S, L], position_cache [P, S, R].  Returns (status, out [T, H, L] f32, lse [T, H]
    base two); status 1 = index out of bounds."""
    query, query_positions = _f32(query), _f32(query_positions)
    latent_cache, position_cache = _f32(latent_cache), _f32(position_cache)
    tokens, heads, latent = query.shape
    positional = query_positions.shape[2]
    cache_pages, page_size, _ = latent_cache.shape
    qo = np.ascontiguousarray(query_offsets, dtype=np.int64)
    po = np.ascontiguousarray(page_offsets, dtype=np.int64)
    pg = np.ascontiguousarray(pages, dtype=np.int64)
    lp = np.ascontiguousarray(last_page_lengths, dtype=np.int64)
    out = np.zeros((tokens, heads, latent), dtype=np.float32)
    lse = np.full((tokens, heads), -np.inf, dtype=np.float32)
    status = lib().oracle_paged_mla_attention(
        _ptr(out), _ptr(lse), _ptr(query), _ptr(query_positions), _ptr(latent_cache), _ptr(position_cache), _ptr(qo), _ptr(po),
        _ptr(pg), _ptr(lp), _c_size(len(lp)), _c_size(len(pg)), _c_size(tokens), _c_size(heads), _c_size(latent),
        _c_size(positional), _c_size(page_size), _c_size(cache_pages), _c_int(scale is not None),
        _c_float(scale if scale is not None else 0.0), _c_int(bool(causal)), _c_int(threads))
    return int(status), out, lse


def paged_slots(page_offsets, pages, last_page_lengths, *, page_size):
    """Cache row of every key, [sequence][key], and each sequence's key count
    (normalization/attention.rs:470-479)."""
    po = np.ascontiguousarray(page_offsets, dtype=np.int64)
    pg = np.ascontiguousarray(pages, dtype=np.int64)
    lp = np.ascontiguousarray(last_page_lengths, dtype=np.int64)
    counts = np.empty(len(lp), dtype=np.uint64)
    total = lib().oracle_paged_slots(None, _ptr(counts), _ptr(po), _ptr(pg), _ptr(lp), _c_size(len(lp)),
                                     _c_size(page_size))
    slots = np.empty(int(total), dtype=np.uint64)
    lib().oracle_paged_slots(_ptr(slots), _ptr(counts), _ptr(po), _ptr(pg), _ptr(lp), _c_size(len(lp)),
                             _c_size(page_size))
    return slots, counts


def rotary_embedding_f32(values, cos, sin):
    """singe/src/backend/cpu/normalization/attention.rs:132-188: values [..., sequence, head_dim], cos/sin
    [sequence, rotary_pairs]; interleaved pairs."""
    values, cos, sin = _f32(values), _f32(cos), _f32(sin)
    sequence, pairs = cos.shape
    head_dim = values.shape[-1]
    out = np.empty_like(values)
    lib().oracle_rotary_embedding_f32(_ptr(out), _ptr(values), _ptr(cos), _ptr(sin), _c_size(values.size // head_dim),
                                      _c_size(sequence), _c_size(head_dim), _c_size(pairs))
    return out


def rotary_cache_write_f32(query, key, value, cos, sin, pages, slots, key_cache, value_cache, *, query_norm=None,
                           key_norm=None, in_place=False):
    """The fused rotate-and-append step (singe/src/backend/cuda/kernel_plan/source/rotary_cache.rs:249-427).
    query [T, H, D] or None, key/value [T, G, D], cos/sin [T, D/2], caches [P, S, G, D] (copied, then the
    selected cells written; ``in_place`` writes into the caches given, contiguous float32 arrays, instead, for
    timing); a norm is (eps, weight or None).  Returns (status, query_out, key_cache, value_cache)."""
    key, value, cos, sin = _f32(key), _f32(value), _f32(cos), _f32(sin)
    if in_place:
        assert all(c.dtype == np.float32 and c.flags["C_CONTIGUOUS"] for c in (key_cache, value_cache))
    else:
        key_cache, value_cache = _f32(key_cache).copy(), _f32(value_cache).copy()
    tokens, cache_heads, head_dim = key.shape
    cache_pages, page_slots = key_cache.shape[:2]
    query_heads = 0 if query is None else query.shape[1]
    query_a = None if query is None else _f32(query)
    query_out = None if query is None else np.zeros_like(query_a)
    pg = np.ascontiguousarray(pages, dtype=np.int64)
    sl = np.ascontiguousarray(slots, dtype=np.int64)
    def norm(spec):
        if spec is None:
            return 0, 0.0, None
        eps, weight = spec
        return 1, float(eps), (None if weight is None else _f32(weight))
    qn, qe, qw = norm(query_norm)
    kn, ke, kw = norm(key_norm)
    status = lib().oracle_rotary_cache_write_f32(
        _ptr(query_out), _ptr(key_cache), _ptr(value_cache), _ptr(query_a), _ptr(key), _ptr(value), _ptr(cos), _ptr(sin),
        _ptr(pg), _ptr(sl), _c_size(tokens), _c_size(query_heads), _c_size(cache_heads), _c_size(head_dim),
        _c_size(cache_pages), _c_size(page_slots), _c_int(qn), _c_float(qe), _ptr(qw), _c_int(kn), _c_float(ke), _ptr(kw))
    return int(status), query_out, key_cache, value_cache


def paging_indices(query_offsets, page_offsets, pages, last_page_lengths, *, tokens, page_size, cache_pages, width,
                   row_elements):
    """CSR paging -> block-table paging (kernel_plan/source/paged_attention.rs:325-398).  Returns (status,
    packed_offsets, query_lengths, key_lengths, page_table [sequences, width])."""
    qo = np.ascontiguousarray(query_offsets, dtype=np.int64)
    po = np.ascontiguousarray(page_offsets, dtype=np.int64)
    pg = np.ascontiguousarray(pages, dtype=np.int64)
    lp = np.ascontiguousarray(last_page_lengths, dtype=np.int64)
    sequences = len(lp)
    packed = np.zeros(sequences + 1, dtype=np.int32)
    query_lengths = np.zeros(sequences, dtype=np.int32)
    key_lengths = np.zeros(sequences, dtype=np.int32)
    table = np.zeros((sequences, width), dtype=np.int32)
    status = lib().oracle_paging_indices(_ptr(packed), _ptr(query_lengths), _ptr(key_lengths), _ptr(table), _ptr(qo), _ptr(po),
                                         _ptr(pg), _ptr(lp), _c_size(sequences), _c_i64(tokens), _c_i64(len(pg)),
                                         _c_i64(page_size), _c_i64(cache_pages), _c_size(width), _c_i64(row_elements))
    return int(status), packed, query_lengths, key_lengths, table
