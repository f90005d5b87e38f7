"""Host-side mirror of ``singe_kernel::cuda::attention`` for the paged / dense attention path.

Same names, argument order and error behaviour as the reference's launch functions
(singe-kernel/src/cuda/attention/paged.rs:118-420, fmha.rs:584-790) and config structs
(mod.rs:76-108, 253-274).  Device buffers are torch tensors (a pointer plus an element count, which
is all the reference's DeviceInput/DeviceOutput carry); ``stream`` is a ``torch.cuda.Stream`` or
``None`` for the current one.  Every call only enqueues work.
"""
from __future__ import annotations

import contextlib
import ctypes
import math
from dataclasses import dataclass

import torch

from .. import _native, error

I32_MAX = 2**31 - 1


def _stream_handle(stream) -> int:
    if stream is None:
        stream = torch.cuda.current_stream()
    return int(stream.cuda_stream)


def _ptr(tensor: torch.Tensor) -> int:
    return int(tensor.data_ptr())


def _require(tensor: torch.Tensor, dtype: torch.dtype, name: str) -> None:
    if not isinstance(tensor, torch.Tensor) or not tensor.is_cuda:
        raise error.NullPointer(f"{name} is not a device buffer")
    if tensor.dtype != dtype:
        raise error.InvalidArgument(f"{name} must be {dtype}, got {tensor.dtype}")
    if not tensor.is_contiguous():
        raise error.InvalidArgument(f"{name} must be contiguous")


@dataclass(frozen=True)
class PagedKvDecodeAttentionConfig:
    """Decode attention over paged KV caches (mod.rs:76-90): one query token per batch item, caches
    addressed through a per-batch block table, ``actual_seq_lens`` selecting each item's prefix."""
    batch: int
    heads: int
    kv_heads: int
    head_dim: int
    block_size: int
    physical_blocks: int
    block_table_batch_stride: int
    scale: float

    @classmethod
    def contiguous(cls, batch, heads, kv_heads, head_dim, block_size, physical_blocks,
                   block_table_batch_stride, scale) -> "PagedKvDecodeAttentionConfig":
        """mod.rs:686-709: builds the config and validates it."""
        config = cls(batch, heads, kv_heads, head_dim, block_size, physical_blocks, block_table_batch_stride, scale)
        config.validate()
        return config

    def reserve_workspace(self, device: "torch.device | None" = None) -> None:
        """Sizes this module's per-device scratch for the config now, so that a later decode call without a
        ``workspace`` of its own allocates nothing (the call is then enqueue-only, legal under stream capture, as the
        reference asks of its launch functions: singe-kernel/src/cuda/mod.rs:3-12).  Always an explicit call: building
        a config touches no device.  Without a visible GPU it does nothing."""
        if not torch.cuda.is_available():
            return
        device = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
        need = self.workspace_bytes()
        if need > 0:
            _workspaces.get(device, need)

    def validate(self) -> None:
        """validate_paged_kv_decode_attention_config (mod.rs:2963-2985)."""
        extents = (self.batch, self.heads, self.kv_heads, self.head_dim, self.block_size, self.physical_blocks,
                   self.block_table_batch_stride)
        if any(e <= 0 for e in extents) or self.heads % self.kv_heads != 0 or not math.isfinite(self.scale):
            raise error.InvalidLength("invalid length")
        if any(e > I32_MAX for e in extents):
            raise error.LengthExceedsI32("length exceeds i32")

    def output_len(self) -> int:
        return self.batch * self.heads * self.head_dim

    def _c(self) -> _native.PagedKvDecodeAttentionConfigC:
        return _native.PagedKvDecodeAttentionConfigC(self.batch, self.heads, self.kv_heads, self.head_dim,
                                                     self.block_size, self.physical_blocks,
                                                     self.block_table_batch_stride, self.scale)

    def workspace_bytes(self) -> int:
        c = self._c()
        return int(_native.lib().singe_hip_paged_kv_decode_attention_workspace_bytes(ctypes.byref(c)))


class _Workspaces:
    """Scratch per device for calls that bring none, grown on demand.  The C ABI never allocates; this host layer
    owns the scratch the way the reference's callers own split-KV scratch (mod.rs:2456-2539).  A buffer that has been
    handed out may sit in a captured graph or under work in flight on another stream, so growing never frees one:
    outgrown buffers are kept until the process ends.  Growing is refused while the current stream is being captured
    (the allocation would not be legal there, and the graph would keep a pointer this layer cannot track): size the
    scratch beforehand with ``reserve_workspace``, pass ``workspace=``, or take the entry point that allocates nothing."""

    def __init__(self):
        self._buffers = {}
        self._outgrown = []

    def get(self, device: torch.device, nbytes: int) -> torch.Tensor:
        key = device.index if device.index is not None else torch.cuda.current_device()
        buffer = self._buffers.get(key)
        if buffer is None or buffer.numel() < nbytes:
            if torch.cuda.is_current_stream_capturing():
                raise error.UnsupportedConfiguration(
                    f"a call under stream capture needs {nbytes} bytes of scratch and the reserved buffer holds "
                    f"{0 if buffer is None else buffer.numel()}: call reserve_workspace() on the config before the "
                    "capture, pass workspace=, or use paged_kv_decode_attention_no_alloc_bf16")
            if buffer is not None:
                self._outgrown.append(buffer)
            buffer = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=device)
            self._buffers[key] = buffer
        return buffer


_workspaces = _Workspaces()


def paged_kv_decode_attention_bf16(stream, out: torch.Tensor, query: torch.Tensor, key_cache: torch.Tensor,
                                   value_cache: torch.Tensor, actual_seq_lens: torch.Tensor,
                                   block_table: torch.Tensor, config: PagedKvDecodeAttentionConfig,
                                   workspace: torch.Tensor | None = None, phases: int = 3) -> None:
    """paged_kv_decode_attention_bf16 (paged.rs:210-249).

    out/query [batch, heads, dim] bf16; caches [blocks, block_size, kv_heads, dim] bf16;
    actual_seq_lens [batch] i32; block_table [batch, stride] u32 (an int32 tensor is read as u32).
    ``phases``: 1 = split kernel only (fills the scratch), 2 = reduce only, 3 = both (the op).
    """
    _require(out, torch.bfloat16, "out")
    _require(query, torch.bfloat16, "query")
    _require(key_cache, torch.bfloat16, "key_cache")
    _require(value_cache, torch.bfloat16, "value_cache")
    _require(actual_seq_lens, torch.int32, "actual_seq_lens")
    if block_table.dtype not in (torch.int32, torch.uint32):
        raise error.InvalidArgument(f"block_table must hold 32-bit entries, got {block_table.dtype}")
    _require(block_table, block_table.dtype, "block_table")
    c = config._c()
    if workspace is None:
        need = int(_native.lib().singe_hip_paged_kv_decode_attention_workspace_bytes(ctypes.byref(c)))
        workspace = _workspaces.get(out.device, need)
    status = _native.lib().singe_hip_paged_kv_decode_attention_phases_bf16(
        _stream_handle(stream), _ptr(out), out.numel(), _ptr(query), query.numel(), _ptr(key_cache),
        key_cache.numel(), _ptr(value_cache), value_cache.numel(), _ptr(actual_seq_lens),
        actual_seq_lens.numel(), _ptr(block_table), block_table.numel(), _ptr(workspace),
        workspace.numel() * workspace.element_size(), ctypes.byref(c), phases)
    _native.check(status, "paged_kv_decode_attention_bf16")


STATIC_SCRATCH_BYTES = 16 << 20


def paged_kv_decode_attention_no_alloc_bf16(stream, out: torch.Tensor, query: torch.Tensor, key_cache: torch.Tensor,
                                            value_cache: torch.Tensor, actual_seq_lens: torch.Tensor,
                                            block_table: torch.Tensor, config: PagedKvDecodeAttentionConfig) -> None:
    """paged_kv_decode_attention_bf16 on the library's fixed device scratch (STATIC_SCRATCH_BYTES per GPU): neither
    this wrapper nor the library allocates, for callers that cannot (graph capture, serving loops).  Calls that
    overlap on one GPU share the scratch and race.  No counterpart in the reference."""
    _require(out, torch.bfloat16, "out")
    _require(query, torch.bfloat16, "query")
    _require(key_cache, torch.bfloat16, "key_cache")
    _require(value_cache, torch.bfloat16, "value_cache")
    _require(actual_seq_lens, torch.int32, "actual_seq_lens")
    if block_table.dtype not in (torch.int32, torch.uint32):
        raise error.InvalidArgument(f"block_table must hold 32-bit entries, got {block_table.dtype}")
    _require(block_table, block_table.dtype, "block_table")
    c = config._c()
    status = _native.lib().singe_hip_paged_kv_decode_attention_no_alloc_bf16(
        _stream_handle(stream), _ptr(out), out.numel(), _ptr(query), query.numel(), _ptr(key_cache),
        key_cache.numel(), _ptr(value_cache), value_cache.numel(), _ptr(actual_seq_lens),
        actual_seq_lens.numel(), _ptr(block_table), block_table.numel(), ctypes.byref(c))
    _native.check(status, "paged_kv_decode_attention_no_alloc_bf16")


def paged_kv_decode_attention_f8e4m3kv_bf16(stream, out: torch.Tensor, query: torch.Tensor, key_cache: torch.Tensor,
                                            value_cache: torch.Tensor, key_scales: torch.Tensor,
                                            value_scales: torch.Tensor, actual_seq_lens: torch.Tensor,
                                            block_table: torch.Tensor, config: PagedKvDecodeAttentionConfig,
                                            workspace: torch.Tensor | None = None, phases: int = 3) -> None:
    """Paged decode over an fp8 e4m3 KV cache (uint8 codes, or torch.float8_e4m3fn) with one f32 scale
    per (block, kv head); same result as paged_kv_decode_attention_bf16 on the cache dequantised to
    bf16_rne(f8e4m3_value(code) * scale).  No counterpart in the reference's launch API."""
    _require(out, torch.bfloat16, "out")
    _require(query, torch.bfloat16, "query")
    for tensor, name in ((key_cache, "key_cache"), (value_cache, "value_cache")):
        if tensor.dtype not in (torch.uint8, torch.float8_e4m3fn):
            raise error.InvalidArgument(f"{name} must hold fp8 e4m3 codes, got {tensor.dtype}")
        _require(tensor, tensor.dtype, name)
    _require(key_scales, torch.float32, "key_scales")
    _require(value_scales, torch.float32, "value_scales")
    _require(actual_seq_lens, torch.int32, "actual_seq_lens")
    if block_table.dtype not in (torch.int32, torch.uint32):
        raise error.InvalidArgument(f"block_table must hold 32-bit entries, got {block_table.dtype}")
    _require(block_table, block_table.dtype, "block_table")
    c = config._c()
    if workspace is None:
        need = int(_native.lib().singe_hip_paged_kv_decode_attention_workspace_bytes(ctypes.byref(c)))
        workspace = _workspaces.get(out.device, need)
    status = _native.lib().singe_hip_paged_kv_decode_attention_f8e4m3kv_bf16(
        _stream_handle(stream), _ptr(out), out.numel(), _ptr(query), query.numel(), _ptr(key_cache),
        key_cache.numel(), _ptr(value_cache), value_cache.numel(), _ptr(key_scales), key_scales.numel(),
        _ptr(value_scales), value_scales.numel(), _ptr(actual_seq_lens), actual_seq_lens.numel(),
        _ptr(block_table), block_table.numel(), _ptr(workspace), workspace.numel() * workspace.element_size(),
        ctypes.byref(c), phases)
    _native.check(status, "paged_kv_decode_attention_f8e4m3kv_bf16")


def set_relaxed_numerics(relaxed: bool) -> None:
    """NumericalPolicy precision: Full (False, default) or Relaxed (True)."""
    _native.lib().singe_hip_set_relaxed_numerics(1 if relaxed else 0)


@contextlib.contextmanager
def thread_options(relaxed: "bool | None" = None, decode_workers: int = 0, paged_attention_splits: int = 0,
                   paged_mla_attention_splits: int = 0, split_below_blocks: "int | None" = None):
    """The calling thread's own settings for the calls inside the block, like NumericalPolicy::scope
    (singe/src/graph/numerics/mod.rs:44-49) and a TuningChoice::Explicit carried by the call: size queries and
    launches made by this thread read them whatever other threads or the process-wide setters say; the thread's
    previous options come back on exit.  None / 0 follow the process-wide setting."""
    lib = _native.lib()
    before = _native.ThreadOptionsC()
    lib.singe_hip_thread_options(ctypes.byref(before))
    wanted = _native.ThreadOptionsC(-1 if relaxed is None else int(bool(relaxed)), decode_workers, paged_attention_splits,
                                    paged_mla_attention_splits, split_below_blocks is not None, split_below_blocks or 0)
    _native.check(lib.singe_hip_set_thread_options(ctypes.byref(wanted)), "thread_options")
    try:
        yield
    finally:
        lib.singe_hip_set_thread_options(ctypes.byref(before))


@dataclass(frozen=True)
class PagedKvPrefillAttentionConfig:
    """Prefill attention over paged KV caches (mod.rs:92-108): query tokens packed across the batch and
    indexed by sequence offsets, K/V cache tokens addressed through a block table."""
    batch: int
    total_query_tokens: int
    heads: int
    kv_heads: int
    head_dim: int
    block_size: int
    physical_blocks: int
    block_table_batch_stride: int
    causal: bool
    scale: float

    @classmethod
    def contiguous(cls, batch, total_query_tokens, heads, kv_heads, head_dim, block_size, physical_blocks,
                   block_table_batch_stride, causal, scale) -> "PagedKvPrefillAttentionConfig":
        """mod.rs:746-773: builds the config and validates it."""
        config = cls(batch, total_query_tokens, heads, kv_heads, head_dim, block_size, physical_blocks,
                     block_table_batch_stride, bool(causal), scale)
        config.validate()
        return config

    def validate(self) -> None:
        """validate_paged_kv_prefill_attention_config (mod.rs:2987-3011)."""
        extents = (self.batch, self.total_query_tokens, self.heads, self.kv_heads, self.head_dim, self.block_size,
                   self.physical_blocks, self.block_table_batch_stride)
        if any(e <= 0 for e in extents) or self.heads % self.kv_heads != 0 or not math.isfinite(self.scale):
            raise error.InvalidLength("invalid length")
        if any(e > I32_MAX for e in extents):
            raise error.LengthExceedsI32("length exceeds i32")

    def output_len(self) -> int:
        return self.total_query_tokens * self.heads * self.head_dim

    def lse_len(self) -> int:
        return self.total_query_tokens * self.heads

    def _c(self) -> _native.PagedKvPrefillAttentionConfigC:
        return _native.PagedKvPrefillAttentionConfigC(self.batch, self.total_query_tokens, self.heads, self.kv_heads,
                                                      self.head_dim, self.block_size, self.physical_blocks,
                                                      self.block_table_batch_stride, 1 if self.causal else 0,
                                                      self.scale)


def paged_kv_prefill_attention_bf16(stream, out: torch.Tensor, lse: torch.Tensor, query: torch.Tensor,
                                    key_cache: torch.Tensor, value_cache: torch.Tensor,
                                    actual_seq_lens_q: torch.Tensor, actual_seq_lens_kv: torch.Tensor,
                                    actual_seq_offsets: torch.Tensor, block_table: torch.Tensor,
                                    config: PagedKvPrefillAttentionConfig) -> None:
    """paged_kv_prefill_attention_bf16 (paged.rs:370-420).

    out/query [total_query_tokens, heads, dim] bf16; lse [total_query_tokens, heads] f32 (natural log,
    -1e20 for a row without keys); caches [blocks, block_size, kv_heads, dim] bf16; the three per-sequence
    vectors [batch] i32; block_table [batch, stride] u32.  Causal hides key index > query index.
    """
    _require(out, torch.bfloat16, "out")
    _require(lse, torch.float32, "lse")
    _require(query, torch.bfloat16, "query")
    _require(key_cache, torch.bfloat16, "key_cache")
    _require(value_cache, torch.bfloat16, "value_cache")
    _require(actual_seq_lens_q, torch.int32, "actual_seq_lens_q")
    _require(actual_seq_lens_kv, torch.int32, "actual_seq_lens_kv")
    _require(actual_seq_offsets, torch.int32, "actual_seq_offsets")
    if block_table.dtype not in (torch.int32, torch.uint32):
        raise error.InvalidArgument(f"block_table must hold 32-bit entries, got {block_table.dtype}")
    _require(block_table, block_table.dtype, "block_table")
    c = config._c()
    status = _native.lib().singe_hip_paged_kv_prefill_attention_bf16(
        _stream_handle(stream), _ptr(out), out.numel(), _ptr(lse), lse.numel(), _ptr(query), query.numel(),
        _ptr(key_cache), key_cache.numel(), _ptr(value_cache), value_cache.numel(), _ptr(actual_seq_lens_q),
        actual_seq_lens_q.numel(), _ptr(actual_seq_lens_kv), actual_seq_lens_kv.numel(), _ptr(actual_seq_offsets),
        actual_seq_offsets.numel(), _ptr(block_table), block_table.numel(), ctypes.byref(c))
    _native.check(status, "paged_kv_prefill_attention_bf16")


def paged_kv_prefill_attention_f16(stream, out: torch.Tensor, lse: torch.Tensor, query: torch.Tensor,
                                    key_cache: torch.Tensor, value_cache: torch.Tensor,
                                    actual_seq_lens_q: torch.Tensor, actual_seq_lens_kv: torch.Tensor,
                                    actual_seq_offsets: torch.Tensor, block_table: torch.Tensor,
                                    config: PagedKvPrefillAttentionConfig) -> None:
    """paged_kv_prefill_attention_f16 (paged.rs): the bf16 op on f16 operands.

    out/query [total_query_tokens, heads, dim] f16; lse [total_query_tokens, heads] f32 (natural log,
    -1e20 for a row without keys); caches [blocks, block_size, kv_heads, dim] f16; the three per-sequence
    vectors [batch] i32; block_table [batch, stride] u32.  Causal hides key index > query index.
    """
    _require(out, torch.float16, "out")
    _require(lse, torch.float32, "lse")
    _require(query, torch.float16, "query")
    _require(key_cache, torch.float16, "key_cache")
    _require(value_cache, torch.float16, "value_cache")
    _require(actual_seq_lens_q, torch.int32, "actual_seq_lens_q")
    _require(actual_seq_lens_kv, torch.int32, "actual_seq_lens_kv")
    _require(actual_seq_offsets, torch.int32, "actual_seq_offsets")
    if block_table.dtype not in (torch.int32, torch.uint32):
        raise error.InvalidArgument(f"block_table must hold 32-bit entries, got {block_table.dtype}")
    _require(block_table, block_table.dtype, "block_table")
    c = config._c()
    status = _native.lib().singe_hip_paged_kv_prefill_attention_f16(
        _stream_handle(stream), _ptr(out), out.numel(), _ptr(lse), lse.numel(), _ptr(query), query.numel(),
        _ptr(key_cache), key_cache.numel(), _ptr(value_cache), value_cache.numel(), _ptr(actual_seq_lens_q),
        actual_seq_lens_q.numel(), _ptr(actual_seq_lens_kv), actual_seq_lens_kv.numel(), _ptr(actual_seq_offsets),
        actual_seq_offsets.numel(), _ptr(block_table), block_table.numel(), ctypes.byref(c))
    _native.check(status, "paged_kv_prefill_attention_f16")


@dataclass(frozen=True)
class FmhaPrefillConfig:
    """Dense prefill attention (mod.rs:253-274): query/out [batch, query_len, heads, dim], key/value
    [batch, key_len, kv_heads, dim], addressed through element strides; ``causal`` is top-left."""
    batch: int
    query_len: int
    key_len: int
    heads: int
    kv_heads: int
    head_dim: int
    query_batch_stride: int
    key_batch_stride: int
    value_batch_stride: int
    output_batch_stride: int
    query_sequence_stride: int
    key_sequence_stride: int
    value_sequence_stride: int
    output_sequence_stride: int
    query_head_stride: int
    key_head_stride: int
    value_head_stride: int
    output_head_stride: int
    scale: float
    causal: bool

    @classmethod
    def contiguous(cls, batch, query_len, key_len, heads, kv_heads, head_dim, scale, causal) -> "FmhaPrefillConfig":
        """mod.rs:1602-1632: packed [batch, len, heads, dim] strides.  Like the reference, this does
        not validate; the launch functions do."""
        q_features, kv_features = heads * head_dim, kv_heads * head_dim
        return cls(batch, query_len, key_len, heads, kv_heads, head_dim, query_len * q_features,
                   key_len * kv_features, key_len * kv_features, query_len * q_features, q_features, kv_features,
                   kv_features, q_features, head_dim, head_dim, head_dim, head_dim, scale, causal)

    def _c(self) -> _native.FmhaPrefillConfigC:
        return _native.FmhaPrefillConfigC(
            self.batch, self.query_len, self.key_len, self.heads, self.kv_heads, self.head_dim,
            self.query_batch_stride, self.key_batch_stride, self.value_batch_stride, self.output_batch_stride,
            self.query_sequence_stride, self.key_sequence_stride, self.value_sequence_stride,
            self.output_sequence_stride, self.query_head_stride, self.key_head_stride, self.value_head_stride,
            self.output_head_stride, self.scale, 1 if self.causal else 0)


def fmha_prefill_bf16(stream, out: torch.Tensor, query: torch.Tensor, key: torch.Tensor, value: torch.Tensor,
                      config: FmhaPrefillConfig) -> None:
    """fmha_prefill_bf16 (fmha.rs:744-790)."""
    for tensor, name in ((out, "out"), (query, "query"), (key, "key"), (value, "value")):
        _require(tensor, torch.bfloat16, name)
    c = config._c()
    status = _native.lib().singe_hip_fmha_prefill_bf16(
        _stream_handle(stream), _ptr(out), out.numel(), _ptr(query), query.numel(), _ptr(key), key.numel(),
        _ptr(value), value.numel(), ctypes.byref(c))
    _native.check(status, "fmha_prefill_bf16")


def fmha_prefill_lse_bf16(stream, out: torch.Tensor, lse: torch.Tensor, query: torch.Tensor, key: torch.Tensor,
                          value: torch.Tensor, config: FmhaPrefillConfig) -> None:
    """fmha_prefill_lse_bf16 (fmha.rs:638-690): also writes lse [batch, heads, query_len], natural log."""
    for tensor, name in ((out, "out"), (query, "query"), (key, "key"), (value, "value")):
        _require(tensor, torch.bfloat16, name)
    _require(lse, torch.float32, "lse")
    c = config._c()
    status = _native.lib().singe_hip_fmha_prefill_lse_bf16(
        _stream_handle(stream), _ptr(out), out.numel(), _ptr(lse), lse.numel(), _ptr(query), query.numel(),
        _ptr(key), key.numel(), _ptr(value), value.numel(), ctypes.byref(c))
    _native.check(status, "fmha_prefill_lse_bf16")


def fmha_prefill_f16(stream, out: torch.Tensor, query: torch.Tensor, key: torch.Tensor, value: torch.Tensor,
                     config: FmhaPrefillConfig) -> None:
    """fmha_prefill_f16 (fmha.rs:692-742)."""
    for tensor, name in ((out, "out"), (query, "query"), (key, "key"), (value, "value")):
        _require(tensor, torch.float16, name)
    c = config._c()
    status = _native.lib().singe_hip_fmha_prefill_f16(
        _stream_handle(stream), _ptr(out), out.numel(), _ptr(query), query.numel(), _ptr(key), key.numel(),
        _ptr(value), value.numel(), ctypes.byref(c))
    _native.check(status, "fmha_prefill_f16")


def fmha_prefill_lse_f16(stream, out: torch.Tensor, lse: torch.Tensor, query: torch.Tensor, key: torch.Tensor,
                         value: torch.Tensor, config: FmhaPrefillConfig) -> None:
    """fmha_prefill_lse_f16 (fmha.rs:584-636): also writes lse [batch, heads, query_len], natural log."""
    for tensor, name in ((out, "out"), (query, "query"), (key, "key"), (value, "value")):
        _require(tensor, torch.float16, name)
    _require(lse, torch.float32, "lse")
    c = config._c()
    status = _native.lib().singe_hip_fmha_prefill_lse_f16(
        _stream_handle(stream), _ptr(out), out.numel(), _ptr(lse), lse.numel(), _ptr(query), query.numel(),
        _ptr(key), key.numel(), _ptr(value), value.numel(), ctypes.byref(c))
    _native.check(status, "fmha_prefill_lse_f16")


def fmha_prefill_f32(stream, out: torch.Tensor, query: torch.Tensor, key: torch.Tensor, value: torch.Tensor,
                     config: FmhaPrefillConfig) -> None:
    """fmha_prefill_f32 (fmha.rs:146-190): any head_dim up to 256, any strides."""
    for tensor, name in ((out, "out"), (query, "query"), (key, "key"), (value, "value")):
        _require(tensor, torch.float32, name)
    c = config._c()
    status = _native.lib().singe_hip_fmha_prefill_f32(
        _stream_handle(stream), _ptr(out), out.numel(), _ptr(query), query.numel(), _ptr(key), key.numel(),
        _ptr(value), value.numel(), ctypes.byref(c))
    _native.check(status, "fmha_prefill_f32")


def fmha_prefill_lse_f32(stream, out: torch.Tensor, lse: torch.Tensor, query: torch.Tensor, key: torch.Tensor,
                         value: torch.Tensor, config: FmhaPrefillConfig) -> None:
    """fmha_prefill_lse_f32 (fmha.rs:48-95)."""
    for tensor, name in ((out, "out"), (lse, "lse"), (query, "query"), (key, "key"), (value, "value")):
        _require(tensor, torch.float32, name)
    c = config._c()
    status = _native.lib().singe_hip_fmha_prefill_lse_f32(
        _stream_handle(stream), _ptr(out), out.numel(), _ptr(lse), lse.numel(), _ptr(query), query.numel(),
        _ptr(key), key.numel(), _ptr(value), value.numel(), ctypes.byref(c))
    _native.check(status, "fmha_prefill_lse_f32")


@dataclass(frozen=True)
class SoftcappedWindowAttentionConfig:
    """mod.rs:292-296: dense attention with an optional symmetric window and tanh soft cap."""
    attention: FmhaPrefillConfig
    window_size: int = 0
    soft_cap: float | None = None


def softcapped_window_attention_f32(stream, out: torch.Tensor, query: torch.Tensor, key: torch.Tensor,
                                    value: torch.Tensor, config: SoftcappedWindowAttentionConfig) -> None:
    """softcapped_window_attention_f32 (fmha.rs:245-290)."""
    for tensor, name in ((out, "out"), (query, "query"), (key, "key"), (value, "value")):
        _require(tensor, torch.float32, name)
    c = _native.SoftcappedWindowAttentionConfigC(config.attention._c(), config.window_size,
                                                 1 if config.soft_cap is not None else 0,
                                                 config.soft_cap if config.soft_cap is not None else 0.0)
    status = _native.lib().singe_hip_softcapped_window_attention_f32(
        _stream_handle(stream), _ptr(out), out.numel(), _ptr(query), query.numel(), _ptr(key), key.numel(),
        _ptr(value), value.numel(), ctypes.byref(c))
    _native.check(status, "softcapped_window_attention_f32")


def bhsd_config(batch, heads, kv_heads, query_len, key_len, head_dim, scale, causal) -> FmhaPrefillConfig:
    """FmhaPrefillConfig strides for tensors stored [batch, heads, len, dim] (the order of the CPU
    softcapped_window_attention_f32 and of singe's scaled_dot_product_attention)."""
    return FmhaPrefillConfig(batch, query_len, key_len, heads, kv_heads, head_dim,
                             heads * query_len * head_dim, kv_heads * key_len * head_dim, kv_heads * key_len * head_dim,
                             heads * query_len * head_dim, head_dim, head_dim, head_dim, head_dim,
                             query_len * head_dim, key_len * head_dim, key_len * head_dim, query_len * head_dim,
                             scale, causal)


@dataclass(frozen=True)
class SplitKReduceConfig:
    """SplitKReduceConfig (mod.rs:385-398): strides in elements."""
    batch: int
    heads: int
    splits: int
    head_dim: int
    attn_batch_stride: int
    attn_head_stride: int
    attn_split_stride: int
    lse_batch_stride: int
    lse_head_stride: int
    output_batch_stride: int
    output_head_stride: int

    @classmethod
    def contiguous(cls, batch, heads, splits, head_dim) -> "SplitKReduceConfig":
        """mod.rs:2312-2328: attn [batch, heads, splits, dim], lse [batch, heads, splits], out [batch, heads, dim]."""
        return cls(batch, heads, splits, head_dim, heads * splits * head_dim, splits * head_dim, head_dim,
                   heads * splits, splits, heads * head_dim, head_dim)

    def _c(self) -> _native.SplitKReduceConfigC:
        return _native.SplitKReduceConfigC(self.batch, self.heads, self.splits, self.head_dim, self.attn_batch_stride,
                                           self.attn_head_stride, self.attn_split_stride, self.lse_batch_stride,
                                           self.lse_head_stride, self.output_batch_stride, self.output_head_stride)


def splitk_reduce_f32(stream, out: torch.Tensor, attn_splitk: torch.Tensor, lse_splitk: torch.Tensor,
                      config: SplitKReduceConfig) -> None:
    """splitk_reduce_f32 (fmha.rs:1038-1067): folds per-split partial rows and natural-log LSEs."""
    _require(out, torch.float32, "out")
    _require(attn_splitk, torch.float32, "attn_splitk")
    _require(lse_splitk, torch.float32, "lse_splitk")
    c = config._c()
    status = _native.lib().singe_hip_splitk_reduce_f32(_stream_handle(stream), _ptr(out), out.numel(), _ptr(attn_splitk),
                                                       attn_splitk.numel(), _ptr(lse_splitk), lse_splitk.numel(),
                                                       ctypes.byref(c))
    _native.check(status, "splitk_reduce_f32")


@dataclass(frozen=True)
class FmhaDecodeConfig:
    """FmhaDecodeConfig (mod.rs:366-383): one query per (batch, head); query / out [batch, heads, dim], key /
    value [batch, key_len, kv_heads, dim]; strides in elements."""
    batch: int
    key_len: int
    heads: int
    kv_heads: int
    head_dim: int
    query_batch_stride: int
    key_batch_stride: int
    value_batch_stride: int
    output_batch_stride: int
    query_head_stride: int
    key_sequence_stride: int
    value_sequence_stride: int
    output_head_stride: int
    key_head_stride: int
    value_head_stride: int
    scale: float

    @classmethod
    def contiguous(cls, batch, key_len, heads, kv_heads, head_dim, scale) -> "FmhaDecodeConfig":
        """mod.rs:2233-2261."""
        q_features, kv_features = heads * head_dim, kv_heads * head_dim
        return cls(batch, key_len, heads, kv_heads, head_dim, q_features, key_len * kv_features, key_len * kv_features,
                   q_features, head_dim, kv_features, kv_features, head_dim, head_dim, head_dim, scale)

    def _c(self) -> _native.FmhaDecodeConfigC:
        return _native.FmhaDecodeConfigC(*(getattr(self, name) for name in _native._DECODE_FIELDS), self.scale)


@dataclass(frozen=True)
class FmhaDecodeSplitKConfig:
    """FmhaDecodeSplitKConfig (mod.rs:401-423): the decode layout plus the split count, the keys per split and
    where each split's partial output and LSE go."""
    batch: int
    key_len: int
    heads: int
    kv_heads: int
    splits: int
    kv_len_per_split: int
    head_dim: int
    query_batch_stride: int
    key_batch_stride: int
    value_batch_stride: int
    output_batch_stride: int
    query_head_stride: int
    key_sequence_stride: int
    value_sequence_stride: int
    output_head_stride: int
    output_split_stride: int
    key_head_stride: int
    value_head_stride: int
    lse_batch_stride: int
    lse_head_stride: int
    scale: float

    @classmethod
    def contiguous(cls, batch, key_len, heads, kv_heads, splits, kv_len_per_split, head_dim, scale) -> "FmhaDecodeSplitKConfig":
        """mod.rs:2662-2697: out [batch, heads, splits, dim], lse [batch, heads, splits]."""
        q_features, kv_features, split_values = heads * head_dim, kv_heads * head_dim, splits * head_dim
        return cls(batch, key_len, heads, kv_heads, splits, kv_len_per_split, head_dim, q_features,
                   key_len * kv_features, key_len * kv_features, heads * split_values, head_dim, kv_features,
                   kv_features, split_values, head_dim, head_dim, head_dim, heads * splits, splits, scale)

    def _c(self) -> _native.FmhaDecodeSplitKConfigC:
        names = [name for name, _ in _native.FmhaDecodeSplitKConfigC._fields_]
        return _native.FmhaDecodeSplitKConfigC(*(getattr(self, name) for name in names))


def fmha_decode_splitk_f32(stream, out: torch.Tensor, lse: torch.Tensor, query: torch.Tensor, key: torch.Tensor,
                           value: torch.Tensor, config: FmhaDecodeSplitKConfig) -> None:
    """fmha_decode_splitk_f32 (fmha.rs:1074-1118): per split a normalised partial output and a natural-log LSE
    (zeros and -1e20 for a split without keys)."""
    for tensor, name in ((out, "out"), (lse, "lse"), (query, "query"), (key, "key"), (value, "value")):
        _require(tensor, torch.float32, name)
    c = config._c()
    status = _native.lib().singe_hip_fmha_decode_splitk_f32(
        _stream_handle(stream), _ptr(out), out.numel(), _ptr(lse), lse.numel(), _ptr(query), query.numel(), _ptr(key),
        key.numel(), _ptr(value), value.numel(), ctypes.byref(c))
    _native.check(status, "fmha_decode_splitk_f32")


@dataclass(frozen=True)
class AttentionSplitKTuning:
    """AttentionSplitKTuning (mod.rs:442-450)."""
    splits: int

    @classmethod
    def create(cls, splits: int) -> "AttentionSplitKTuning":
        return cls(splits)


@dataclass(frozen=True)
class TuneOptions:
    """TuneOptions (singe-kernel/src/cuda/autotune.rs:34-71): zero repeats count as one."""
    warmup: int = 1
    repeats: int = 5
    max_candidates: int = 2**64 - 1

    @classmethod
    def create(cls, warmup: int, repeats: int, max_candidates: int) -> "TuneOptions":
        return cls(warmup, repeats, max_candidates)


@dataclass(frozen=True)
class TuningChoice:
    """TuningChoice<T> (autotune.rs:77-89): ``kind`` is one of the class constants; ``value`` the explicit
    tuning or the options of Tune / Retune."""
    kind: int = 0
    value: object = None

    DEFAULT, EXPLICIT, CACHED, TUNE, RETUNE = range(5)

    @classmethod
    def Default(cls) -> "TuningChoice":
        return cls(cls.DEFAULT)

    @classmethod
    def Explicit(cls, tuning: AttentionSplitKTuning) -> "TuningChoice":
        return cls(cls.EXPLICIT, tuning)

    @classmethod
    def Cached(cls) -> "TuningChoice":
        return cls(cls.CACHED)

    @classmethod
    def Tune(cls, options: TuneOptions) -> "TuningChoice":
        return cls(cls.TUNE, options)

    @classmethod
    def Retune(cls, options: TuneOptions) -> "TuningChoice":
        return cls(cls.RETUNE, options)


@dataclass(frozen=True)
class FmhaDecodeSplitKReduceConfig:
    """FmhaDecodeSplitKReduceConfig (mod.rs:452-505)."""
    decode: FmhaDecodeConfig
    max_splits: int
    tuning: TuningChoice = TuningChoice()

    @classmethod
    def contiguous(cls, batch, key_len, heads, kv_heads, head_dim, max_splits, scale) -> "FmhaDecodeSplitKReduceConfig":
        """mod.rs:461-478: validates, unlike the other ``contiguous`` builders
        (validate_fmha_decode_splitk_reduce_config, mod.rs:2554-2560)."""
        decode = FmhaDecodeConfig.contiguous(batch, key_len, heads, kv_heads, head_dim, scale)
        extents = [getattr(decode, name) for name in _native._DECODE_FIELDS]
        if any(extent == 0 for extent in extents) or not math.isfinite(scale) or heads % kv_heads != 0 or max_splits == 0:
            raise error.InvalidLength("invalid length")
        return cls(decode, max_splits)

    def with_tuning(self, tuning: TuningChoice) -> "FmhaDecodeSplitKReduceConfig":
        return FmhaDecodeSplitKReduceConfig(self.decode, self.max_splits, tuning)

    def explicit_tuning(self, tuning: AttentionSplitKTuning) -> "FmhaDecodeSplitKReduceConfig":
        return self.with_tuning(TuningChoice.Explicit(tuning))

    def cached_tuning(self) -> "FmhaDecodeSplitKReduceConfig":
        return self.with_tuning(TuningChoice.Cached())

    def tune(self, options: TuneOptions) -> "FmhaDecodeSplitKReduceConfig":
        return self.with_tuning(TuningChoice.Tune(options))

    def retune(self, options: TuneOptions) -> "FmhaDecodeSplitKReduceConfig":
        return self.with_tuning(TuningChoice.Retune(options))

    def _c(self) -> _native.FmhaDecodeSplitKReduceConfigC:
        explicit = self.tuning.value.splits if self.tuning.kind == TuningChoice.EXPLICIT else 0
        options = self.tuning.value if self.tuning.kind in (TuningChoice.TUNE, TuningChoice.RETUNE) else TuneOptions()
        return _native.FmhaDecodeSplitKReduceConfigC(
            self.decode._c(), self.max_splits, self.tuning.kind, explicit,
            _native.TuneOptionsC(options.warmup, options.repeats, min(options.max_candidates, 2**64 - 1)))


def attention_splitk_candidates(config: FmhaDecodeSplitKReduceConfig) -> list:
    """attention_splitk_candidates (mod.rs:2364-2380): the split counts tuning tries."""
    c = config._c()
    found = (_native.c_size * 16)()
    count = _native.c_size(0)
    _native.check(_native.lib().singe_hip_attention_splitk_candidates(ctypes.byref(c), found, 16, ctypes.byref(count)),
                  "attention_splitk_candidates")
    return [AttentionSplitKTuning(int(found[i])) for i in range(min(int(count.value), 16))]


def fmha_decode_splitk_reduce_f32(stream, out: torch.Tensor, attn_scratch: torch.Tensor, lse_scratch: torch.Tensor,
                                  query: torch.Tensor, key: torch.Tensor, value: torch.Tensor,
                                  config: FmhaDecodeSplitKReduceConfig) -> None:
    """fmha_decode_splitk_reduce_f32 (fmha.rs:1155-1250): the split kernel into the caller's scratch, then the
    reduce, with the split count the config's TuningChoice asks for."""
    for tensor, name in ((out, "out"), (attn_scratch, "attn_scratch"), (lse_scratch, "lse_scratch"), (query, "query"),
                         (key, "key"), (value, "value")):
        _require(tensor, torch.float32, name)
    c = config._c()
    status = _native.lib().singe_hip_fmha_decode_splitk_reduce_f32(
        _stream_handle(stream), _ptr(out), out.numel(), _ptr(attn_scratch), attn_scratch.numel(), _ptr(lse_scratch),
        lse_scratch.numel(), _ptr(query), query.numel(), _ptr(key), key.numel(), _ptr(value), value.numel(),
        ctypes.byref(c))
    _native.check(status, "fmha_decode_splitk_reduce_f32")


def tune_fmha_decode_splitk_reduce_f32(stream, out: torch.Tensor, attn_scratch: torch.Tensor, lse_scratch: torch.Tensor,
                                       query: torch.Tensor, key: torch.Tensor, value: torch.Tensor,
                                       config: FmhaDecodeSplitKReduceConfig, options: TuneOptions) -> AttentionSplitKTuning:
    """tune_fmha_decode_splitk_reduce_f32 (fmha.rs:1257-1313): times the candidates again, caches the winner and
    returns it; ``out`` holds the winner's result."""
    fmha_decode_splitk_reduce_f32(stream, out, attn_scratch, lse_scratch, query, key, value, config.retune(options))
    return cached_fmha_decode_splitk_reduce_tuning(config)


def cached_fmha_decode_splitk_reduce_tuning(config: FmhaDecodeSplitKReduceConfig):
    """The cached winner for this problem on the current device, or None."""
    c = config._c()
    splits = _native.c_size(0)
    _native.check(_native.lib().singe_hip_fmha_decode_splitk_reduce_tuned_splits(ctypes.byref(c), ctypes.byref(splits)),
                  "fmha_decode_splitk_reduce_f32")
    return AttentionSplitKTuning(int(splits.value)) if splits.value else None


def clear_tune_cache() -> None:
    """MemoryTuneCache::clear."""
    _native.lib().singe_hip_clear_tune_cache()


def paged_kv_decode_attention_f32(stream, out: torch.Tensor, query: torch.Tensor, key_cache: torch.Tensor,
                                  value_cache: torch.Tensor, actual_seq_lens: torch.Tensor, block_table: torch.Tensor,
                                  config: PagedKvDecodeAttentionConfig, workspace: torch.Tensor | None = None) -> None:
    """paged_kv_decode_attention_f32 (paged.rs; CPU form cpu/attention.rs:1172-1246): the bf16 op's operands in f32."""
    for tensor, name in ((out, "out"), (query, "query"), (key_cache, "key_cache"), (value_cache, "value_cache")):
        _require(tensor, torch.float32, name)
    _require(actual_seq_lens, torch.int32, "actual_seq_lens")
    if block_table.dtype not in (torch.int32, torch.uint32):
        raise error.InvalidArgument(f"block_table must hold 32-bit entries, got {block_table.dtype}")
    _require(block_table, block_table.dtype, "block_table")
    c = config._c()
    if workspace is None:
        need = int(_native.lib().singe_hip_paged_kv_decode_attention_f32_workspace_bytes(ctypes.byref(c)))
        workspace = _workspaces.get(out.device, need)
    status = _native.lib().singe_hip_paged_kv_decode_attention_f32(
        _stream_handle(stream), _ptr(out), out.numel(), _ptr(query), query.numel(), _ptr(key_cache), key_cache.numel(),
        _ptr(value_cache), value_cache.numel(), _ptr(actual_seq_lens), actual_seq_lens.numel(), _ptr(block_table),
        block_table.numel(), _ptr(workspace), workspace.numel() * workspace.element_size(), ctypes.byref(c))
    _native.check(status, "paged_kv_decode_attention_f32")


def paged_kv_prefill_attention_f32(stream, out: torch.Tensor, lse: torch.Tensor, query: torch.Tensor,
                                   key_cache: torch.Tensor, value_cache: torch.Tensor, actual_seq_lens_q: torch.Tensor,
                                   actual_seq_lens_kv: torch.Tensor, actual_seq_offsets: torch.Tensor,
                                   block_table: torch.Tensor, config: PagedKvPrefillAttentionConfig) -> None:
    """paged_kv_prefill_attention_f32 (paged.rs; CPU form cpu/attention.rs:1248-1341): the bf16 op's operands in
    f32.  Every token row is written: zeros and an LSE of 0 where no sequence covers the token."""
    for tensor, name in ((out, "out"), (lse, "lse"), (query, "query"), (key_cache, "key_cache"), (value_cache, "value_cache")):
        _require(tensor, torch.float32, name)
    for tensor, name in ((actual_seq_lens_q, "actual_seq_lens_q"), (actual_seq_lens_kv, "actual_seq_lens_kv"),
                         (actual_seq_offsets, "actual_seq_offsets")):
        _require(tensor, torch.int32, name)
    if block_table.dtype not in (torch.int32, torch.uint32):
        raise error.InvalidArgument(f"block_table must hold 32-bit entries, got {block_table.dtype}")
    _require(block_table, block_table.dtype, "block_table")
    c = config._c()
    status = _native.lib().singe_hip_paged_kv_prefill_attention_f32(
        _stream_handle(stream), _ptr(out), out.numel(), _ptr(lse), lse.numel(), _ptr(query), query.numel(),
        _ptr(key_cache), key_cache.numel(), _ptr(value_cache), value_cache.numel(), _ptr(actual_seq_lens_q),
        actual_seq_lens_q.numel(), _ptr(actual_seq_lens_kv), actual_seq_lens_kv.numel(), _ptr(actual_seq_offsets),
        actual_seq_offsets.numel(), _ptr(block_table), block_table.numel(), ctypes.byref(c))
    _native.check(status, "paged_kv_prefill_attention_f32")


def paged_kv_decode_attention_f16(stream, out: torch.Tensor, query: torch.Tensor, key_cache: torch.Tensor,
                                  value_cache: torch.Tensor, actual_seq_lens: torch.Tensor, block_table: torch.Tensor,
                                  config: PagedKvDecodeAttentionConfig, workspace: torch.Tensor | None = None) -> None:
    """paged_kv_decode_attention_f16 (paged.rs): the bf16 op on f16 operands, same scratch."""
    for tensor, name in ((out, "out"), (query, "query"), (key_cache, "key_cache"), (value_cache, "value_cache")):
        _require(tensor, torch.float16, name)
    _require(actual_seq_lens, torch.int32, "actual_seq_lens")
    if block_table.dtype not in (torch.int32, torch.uint32):
        raise error.InvalidArgument(f"block_table must hold 32-bit entries, got {block_table.dtype}")
    _require(block_table, block_table.dtype, "block_table")
    c = config._c()
    if workspace is None:
        need = int(_native.lib().singe_hip_paged_kv_decode_attention_workspace_bytes(ctypes.byref(c)))
        workspace = _workspaces.get(out.device, need)
    status = _native.lib().singe_hip_paged_kv_decode_attention_f16(
        _stream_handle(stream), _ptr(out), out.numel(), _ptr(query), query.numel(), _ptr(key_cache), key_cache.numel(),
        _ptr(value_cache), value_cache.numel(), _ptr(actual_seq_lens), actual_seq_lens.numel(), _ptr(block_table),
        block_table.numel(), _ptr(workspace), workspace.numel() * workspace.element_size(), ctypes.byref(c))
    _native.check(status, "paged_kv_decode_attention_f16")


# ---- the rest of the dense family (fmha.rs:193-1036, paged.rs:36-116, 427-576) --------------------------------------

_ELEMENTS = {torch.float32: "f32", torch.bfloat16: "bf16", torch.float16: "f16"}


def _call_family(name: str, dtype: torch.dtype, stream, tensors, config_c) -> None:
    """Launches singe_hip_<name>_<element>(stream, (pointer, length) of every tensor in order, config)."""
    element = _ELEMENTS[dtype]
    arguments = []
    for tensor in tensors:
        arguments += [_ptr(tensor), tensor.numel()]
    status = getattr(_native.lib(), f"singe_hip_{name}_{element}")(_stream_handle(stream), *arguments, ctypes.byref(config_c))
    _native.check(status, f"{name}_{element}")


def _softcapped_window_attention(dtype, stream, out, query, key, value, config: SoftcappedWindowAttentionConfig) -> None:
    for tensor, name in ((out, "out"), (query, "query"), (key, "key"), (value, "value")):
        _require(tensor, dtype, name)
    c = _native.SoftcappedWindowAttentionConfigC(config.attention._c(), config.window_size, 1 if config.soft_cap is not None else 0,
                                                 config.soft_cap if config.soft_cap is not None else 0.0)
    _call_family("softcapped_window_attention", dtype, stream, (out, query, key, value), c)


def softcapped_window_attention_bf16(stream, out, query, key, value, config: SoftcappedWindowAttentionConfig) -> None:
    """softcapped_window_attention_bf16 (fmha.rs:345-393)."""
    _softcapped_window_attention(torch.bfloat16, stream, out, query, key, value, config)


def softcapped_window_attention_f16(stream, out, query, key, value, config: SoftcappedWindowAttentionConfig) -> None:
    """softcapped_window_attention_f16 (fmha.rs:295-343)."""
    _softcapped_window_attention(torch.float16, stream, out, query, key, value, config)


@dataclass(frozen=True)
class AttentionSinkPrefillConfig:
    """AttentionSinkPrefillConfig (mod.rs:299-304): prefill whose softmax also holds one sink logit per head; query q
    sits at position start_q + q; window w > 0 keeps the w keys up to that position."""
    attention: FmhaPrefillConfig
    start_q: int = 0
    window: int = 0

    @classmethod
    def contiguous(cls, batch, query_len, key_len, heads, kv_heads, head_dim, start_q, window, scale, causal):
        """mod.rs:1823-1841."""
        return cls(FmhaPrefillConfig.contiguous(batch, query_len, key_len, heads, kv_heads, head_dim, scale, causal), start_q, window)

    def _c(self):
        return _native.AttentionSinkPrefillConfigC(self.attention._c(), self.start_q, self.window)


def _attention_sink_prefill(dtype, stream, out, query, key, value, sinks, config: AttentionSinkPrefillConfig) -> None:
    for tensor, name in ((out, "out"), (query, "query"), (key, "key"), (value, "value"), (sinks, "sinks")):
        _require(tensor, dtype, name)
    _call_family("attention_sink_prefill", dtype, stream, (out, query, key, value, sinks), config._c())


def attention_sink_prefill_f32(stream, out, query, key, value, sinks, config: AttentionSinkPrefillConfig) -> None:
    """attention_sink_prefill_f32 (fmha.rs:193-243; CPU form cpu/attention.rs:2073-2155)."""
    _attention_sink_prefill(torch.float32, stream, out, query, key, value, sinks, config)


def attention_sink_prefill_bf16(stream, out, query, key, value, sinks, config: AttentionSinkPrefillConfig) -> None:
    """attention_sink_prefill_bf16 (fmha.rs:848-898)."""
    _attention_sink_prefill(torch.bfloat16, stream, out, query, key, value, sinks, config)


def attention_sink_prefill_f16(stream, out, query, key, value, sinks, config: AttentionSinkPrefillConfig) -> None:
    """attention_sink_prefill_f16 (fmha.rs:796-846)."""
    _attention_sink_prefill(torch.float16, stream, out, query, key, value, sinks, config)


def _fmha_decode_lse(dtype, stream, out, lse, query, key, value, config: FmhaDecodeConfig) -> None:
    for tensor, name in ((out, "out"), (query, "query"), (key, "key"), (value, "value")):
        _require(tensor, dtype, name)
    _require(lse, torch.float32, "lse")
    _call_family("fmha_decode_lse", dtype, stream, (out, lse, query, key, value), config._c())


def fmha_decode_lse_f32(stream, out, lse, query, key, value, config: FmhaDecodeConfig) -> None:
    """fmha_decode_lse_f32 (fmha.rs:395-438): one query per batch item, lse [batch, heads] natural log."""
    _fmha_decode_lse(torch.float32, stream, out, lse, query, key, value, config)


def fmha_decode_lse_bf16(stream, out, lse, query, key, value, config: FmhaDecodeConfig) -> None:
    """fmha_decode_lse_bf16 (fmha.rs:993-1036)."""
    _fmha_decode_lse(torch.bfloat16, stream, out, lse, query, key, value, config)


def fmha_decode_lse_f16(stream, out, lse, query, key, value, config: FmhaDecodeConfig) -> None:
    """fmha_decode_lse_f16 (fmha.rs:900-943)."""
    _fmha_decode_lse(torch.float16, stream, out, lse, query, key, value, config)


@dataclass(frozen=True)
class SoftcappedWindowDecodeConfig:
    """SoftcappedWindowDecodeConfig (mod.rs:307-311): decode whose query sits at position key_len - 1; window_size w > 0
    keeps the keys with key + w >= that position; optional tanh soft cap."""
    decode: FmhaDecodeConfig
    window_size: int = 0
    soft_cap: float | None = None

    @classmethod
    def bnsd_contiguous(cls, batch, key_len, heads, kv_heads, head_dim, scale, window_size, soft_cap):
        """mod.rs:2563-2602: key / value stored [batch, kv_heads, key_len, dim]."""
        key_head_stride = key_len * head_dim
        decode = FmhaDecodeConfig(batch, key_len, heads, kv_heads, head_dim, heads * head_dim, kv_heads * key_head_stride,
                                  kv_heads * key_head_stride, heads * head_dim, head_dim, head_dim, head_dim, head_dim,
                                  key_head_stride, key_head_stride, scale)
        return cls(decode, window_size, soft_cap)

    def _c(self):
        return _native.SoftcappedWindowDecodeConfigC(self.decode._c(), self.window_size, 1 if self.soft_cap is not None else 0,
                                                     self.soft_cap if self.soft_cap is not None else 0.0)


def _softcapped_window_decode_lse(dtype, stream, out, lse, query, key, value, config: SoftcappedWindowDecodeConfig) -> None:
    for tensor, name in ((out, "out"), (query, "query"), (key, "key"), (value, "value")):
        _require(tensor, dtype, name)
    _require(lse, torch.float32, "lse")
    _call_family("softcapped_window_decode_lse", dtype, stream, (out, lse, query, key, value), config._c())


def softcapped_window_decode_lse_f32(stream, out, lse, query, key, value, config: SoftcappedWindowDecodeConfig) -> None:
    """softcapped_window_decode_lse_f32 (fmha.rs:440-486; CPU form cpu/attention.rs:1927-1998)."""
    _softcapped_window_decode_lse(torch.float32, stream, out, lse, query, key, value, config)


def softcapped_window_decode_lse_bf16(stream, out, lse, query, key, value, config: SoftcappedWindowDecodeConfig) -> None:
    """softcapped_window_decode_lse_bf16 (fmha.rs:536-582)."""
    _softcapped_window_decode_lse(torch.bfloat16, stream, out, lse, query, key, value, config)


def softcapped_window_decode_lse_f16(stream, out, lse, query, key, value, config: SoftcappedWindowDecodeConfig) -> None:
    """softcapped_window_decode_lse_f16 (fmha.rs:488-534)."""
    _softcapped_window_decode_lse(torch.float16, stream, out, lse, query, key, value, config)


@dataclass(frozen=True)
class RaggedKvPrefillAttentionConfig:
    """RaggedKvPrefillAttentionConfig (mod.rs:110-123): query, key and value tokens packed by sequence; per-batch lengths
    and offsets describe each ragged segment."""
    batch: int
    total_query_tokens: int
    total_kv_tokens: int
    heads: int
    kv_heads: int
    head_dim: int
    causal: bool
    scale: float

    @classmethod
    def contiguous(cls, batch, total_query_tokens, total_kv_tokens, heads, kv_heads, head_dim, causal, scale):
        """mod.rs:821-842: builds the config and validates it (validate_ragged_kv_prefill_attention_config, mod.rs:3013-3035)."""
        config = cls(batch, total_query_tokens, total_kv_tokens, heads, kv_heads, head_dim, causal, scale)
        extents = (batch, total_query_tokens, total_kv_tokens, heads, kv_heads, head_dim)
        if any(e <= 0 for e in extents) or heads % kv_heads != 0 or not math.isfinite(scale):
            raise error.InvalidLength("invalid length")
        if any(e > I32_MAX for e in extents):
            raise error.LengthExceedsI32("length exceeds i32")
        return config

    def _c(self):
        return _native.RaggedKvPrefillAttentionConfigC(self.batch, self.total_query_tokens, self.total_kv_tokens, self.heads,
                                                       self.kv_heads, self.head_dim, 1 if self.causal else 0, self.scale)


def _ragged_kv_prefill_attention(dtype, stream, out, lse, query, key, value, lens_q, lens_kv, offsets,
                                 config: RaggedKvPrefillAttentionConfig) -> None:
    for tensor, name in ((out, "out"), (query, "query"), (key, "key"), (value, "value")):
        _require(tensor, dtype, name)
    _require(lse, torch.float32, "lse")
    for tensor, name in ((lens_q, "actual_seq_lens_q"), (lens_kv, "actual_seq_lens_kv"), (offsets, "actual_seq_offsets")):
        _require(tensor, torch.int32, name)
    _call_family("ragged_kv_prefill_attention", dtype, stream, (out, lse, query, key, value, lens_q, lens_kv, offsets), config._c())


def ragged_kv_prefill_attention_f32(stream, out, lse, query, key, value, actual_seq_lens_q, actual_seq_lens_kv, actual_seq_offsets,
                                    config: RaggedKvPrefillAttentionConfig) -> None:
    """ragged_kv_prefill_attention_f32 (paged.rs:427-477; CPU form cpu/attention.rs:1343-1420)."""
    _ragged_kv_prefill_attention(torch.float32, stream, out, lse, query, key, value, actual_seq_lens_q, actual_seq_lens_kv,
                                 actual_seq_offsets, config)


def ragged_kv_prefill_attention_bf16(stream, out, lse, query, key, value, actual_seq_lens_q, actual_seq_lens_kv, actual_seq_offsets,
                                     config: RaggedKvPrefillAttentionConfig) -> None:
    """ragged_kv_prefill_attention_bf16 (paged.rs:531-576)."""
    _ragged_kv_prefill_attention(torch.bfloat16, stream, out, lse, query, key, value, actual_seq_lens_q, actual_seq_lens_kv,
                                 actual_seq_offsets, config)


def ragged_kv_prefill_attention_f16(stream, out, lse, query, key, value, actual_seq_lens_q, actual_seq_lens_kv, actual_seq_offsets,
                                    config: RaggedKvPrefillAttentionConfig) -> None:
    """ragged_kv_prefill_attention_f16 (paged.rs:479-529)."""
    _ragged_kv_prefill_attention(torch.float16, stream, out, lse, query, key, value, actual_seq_lens_q, actual_seq_lens_kv,
                                 actual_seq_offsets, config)


@dataclass(frozen=True)
class SlidingWindowAttentionConfig:
    """SlidingWindowAttentionConfig (mod.rs:32-56): query q at position query_start + q, key k at key_start + k; a key is
    kept when its position is at most the query's and position + window is beyond it."""
    batch: int
    query_len: int
    key_len: int
    heads: int
    kv_heads: int
    head_dim: int
    query_start: int
    key_start: int
    window: int
    query_batch_stride: int
    key_batch_stride: int
    value_batch_stride: int
    output_batch_stride: int
    query_sequence_stride: int
    key_sequence_stride: int
    value_sequence_stride: int
    output_sequence_stride: int
    query_head_stride: int
    key_head_stride: int
    value_head_stride: int
    output_head_stride: int
    scale: float
    output_scale: float = 1.0

    @classmethod
    def contiguous(cls, batch, query_len, key_len, heads, kv_heads, head_dim, query_start, key_start, window, scale):
        """mod.rs:502-541: packed [batch, len, heads, dim] strides, output_scale 1."""
        q_features, kv_features = heads * head_dim, kv_heads * head_dim
        return cls(batch, query_len, key_len, heads, kv_heads, head_dim, query_start, key_start, window, query_len * q_features,
                   key_len * kv_features, key_len * kv_features, query_len * q_features, q_features, kv_features, kv_features,
                   q_features, head_dim, head_dim, head_dim, head_dim, scale, 1.0)

    def with_output_scale(self, output_scale: float) -> "SlidingWindowAttentionConfig":
        """mod.rs:543-547."""
        import dataclasses

        return dataclasses.replace(self, output_scale=output_scale)

    def _c(self):
        return _native.SlidingWindowAttentionConfigC(*(getattr(self, name) for name in _native._SLIDING_FIELDS), self.scale,
                                                     self.output_scale)


def sliding_window_attention_f32(stream, out, query, key, value, config: SlidingWindowAttentionConfig) -> None:
    """sliding_window_attention_f32 (mod.rs:2812-2855; CPU form cpu/attention.rs:1089-1170)."""
    for tensor, name in ((out, "out"), (query, "query"), (key, "key"), (value, "value")):
        _require(tensor, torch.float32, name)
    _call_family("sliding_window_attention", torch.float32, stream, (out, query, key, value), config._c())


@dataclass(frozen=True)
class PackedQkvAttentionConfig:
    """PackedQkvAttentionConfig (mod.rs:59-64): query, key and value are views of one buffer from these offsets on."""
    attention: SlidingWindowAttentionConfig
    query_offset: int
    key_offset: int
    value_offset: int


def sliding_window_attention_packed_qkv_f32(stream, out, qkv, config: PackedQkvAttentionConfig) -> None:
    """sliding_window_attention_packed_qkv_f32 (paged.rs:36-50)."""
    _require(out, torch.float32, "out")
    _require(qkv, torch.float32, "qkv")
    c = _native.PackedQkvAttentionConfigC(config.attention._c(), config.query_offset, config.key_offset, config.value_offset)
    status = _native.lib().singe_hip_sliding_window_attention_packed_qkv_f32(_stream_handle(stream), _ptr(out), out.numel(), _ptr(qkv),
                                                                             qkv.numel(), ctypes.byref(c))
    _native.check(status, "sliding_window_attention_packed_qkv_f32")


@dataclass(frozen=True)
class PagedKvAttentionConfig:
    """PagedKvAttentionConfig (mod.rs:67-74): the sliding-window attention's keys and values behind a block table."""
    attention: SlidingWindowAttentionConfig
    block_size: int
    physical_blocks: int
    block_table_batch_stride: int
    key_cache_block_stride: int
    value_cache_block_stride: int


def sliding_window_attention_paged_kv_f32(stream, out, query, key_cache, value_cache, block_table, config: PagedKvAttentionConfig) -> None:
    """sliding_window_attention_paged_kv_f32 (paged.rs:56-116)."""
    for tensor, name in ((out, "out"), (query, "query"), (key_cache, "key_cache"), (value_cache, "value_cache")):
        _require(tensor, torch.float32, name)
    if block_table.dtype not in (torch.int32, torch.uint32):
        raise error.InvalidArgument(f"block_table must hold 32-bit entries, got {block_table.dtype}")
    _require(block_table, block_table.dtype, "block_table")
    c = _native.PagedKvAttentionConfigC(config.attention._c(), config.block_size, config.physical_blocks,
                                        config.block_table_batch_stride, config.key_cache_block_stride, config.value_cache_block_stride)
    _call_family("sliding_window_attention_paged_kv", torch.float32, stream, (out, query, key_cache, value_cache, block_table), c)
