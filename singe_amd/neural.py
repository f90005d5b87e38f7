"""Host-side mirror of the ``singe`` crate's attention ops on tensors
(singe/src/tensor/neural.rs:25-32, 92-175, 409-457): ``AttentionOptions``, the dense
``scaled_dot_product_attention`` / ``attend`` / ``attend_padded``, and ``Paging`` with ``paged_attention``,
which attends ragged queries over a paged key/value cache as FlashInfer batches decode and prefill, and
returns the output and each row's base-two log-sum-exp."""
from __future__ import annotations

import ctypes
import functools
from dataclasses import dataclass

import torch

from . import _native, error

STATUS_INDEX_OUT_OF_BOUNDS = 1  # singe/src/backend/kernel_lowering/mod.rs:40-61


def _on_stream(op):
    """Runs ``op`` with its ``stream=`` argument as torch's current stream, so everything the op does besides its
    own launch (allocating and filling the outputs and the status word, converting a mask, reading the status
    word back) is ordered on the stream the kernel runs on, as the reference keeps one kernel stream per device
    for its launches and their buffers (kernel_plan/mod.rs:156-232)."""
    @functools.wraps(op)
    def ordered(*args, stream=None, **kwargs):
        if stream is None or stream == torch.cuda.current_stream(stream.device):
            return op(*args, stream=stream, **kwargs)
        with torch.cuda.stream(stream):
            return op(*args, stream=stream, **kwargs)
    return ordered


@dataclass(frozen=True)
class AttentionOptions:
    """How attention scores and masks keys (tensor/neural.rs:25-32): the scale, which defaults to
    1 / sqrt(head_dim), a causal mask, a sliding window of the keys each query sees up to itself, and a
    cap on the scaled scores."""
    scale: float | None = None
    causal: bool = False
    window: int | None = None
    softcap: float | None = None


@dataclass(frozen=True)
class Paging:
    """Where ragged queries and their keys sit in a paged cache (tensor/neural.rs:409-417): int32 or
    int64 vectors, all of one type."""
    query_offsets: torch.Tensor
    page_offsets: torch.Tensor
    pages: torch.Tensor
    last_page_lengths: torch.Tensor


def _problem(query, key_cache, value_cache, paging: Paging, options: AttentionOptions):
    """spec::paged_attention_problem (singe/src/backend/spec/neural/attention.rs:337-438)."""
    if query.dim() != 3 or key_cache.dim() != 4:
        raise error.InvalidArgument("paged attention query or cache rank")
    if key_cache.shape != value_cache.shape:
        raise error.InvalidArgument("paged attention value cache shape")
    tokens, heads, head_dim = query.shape
    cache_pages, page_size, kv_heads, key_dim = key_cache.shape
    if key_dim != head_dim or kv_heads <= 0 or heads % kv_heads != 0 or page_size <= 0:
        raise error.InvalidArgument("paged attention heads, head dimension, or page size")
    indices = (paging.query_offsets, paging.page_offsets, paging.pages, paging.last_page_lengths)
    kinds = {t.dtype for t in indices}
    if not kinds <= {torch.int32, torch.int64}:
        raise error.InvalidArgument("paged attention index type")
    if len(kinds) != 1:
        raise error.InvalidArgument("paged attention index tensors must share one type")
    if any(t.dim() != 1 for t in indices):
        raise error.InvalidArgument("paged attention index rank")
    sequences = paging.last_page_lengths.numel()
    if paging.query_offsets.numel() != sequences + 1 or paging.page_offsets.numel() != sequences + 1:
        raise error.InvalidArgument("paged attention offset count")
    return _native.PagedAttentionProblemC(
        tokens, heads, kv_heads, head_dim, page_size, sequences, cache_pages, paging.pages.numel(),
        1 if paging.pages.dtype == torch.int64 else 0, 1 if options.causal else 0,
        1 if options.scale is not None else 0, 1 if options.window is not None else 0,
        1 if options.softcap is not None else 0, options.scale if options.scale is not None else 0.0,
        options.softcap if options.softcap is not None else 0.0, options.window if options.window is not None else 0)


_DATA_TYPES = {torch.float32: _native.DATA_TYPE_F32, torch.bfloat16: _native.DATA_TYPE_BF16,
               torch.float16: _native.DATA_TYPE_F16}
# The dense op and the paged op also take f64 (on the vector-unit kernels, in f64 arithmetic).
_ATTENTION_TYPES = {**_DATA_TYPES, torch.float64: _native.DATA_TYPE_F64}


def scaled_dot_product_attention(query, key, value, scale: float | None = None, causal: bool = False, *, stream=None):
    """Tensor::scaled_dot_product_attention (tensor/neural.rs:92-110)."""
    return _attend_all(query, key, value, None, None, None, AttentionOptions(scale=scale, causal=causal), stream)


def attend(query, key, value, mask=None, sinks=None, options: AttentionOptions = AttentionOptions(), *, stream=None):
    """Tensor::attend (tensor/neural.rs:112-124): a ``mask`` broadcast to the scores' [B, H, L, S] adds to
    them after any cap (a Boolean mask lets the keys where it holds take part and hides the others);
    ``sinks``, one logit per query head, join each row's softmax without weighing a value."""
    return _attend_all(query, key, value, mask, sinks, None, options, stream)


def attend_padded(query, key, value, key_lengths, options: AttentionOptions = AttentionOptions(), *, stream=None):
    """Tensor::attend_padded (tensor/neural.rs:126-137): batch b attends to its first key_lengths[b] keys
    ([B] int32); a batch of no keys gives zeros."""
    return _attend_all(query, key, value, None, None, key_lengths, options, stream)


def _attend_all(query, key, value, mask, sinks, key_lengths, options, stream):
    return _attend_all_ordered(query, key, value, mask, sinks, key_lengths, options, stream=stream)


@_on_stream
def _attend_all_ordered(query, key, value, mask, sinks, key_lengths, options, *, stream=None):
    """attend_all (tensor/neural.rs:139-175) with the shape rules of spec::attention_problem
    (singe/src/backend/spec/neural/attention.rs:209-290)."""
    for tensor, name in ((query, "query"), (key, "key"), (value, "value")):
        if tensor.dim() != 4:
            raise error.InvalidArgument(f"scaled dot-product attention {name} rank")
        if not tensor.is_cuda or tensor.dtype != query.dtype or not tensor.is_contiguous():
            raise error.InvalidArgument(f"scaled dot-product attention {name} must be a contiguous device tensor of the query's type")
    if query.dtype not in _ATTENTION_TYPES:
        raise error.InvalidArgument(f"scaled dot-product attention data type {query.dtype}")
    batch, heads, query_len, head_dim = query.shape
    key_batch, kv_heads, key_len, key_dim = key.shape
    value_batch, value_heads, value_len, value_dim = value.shape
    if head_dim <= 0 or key_len <= 0:
        raise error.InvalidArgument("scaled dot-product attention head dimension and key length must be positive")
    if batch != key_batch or batch != value_batch:
        raise error.LengthMismatch("scaled dot-product attention batch")
    if kv_heads == 0 or heads % kv_heads != 0:
        raise error.InvalidArgument("scaled dot-product attention key heads must divide the query heads")
    if kv_heads != value_heads or head_dim != key_dim or key_len != value_len:
        raise error.LengthMismatch("scaled dot-product attention key and value shapes")
    strides = [0, 0, 0, 0]
    if mask is not None:
        if mask.dtype == torch.bool:
            mask = torch.where(mask, 0.0, float("-inf")).to(query.dtype)
        else:
            mask = mask.to(query.dtype)
        if mask.dim() > 4:
            raise error.InvalidArgument("scaled dot-product attention mask rank")
        shape = (1,) * (4 - mask.dim()) + tuple(mask.shape)
        target = (batch, heads, query_len, key_len)
        if any(have not in (1, want) for have, want in zip(shape, target)):
            raise error.InvalidArgument("scaled dot-product attention mask does not broadcast to the scores")
        mask = mask.contiguous().reshape(shape)
        strides = [0 if have == 1 else stride for have, stride in zip(shape, mask.stride())]
    if sinks is not None:
        if sinks.numel() != heads:
            raise error.InvalidArgument("scaled dot-product attention sinks must hold one logit per query head")
        sinks = sinks.to(query.dtype).contiguous()
    if key_lengths is not None:
        if key_lengths.dtype != torch.int32 or key_lengths.numel() != batch:
            raise error.InvalidArgument("scaled dot-product attention key lengths must be [batch] int32")
        key_lengths = key_lengths.contiguous()
    problem = _native.AttentionProblemC(
        batch, heads, kv_heads, query_len, key_len, head_dim, value_dim, (ctypes.c_int64 * 4)(*strides),
        _ATTENTION_TYPES[query.dtype], 1 if options.causal else 0, 1 if options.scale is not None else 0,
        1 if options.window is not None else 0, 1 if options.softcap is not None else 0,
        options.scale if options.scale is not None else 0.0, options.softcap if options.softcap is not None else 0.0,
        options.window if options.window is not None else 0)
    output = torch.empty((batch, heads, query_len, value_dim), device=query.device, dtype=query.dtype)
    handle = int((stream or torch.cuda.current_stream()).cuda_stream)
    pointer = lambda tensor: tensor.data_ptr() if tensor is not None else None
    # A decode-shaped call (few query rows, many keys) shares its keys out over several workgroups, on this module's
    # per-device scratch (calls on different streams must then not overlap), as the reference's plan splits them
    # (kernel_plan/source/attention.rs:283-292).
    wanted = int(_native.lib().singe_hip_scaled_dot_product_attention_scratch_bytes(ctypes.byref(problem)))
    if wanted > 0:
        lent = _scratch_for(query.device, wanted)
        code = _native.lib().singe_hip_scaled_dot_product_attention_scratch(
            handle, query.data_ptr(), key.data_ptr(), value.data_ptr(), pointer(mask), pointer(sinks), pointer(key_lengths),
            output.data_ptr(), lent.data_ptr(), lent.numel(), ctypes.byref(problem))
    else:
        code = _native.lib().singe_hip_scaled_dot_product_attention(
            handle, query.data_ptr(), key.data_ptr(), value.data_ptr(), pointer(mask), pointer(sinks), pointer(key_lengths),
            output.data_ptr(), ctypes.byref(problem))
    _native.check(code, "scaled_dot_product_attention")
    return output


@dataclass(frozen=True)
class AttentionParameters:
    """The choices the attention kernels leave open (singe/src/backend/cuda/kernel_plan/source/parameters.rs:21-57).
    On gfx950 `warps` is 4 and `key_tile` 64, `stages` 1 or 2 name the one pipeline the kernels have, `min_blocks` is
    None or 2, and `split_below_blocks` is the number of workgroups below which a launch splits its keys (0 never)."""
    warps: int = 4
    key_tile: int = 64
    stages: int = 1
    split_below_blocks: int = 64
    min_blocks: int | None = None

    def _c(self) -> _native.AttentionParametersC:
        return _native.AttentionParametersC(self.warps, self.key_tile, self.stages, self.split_below_blocks,
                                            0 if self.min_blocks is None else 1, self.min_blocks or 0)

    @classmethod
    def _of(cls, raw: _native.AttentionParametersC) -> "AttentionParameters":
        return cls(raw.warps, raw.key_tile, raw.stages, raw.split_below_blocks, raw.min_blocks if raw.has_min_blocks else None)


def default_attention_parameters() -> AttentionParameters:
    """AttentionParameters::default() of this device: split_below_blocks is twice its compute units."""
    raw = _native.AttentionParametersC()
    _native.lib().singe_hip_attention_parameters_default(ctypes.byref(raw))
    return AttentionParameters._of(raw)


def attention_candidates() -> list:
    """attention_candidates (kernel_plan/source/attention.rs:113-160): what the kernels take, the default first."""
    raw = (_native.AttentionParametersC * 16)()
    count = ctypes.c_size_t(0)
    _native.check(_native.lib().singe_hip_attention_candidates(raw, 16, ctypes.byref(count)), "attention_candidates")
    return [AttentionParameters._of(raw[i]) for i in range(min(count.value, 16))]


def set_attention_parameters(parameters: AttentionParameters | None) -> None:
    """Installs the parameters a tuning record gives the paged and the dense op (None: the default); parameters the
    kernels do not take raise StaleRecord, as the reference refuses them (parameters.rs:245-250)."""
    code = _native.lib().singe_hip_set_attention_parameters(None if parameters is None else ctypes.byref(parameters._c()))
    _native.check(code, "attention parameters")


def attention_parameters() -> AttentionParameters:
    raw = _native.AttentionParametersC()
    _native.lib().singe_hip_attention_parameters(ctypes.byref(raw))
    return AttentionParameters._of(raw)


def paged_attention_parameter_key(query, key_cache, value_cache, paging: Paging, options: AttentionOptions = AttentionOptions()) -> str:
    """parameter_key("paged_attention", ...) (parameters.rs:221-230) of contiguous operands."""
    problem = _problem(query, key_cache, value_cache, paging, options)
    need = int(_native.lib().singe_hip_paged_attention_parameter_key(ctypes.byref(problem), _ATTENTION_TYPES[query.dtype], None, 0))
    buffer = ctypes.create_string_buffer(need + 1)
    _native.lib().singe_hip_paged_attention_parameter_key(ctypes.byref(problem), _ATTENTION_TYPES[query.dtype], buffer, need + 1)
    return buffer.value.decode()


_scratch: dict = {}


def _scratch_for(device, nbytes: int) -> torch.Tensor:
    """A per-device buffer that grows to the largest request (the launch scratch a runtime would own)."""
    held = _scratch.get(device)
    if held is None or held.numel() < nbytes:
        held = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=device)
        _scratch[device] = held
    return held


@_on_stream
def paged_attention(query: torch.Tensor, key_cache: torch.Tensor, value_cache: torch.Tensor, paging: Paging,
                    options: AttentionOptions = AttentionOptions(), *, stream=None, status: torch.Tensor | None = None,
                    check: bool = True, scratch: "torch.Tensor | bool" = True):
    """Tensor::paged_attention (tensor/neural.rs:420-457) for bf16, f16 or f32 tensors on the GPU; bf16 at
    head dimensions 128 and 64 runs on the matrix cores, everything else on the general kernel.

    Returns (output [tokens, heads, dim] of the query's type, lse [tokens, heads] f32 base two).  Like the reference's
    eager launch (kernel_plan/mod.rs:156-251) it zeroes a status word, launches, and reads the word
    back: a paging value outside its buffers raises IndexOutOfBounds.  ``check=False`` skips the
    read-back (and the synchronisation it implies); pass ``status`` to inspect the word yourself.
    """
    for tensor, name in ((query, "query"), (key_cache, "key_cache"), (value_cache, "value_cache")):
        if not tensor.is_cuda or tensor.dtype != query.dtype or not tensor.is_contiguous():
            raise error.InvalidArgument(f"paged attention {name} must be a contiguous device tensor of the query's type")
    if query.dtype not in _ATTENTION_TYPES:
        raise error.InvalidArgument(f"paged attention data type {query.dtype}")
    for tensor in (paging.query_offsets, paging.page_offsets, paging.pages, paging.last_page_lengths):
        if not tensor.is_cuda or not tensor.is_contiguous():
            raise error.InvalidArgument("paged attention index tensors must be contiguous device tensors")
    problem = _problem(query, key_cache, value_cache, paging, options)
    output = torch.zeros_like(query)
    lse = torch.full(query.shape[:2], float("-inf"), device=query.device, dtype=torch.float32)
    if status is None:
        status = torch.zeros(1, device=query.device, dtype=torch.int32)
    handle = int((stream or torch.cuda.current_stream()).cuda_stream)
    entry = {torch.bfloat16: _native.lib().singe_hip_paged_attention_bf16,
             torch.float32: _native.lib().singe_hip_paged_attention_f32,
             torch.float64: _native.lib().singe_hip_paged_attention_f64,
             torch.float16: _native.lib().singe_hip_paged_attention_f16}[query.dtype]
    # bf16 calls with few query rows (decoding) share a row tile's keys out over several workgroups, given
    # scratch: ``scratch`` is a uint8 device tensor, True for this module's own per-device buffer (calls on
    # different streams must then not overlap), or False for none.
    wanted = 0
    if query.dtype in (torch.bfloat16, torch.float16) and scratch is not False:
        wanted = int(_native.lib().singe_hip_paged_attention_scratch_bytes(ctypes.byref(problem)))
    if wanted > 0:
        lent = _scratch_for(query.device, wanted) if scratch is True else scratch
        with_scratch = (_native.lib().singe_hip_paged_attention_scratch_bf16 if query.dtype == torch.bfloat16
                        else _native.lib().singe_hip_paged_attention_scratch_f16)
        code = with_scratch(
            handle, query.data_ptr(), key_cache.data_ptr(), value_cache.data_ptr(), paging.query_offsets.data_ptr(),
            paging.page_offsets.data_ptr(), paging.pages.data_ptr(), paging.last_page_lengths.data_ptr(),
            output.data_ptr(), lse.data_ptr(), status.data_ptr(), lent.data_ptr(), lent.numel(), ctypes.byref(problem))
    else:
        code = entry(
            handle, query.data_ptr(), key_cache.data_ptr(), value_cache.data_ptr(), paging.query_offsets.data_ptr(),
            paging.page_offsets.data_ptr(), paging.pages.data_ptr(), paging.last_page_lengths.data_ptr(),
            output.data_ptr(), lse.data_ptr(), status.data_ptr(), ctypes.byref(problem))
    _native.check(code, "paged_attention")
    if check and int(status.item()) == STATUS_INDEX_OUT_OF_BOUNDS:
        raise error.IndexOutOfBounds("paged attention paging value outside its buffers")
    return output, lse


@_on_stream
def paged_mla_attention(query: torch.Tensor, query_positions: torch.Tensor, latent_cache: torch.Tensor,
                        position_cache: torch.Tensor, paging: Paging, options: AttentionOptions = AttentionOptions(), *,
                        stream=None, status: torch.Tensor | None = None, check: bool = True,
                        scratch: "torch.Tensor | bool" = True):
    """Tensor::paged_mla_attention (singe/src/backend/spec/neural/attention.rs:453-497, CPU
    normalization/attention.rs:540-679): latent attention over paged caches.  ``query`` [tokens, heads, latent],
    ``query_positions`` [tokens, heads, positional], ``latent_cache`` [pages, page_size, latent], ``position_cache``
    [pages, page_size, positional], f32 / bf16 / f16.  Only ``causal`` and ``scale`` of the options apply.  Returns
    (output [tokens, heads, latent] of the query's type, lse [tokens, heads] f32 base two).  ``scratch`` as for
    paged_attention: with few rows (decoding) the matrix-core kernel shares a row tile's keys out over several
    workgroups, given a uint8 device tensor, or True for this module's own per-device buffer; False for none."""
    if options.window is not None or options.softcap is not None:
        raise error.InvalidArgument("paged mla attention takes a scale and a causal mask only")
    operands = ((query, "query"), (query_positions, "query_positions"), (latent_cache, "latent_cache"), (position_cache, "position_cache"))
    for tensor, name in operands:
        if not tensor.is_cuda or tensor.dtype != query.dtype or not tensor.is_contiguous() or tensor.dim() != 3:
            raise error.InvalidArgument(f"paged mla attention {name} must be a contiguous rank-3 device tensor of the query's type")
    if query.dtype not in _DATA_TYPES:
        raise error.InvalidArgument(f"paged mla attention data type {query.dtype}")
    tokens, heads, latent = query.shape
    pages, page_size, cached_latent = latent_cache.shape
    positional = query_positions.shape[2]
    if (tuple(query_positions.shape[:2]) != (tokens, heads) or tuple(position_cache.shape[:2]) != (pages, page_size)
            or cached_latent != latent or position_cache.shape[2] != positional or page_size <= 0 or latent <= 0):
        raise error.InvalidArgument("paged mla attention query or cache shapes")
    indices = (paging.query_offsets, paging.page_offsets, paging.pages, paging.last_page_lengths)
    kinds = {t.dtype for t in indices}
    if len(kinds) != 1 or not kinds <= {torch.int32, torch.int64}:
        raise error.InvalidArgument("paging index tensors must share one integer type")
    for tensor in indices:
        if not tensor.is_cuda or not tensor.is_contiguous():
            raise error.InvalidArgument("paged attention index tensors must be contiguous device tensors")
    sequences = paging.last_page_lengths.numel()
    if paging.query_offsets.numel() != sequences + 1 or paging.page_offsets.numel() != sequences + 1:
        raise error.InvalidArgument("paging offsets must hold one more entry than there are sequences")
    problem = _native.PagedMlaAttentionProblemC(
        tokens, heads, latent, positional, page_size, sequences, pages, paging.pages.numel(), _DATA_TYPES[query.dtype],
        1 if paging.pages.dtype == torch.int64 else 0, 1 if options.causal else 0, 1 if options.scale is not None else 0,
        options.scale if options.scale is not None else 0.0)
    output = torch.zeros_like(query)
    lse = torch.full((tokens, heads), float("-inf"), device=query.device, dtype=torch.float32)
    if status is None:
        status = torch.zeros(1, device=query.device, dtype=torch.int32)
    handle = int((stream or torch.cuda.current_stream()).cuda_stream)
    wanted = 0 if scratch is False else int(_native.lib().singe_hip_paged_mla_attention_scratch_bytes(ctypes.byref(problem)))
    if wanted > 0:
        lent = _scratch_for(query.device, wanted) if scratch is True else scratch
        code = _native.lib().singe_hip_paged_mla_attention_scratch(
            handle, query.data_ptr(), query_positions.data_ptr(), latent_cache.data_ptr(), position_cache.data_ptr(),
            paging.query_offsets.data_ptr(), paging.page_offsets.data_ptr(), paging.pages.data_ptr(), paging.last_page_lengths.data_ptr(),
            output.data_ptr(), lse.data_ptr(), status.data_ptr(), lent.data_ptr(), lent.numel(), ctypes.byref(problem))
    else:
        code = _native.lib().singe_hip_paged_mla_attention(
            handle, query.data_ptr(), query_positions.data_ptr(), latent_cache.data_ptr(), position_cache.data_ptr(),
            paging.query_offsets.data_ptr(), paging.page_offsets.data_ptr(), paging.pages.data_ptr(), paging.last_page_lengths.data_ptr(),
            output.data_ptr(), lse.data_ptr(), status.data_ptr(), ctypes.byref(problem))
    _native.check(code, "paged_mla_attention")
    if check and int(status.item()) == STATUS_INDEX_OUT_OF_BOUNDS:
        raise error.IndexOutOfBounds("paged mla attention paging value outside its buffers")
    return output, lse


@_on_stream
def rotary_paged_attention(query: torch.Tensor, key_cache: torch.Tensor, value_cache: torch.Tensor, paging: Paging,
                           cos: torch.Tensor, sin: torch.Tensor, options: AttentionOptions = AttentionOptions(), *,
                           query_norm: "RotationNorm | None" = None, stream=None, status: torch.Tensor | None = None,
                           check: bool = True):
    """Paged attention over a query the kernel normalises and rotates itself, the reference's fused
    rotary_paged_attention (singe/src/backend/cuda/kernel_plan/source/paged_attention.rs:533-542, 881-977):
    ``query`` [tokens, heads, D] bf16 or f16 (D a multiple of 16 up to 128, the set the reference fuses:
    paged_attention.rs:512-531) before its rotation, ``cos`` / ``sin`` [tokens, 1, D / 2] (or [tokens, D / 2]) of
    f32, bf16 or f16, the same pairs and norm as ``rotary_cache_write``; a softcap and a window are taken.  Returns
    (output, lse) like ``paged_attention``.  Other types and head dimensions raise UnsupportedWidth: rotate with
    ``rotary_cache_write`` and attend with ``paged_attention``, as the reference plans them apart."""
    for tensor, name in ((query, "query"), (key_cache, "key_cache"), (value_cache, "value_cache")):
        if not tensor.is_cuda or tensor.dtype != query.dtype or not tensor.is_contiguous():
            raise error.InvalidArgument(f"paged attention {name} must be a contiguous device tensor of the query's type")
    if query.dtype not in (torch.bfloat16, torch.float16):
        raise error.UnsupportedWidth("rotary_paged_attention (bf16 or f16 tensors)", 8 * query.element_size())
    for tensor in (paging.query_offsets, paging.page_offsets, paging.pages, paging.last_page_lengths):
        if not tensor.is_cuda or not tensor.is_contiguous():
            raise error.InvalidArgument("paged attention index tensors must be contiguous device tensors")
    if cos.dtype not in _DATA_TYPES or sin.dtype != cos.dtype or not cos.is_cuda or not sin.is_cuda:
        raise error.InvalidArgument("rotary paged attention angle tables")
    cos, sin = cos.contiguous(), sin.contiguous()
    tokens, _, head_dim = query.shape
    if cos.numel() != tokens * (head_dim // 2) or sin.numel() != cos.numel():
        raise error.InvalidArgument("rotary paged attention angles must be [tokens, 1, head_dim / 2]")
    weight = None if query_norm is None or query_norm.weight is None else query_norm.weight.to(query.dtype).contiguous()
    if weight is not None and weight.numel() != head_dim:
        raise error.InvalidArgument("rotary paged attention norm weight must hold head_dim values")
    problem = _problem(query, key_cache, value_cache, paging, options)
    rotation = _native.QueryRotationC(_DATA_TYPES[cos.dtype], 1 if query_norm is not None else 0,
                                      query_norm.eps if query_norm is not None else 0.0)
    output = torch.zeros_like(query)
    lse = torch.full(query.shape[:2], float("-inf"), device=query.device, dtype=torch.float32)
    if status is None:
        status = torch.zeros(1, device=query.device, dtype=torch.int32)
    handle = int((stream or torch.cuda.current_stream()).cuda_stream)
    entry = _native.lib().singe_hip_rotary_paged_attention_bf16 if query.dtype == torch.bfloat16 else _native.lib().singe_hip_rotary_paged_attention_f16
    code = entry(
        handle, query.data_ptr(), key_cache.data_ptr(), value_cache.data_ptr(), paging.query_offsets.data_ptr(),
        paging.page_offsets.data_ptr(), paging.pages.data_ptr(), paging.last_page_lengths.data_ptr(), cos.data_ptr(), sin.data_ptr(),
        None if weight is None else weight.data_ptr(), output.data_ptr(), lse.data_ptr(), status.data_ptr(), ctypes.byref(problem),
        ctypes.byref(rotation))
    _native.check(code, "rotary_paged_attention")
    if check and int(status.item()) == STATUS_INDEX_OUT_OF_BOUNDS:
        raise error.IndexOutOfBounds("paged attention paging value outside its buffers")
    return output, lse


@dataclass(frozen=True)
class RotationNorm:
    """The RMS normalisation a rotation applies first (rotary_cache.rs:25-30)."""
    eps: float
    weight: torch.Tensor | None = None


@_on_stream
def rotary_cache_write(query, key, value, cos, sin, pages, slots, key_cache, value_cache, *,
                       query_norm: RotationNorm | None = None, key_norm: RotationNorm | None = None, stream=None,
                       status: torch.Tensor | None = None, check: bool = True):
    """The step before paged attention in a decode layer, as one kernel
    (singe/src/backend/cuda/kernel_plan/source/rotary_cache.rs:249-427): rotates ``query`` [T, H, D] (or None)
    and ``key`` [T, G, D] by the angles ``cos`` / ``sin`` [T, D/2] (half-split pairs), and writes the rotated
    keys and ``value`` [T, G, D] into the caches [P, S, G, D] at (pages[t], slots[t]), in place.  Returns the
    rotated queries (None without a query).  A page or slot outside the cache raises IndexOutOfBounds."""
    tensors = [(key, "key"), (value, "value"), (key_cache, "key_cache"), (value_cache, "value_cache")]
    if query is not None:
        tensors.append((query, "query"))
    for tensor, name in tensors:
        if not tensor.is_cuda or tensor.dtype != key.dtype or not tensor.is_contiguous():
            raise error.InvalidArgument(f"rotary cache {name} must be a contiguous device tensor of the key's type")
    if key.dtype not in _DATA_TYPES or cos.dtype not in _DATA_TYPES or sin.dtype != cos.dtype:
        raise error.InvalidArgument("rotary cache data type")
    tokens, cache_heads, head_dim = key.shape
    if value.shape != key.shape or key_cache.shape != value_cache.shape or key_cache.dim() != 4:
        raise error.InvalidArgument("rotary cache value or cache shape")
    cache_pages, page_slots = key_cache.shape[:2]
    if tuple(key_cache.shape[2:]) != (cache_heads, head_dim):
        raise error.InvalidArgument("rotary cache heads or head dimension")
    cos, sin = cos.contiguous(), sin.contiguous()
    if cos.numel() != tokens * (head_dim // 2) or sin.numel() != cos.numel():
        raise error.InvalidArgument("rotary cache angles must be [tokens, 1, head_dim / 2]")
    if pages.dtype != slots.dtype or pages.dtype not in (torch.int32, torch.int64) or pages.numel() != tokens or slots.numel() != tokens:
        raise error.InvalidArgument("rotary cache pages and slots must be [tokens] of one integer type")
    query_heads = 0 if query is None else query.shape[1]
    query_out = None if query is None else torch.empty_like(query)
    weights = []
    for norm in (query_norm, key_norm):
        weight = None if norm is None or norm.weight is None else norm.weight.to(key.dtype).contiguous()
        if weight is not None and weight.numel() != head_dim:
            raise error.InvalidArgument("rotary cache norm weight must hold head_dim values")
        weights.append(weight)
    problem = _native.RotaryCacheProblemC(
        tokens, query_heads, cache_heads, head_dim, cache_pages, page_slots, _DATA_TYPES[key.dtype], _DATA_TYPES[cos.dtype],
        1 if pages.dtype == torch.int64 else 0, 1 if query_norm is not None else 0, 1 if key_norm is not None else 0,
        query_norm.eps if query_norm is not None else 0.0, key_norm.eps if key_norm is not None else 0.0)
    if status is None:
        status = torch.zeros(1, device=key.device, dtype=torch.int32)
    pointer = lambda tensor: tensor.data_ptr() if tensor is not None else None
    handle = int((stream or torch.cuda.current_stream()).cuda_stream)
    code = _native.lib().singe_hip_rotary_cache_write(
        handle, pointer(query), key.data_ptr(), value.data_ptr(), cos.data_ptr(), sin.data_ptr(), pages.contiguous().data_ptr(),
        slots.contiguous().data_ptr(), pointer(weights[0]), pointer(weights[1]), pointer(query_out), key_cache.data_ptr(),
        value_cache.data_ptr(), status.data_ptr(), ctypes.byref(problem))
    _native.check(code, "rotary_cache_write")
    if check and int(status.item()) == STATUS_INDEX_OUT_OF_BOUNDS:
        raise error.IndexOutOfBounds("rotary cache page or slot outside the cache")
    return query_out


@_on_stream
def paging_indices(paging: Paging, *, tokens: int, page_size: int, cache_pages: int, width: int, row_elements: int,
                   stream=None, status: torch.Tensor | None = None, check: bool = True):
    """FlashInfer CSR paging -> block-table paging, on the device
    (singe/src/backend/cuda/kernel_plan/source/paged_attention.rs:325-398).  Returns int32 tensors
    (packed_offsets [sequences + 1], query_lengths [sequences], key_lengths [sequences],
    page_table [sequences, width])."""
    indices = (paging.query_offsets, paging.page_offsets, paging.pages, paging.last_page_lengths)
    kinds = {t.dtype for t in indices}
    if len(kinds) != 1 or not kinds <= {torch.int32, torch.int64}:
        raise error.InvalidArgument("paging index tensors must share one integer type")
    sequences = paging.last_page_lengths.numel()
    device = paging.pages.device
    packed = torch.zeros(sequences + 1, device=device, dtype=torch.int32)
    query_lengths = torch.zeros(sequences, device=device, dtype=torch.int32)
    key_lengths = torch.zeros(sequences, device=device, dtype=torch.int32)
    table = torch.zeros((sequences, width), device=device, dtype=torch.int32)
    if status is None:
        status = torch.zeros(1, device=device, dtype=torch.int32)
    problem = _native.PagingIndicesProblemC(sequences, tokens, paging.pages.numel(), page_size, cache_pages, width, row_elements,
                                            1 if paging.pages.dtype == torch.int64 else 0)
    handle = int((stream or torch.cuda.current_stream()).cuda_stream)
    code = _native.lib().singe_hip_paging_indices(
        handle, paging.query_offsets.data_ptr(), paging.page_offsets.data_ptr(), paging.pages.data_ptr(),
        paging.last_page_lengths.data_ptr(), packed.data_ptr(), query_lengths.data_ptr(), key_lengths.data_ptr(), table.data_ptr(),
        status.data_ptr(), ctypes.byref(problem))
    _native.check(code, "paging_indices")
    if check and int(status.item()) == STATUS_INDEX_OUT_OF_BOUNDS:
        raise error.IndexOutOfBounds("paging value outside its buffers")
    return packed, query_lengths, key_lengths, table
