"""Host-side mirror of the ``singe`` crate's attention ops on tensors
(singe/src/tensor/neural.rs:25-32, 409-457): ``AttentionOptions``, ``Paging`` and
``paged_attention``, which attends ragged queries over a paged key/value cache as FlashInfer batches
decode and prefill, and returns the output and each row's base-two log-sum-exp."""
from __future__ import annotations

import ctypes
from dataclasses import dataclass

import torch

from . import _native, error

STATUS_INDEX_OUT_OF_BOUNDS = 1  # singe/src/backend/kernel_lowering/mod.rs:40-61


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


def paged_attention(query: torch.Tensor, key_cache: torch.Tensor, value_cache: torch.Tensor, paging: Paging,
                    options: AttentionOptions = AttentionOptions(), *, stream=None, status: torch.Tensor | None = None,
                    check: bool = True):
    """Tensor::paged_attention (tensor/neural.rs:420-457) for bf16 tensors on the GPU.

    Returns (output [tokens, heads, dim] bf16, lse [tokens, heads] f32 base two).  Like the reference's
    eager launch (kernel_plan/mod.rs:156-251) it zeroes a status word, launches, and reads the word
    back: a paging value outside its buffers raises IndexOutOfBounds.  ``check=False`` skips the
    read-back (and the synchronisation it implies); pass ``status`` to inspect the word yourself.
    """
    for tensor, name in ((query, "query"), (key_cache, "key_cache"), (value_cache, "value_cache")):
        if not tensor.is_cuda or tensor.dtype != torch.bfloat16 or not tensor.is_contiguous():
            raise error.InvalidArgument(f"paged attention {name} must be a contiguous bf16 device tensor")
    for tensor in (paging.query_offsets, paging.page_offsets, paging.pages, paging.last_page_lengths):
        if not tensor.is_cuda or not tensor.is_contiguous():
            raise error.InvalidArgument("paged attention index tensors must be contiguous device tensors")
    problem = _problem(query, key_cache, value_cache, paging, options)
    output = torch.zeros_like(query)
    lse = torch.full(query.shape[:2], float("-inf"), device=query.device, dtype=torch.float32)
    if status is None:
        status = torch.zeros(1, device=query.device, dtype=torch.int32)
    handle = int((stream or torch.cuda.current_stream()).cuda_stream)
    code = _native.lib().singe_hip_paged_attention_bf16(
        handle, query.data_ptr(), key_cache.data_ptr(), value_cache.data_ptr(), paging.query_offsets.data_ptr(),
        paging.page_offsets.data_ptr(), paging.pages.data_ptr(), paging.last_page_lengths.data_ptr(),
        output.data_ptr(), lse.data_ptr(), status.data_ptr(), ctypes.byref(problem))
    _native.check(code, "paged_attention")
    if check and int(status.item()) == STATUS_INDEX_OUT_OF_BOUNDS:
        raise error.IndexOutOfBounds("paged attention paging value outside its buffers")
    return output, lse
