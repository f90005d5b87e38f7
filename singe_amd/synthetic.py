"""Seeded synthetic workloads of the shapes the benchmark configurations name.

Two sources of randomness.  The default draws integers (lengths, block tables, page lists) on the host with numpy's
PCG64 and float tensors N(0, 1) with a torch generator on the requested device: quick, what the tests use.
``portable=True`` takes everything from the library's counter stream instead (``csrc/synthetic_inputs.cpp``:
splitmix64 words, Box-Muller on two 24-bit uniforms in double, one stream per tensor with seed = base seed ^ FNV-1a of
the tensor's name), made on the host and rounded to the storage type on the device: the same tensors for any caller
that implements those few lines, whatever its language; what ``bench.py`` measures on.
"""
from __future__ import annotations

import ctypes
import os
from dataclasses import dataclass

import numpy as np
import torch

BASE_SEED = 0x51A6E
_CHUNK = 1 << 26  # elements of a host chunk (256 MiB of f32)


def _host_threads() -> int:
    return max(1, min(16, os.cpu_count() or 1))


class _TorchSource:
    """numpy PCG64 for integers, a torch generator on the device for normal values; draws are taken in call order."""

    def __init__(self, seed: int, device, name: str):
        self.rng = np.random.default_rng(seed)
        self.device = device
        self.gen = torch.Generator(device=device)
        self.gen.manual_seed(seed + 1)

    def integers(self, tensor: str, low: int, high: int, size: int) -> np.ndarray:
        return self.rng.integers(low, high + 1, size=size)

    def permutation(self, tensor: str, count: int) -> np.ndarray:
        return self.rng.permutation(count)

    def normal(self, tensor: str, shape, first_element: int = 0) -> torch.Tensor:
        return torch.randn(tuple(shape), generator=self.gen, device=self.device, dtype=torch.float32)


class _PortableSource:
    """The library's counter stream: tensor `t` of workload `name` is stream seed(base seed, "name.t")."""

    def __init__(self, seed: int, device, name: str):
        from . import _native
        self.lib = _native.lib()
        self.seed, self.device, self.name = seed, device, name
        self.staging = None

    def _stream(self, tensor: str) -> int:
        full = f"{self.name}.{tensor}" if tensor else self.name
        return int(self.lib.singe_hip_synthetic_seed(self.seed, full.encode()))

    def integers(self, tensor: str, low: int, high: int, size: int) -> np.ndarray:
        out = np.empty(size, dtype=np.int64)
        self.lib.singe_hip_synthetic_integers(self._stream(tensor), 0, low, high - low + 1, out.ctypes.data, size)
        return out

    def permutation(self, tensor: str, count: int) -> np.ndarray:
        out = np.empty(count, dtype=np.int64)
        self.lib.singe_hip_synthetic_permutation(self._stream(tensor), out.ctypes.data, count)
        return out

    def normal(self, tensor: str, shape, first_element: int = 0) -> torch.Tensor:
        """Elements first_element .. of the tensor's stream, as f32 on the device."""
        count = int(np.prod(shape))
        out = torch.empty(count, dtype=torch.float32, device=self.device)
        if self.staging is None:
            self.staging = torch.empty(min(_CHUNK, max(count, 1 << 20)), dtype=torch.float32, pin_memory=torch.cuda.is_available())
        stream = self._stream(tensor)
        for first in range(0, count, self.staging.numel()):
            n = min(self.staging.numel(), count - first)
            self.lib.singe_hip_synthetic_normal_f32(stream, first_element + first, self.staging.data_ptr(), n, _host_threads())
            out[first:first + n].copy_(self.staging[:n])  # synchronous: the staging buffer is rewritten next
        return out.view(tuple(shape))


def _source(portable: bool, seed: int, device, name: str):
    return (_PortableSource if portable else _TorchSource)(seed, device, name)


@dataclass
class PagedDecodeWorkload:
    """Paged decode, one query token per sequence (singe-kernel surface)."""
    batch: int
    heads: int
    kv_heads: int
    head_dim: int
    block_size: int
    physical_blocks: int
    block_table_batch_stride: int
    scale: float
    seq_lens: np.ndarray      # [batch] int32
    block_table: np.ndarray   # [batch, stride] uint32
    query: torch.Tensor       # [batch, heads, dim]
    key_cache: torch.Tensor   # [blocks, block_size, kv_heads, dim]
    value_cache: torch.Tensor

    @property
    def total_keys(self) -> int:
        return int(self.seq_lens.astype(np.int64).sum())

    def algorithmic_bytes(self, kv_element_bytes: int = 2) -> int:
        """Every operand element read or written once: valid KV rows, Q, O, the table entries used,
        the lengths."""
        kv = self.total_keys * 2 * self.kv_heads * self.head_dim * kv_element_bytes
        qo = 2 * self.batch * self.heads * self.head_dim * 2
        used = int(np.sum((self.seq_lens.astype(np.int64) + self.block_size - 1) // self.block_size))
        return kv + qo + used * 4 + self.batch * 4

    def algorithmic_flops(self) -> int:
        return 4 * self.heads * self.head_dim * self.total_keys


def paged_block_table(rng, seq_lens: np.ndarray, block_size: int, physical_blocks: int,
                      stride: int | None = None):
    """Consecutive slices of a seeded permutation of the block pool become the rows of the table;
    unused entries are zero."""
    counts = (seq_lens.astype(np.int64) + block_size - 1) // block_size
    if stride is None:
        stride = max(int(counts.max()), 1)
    if int(counts.sum()) > physical_blocks:
        raise ValueError("block pool too small")
    perm = rng.permutation(physical_blocks) if isinstance(rng, np.random.Generator) else rng.permutation("block_table", physical_blocks)
    table = np.zeros((len(seq_lens), stride), dtype=np.uint32)
    at = 0
    for b, n in enumerate(counts):
        table[b, :n] = perm[at:at + n]
        at += int(n)
    return table, stride


def paged_decode_workload(*, batch=32, heads=32, kv_heads=8, head_dim=128, block_size=16, physical_blocks=16384,
                          min_len=512, max_len=4096, seed=BASE_SEED, device="cuda", dtype=torch.bfloat16,
                          fill="all", seq_lens=None, portable=False, name="paged_decode") -> PagedDecodeWorkload:
    """batch sequences with context lengths uniform in [min_len, max_len], block tables drawn as a
    seeded permutation of the physical pool.  ``fill='used'`` only draws the referenced blocks (the
    rest stay zero), which is enough for parity tests on large pools."""
    source = _source(portable, seed, device, name)
    if seq_lens is None:
        seq_lens = source.integers("seq_lens", min_len, max_len, batch).astype(np.int32)
    else:
        seq_lens = np.asarray(seq_lens, dtype=np.int32)
    table, stride = paged_block_table(source.rng if not portable else source, seq_lens, block_size, physical_blocks)
    query = source.normal("query", (batch, heads, head_dim)).to(dtype)
    shape = (physical_blocks, block_size, kv_heads, head_dim)
    if fill == "all":
        key_cache = source.normal("key_cache", shape).to(dtype)
        value_cache = source.normal("value_cache", shape).to(dtype)
    else:
        key_cache = torch.zeros(shape, device=device, dtype=dtype)
        value_cache = torch.zeros(shape, device=device, dtype=dtype)
        counts = (seq_lens.astype(np.int64) + block_size - 1) // block_size
        used = np.concatenate([table[b, :n] for b, n in enumerate(counts)]).astype(np.int64)
        index = torch.from_numpy(used).to(device)
        sub = (len(used), block_size, kv_heads, head_dim)
        key_cache[index] = source.normal("key_cache", sub).to(dtype)
        value_cache[index] = source.normal("value_cache", sub).to(dtype)
    return PagedDecodeWorkload(batch, heads, kv_heads, head_dim, block_size, physical_blocks, stride,
                               float(1.0 / np.sqrt(np.float32(head_dim))), seq_lens, table, query, key_cache,
                               value_cache)


@dataclass
class PagedDecodeFp8Workload(PagedDecodeWorkload):
    """Paged decode over an fp8 e4m3 KV cache: key_cache/value_cache hold codes (uint8),
    key_scales/value_scales [blocks, kv_heads] f32 hold one scale per (block, kv head)."""
    key_scales: torch.Tensor = None
    value_scales: torch.Tensor = None


def quantize_fp8_blocks(values: torch.Tensor):
    """[blocks, block_size, kv_heads, dim] f32 -> (codes uint8, scales [blocks, kv_heads] f32) with
    scale = max |x| over the (block, kv head) tile / 448 and code = e4m3(x / scale), round to nearest
    even (torch's float8_e4m3fn cast, the conversion the reference's encode table is taken from:
    singe-codegen/src/interpret/tests.rs:274-312)."""
    peak = values.abs().amax(dim=(1, 3))
    scales = torch.where(peak > 0, peak / 448.0, torch.ones_like(peak)).to(torch.float32)
    codes = (values / scales[:, None, :, None]).to(torch.float8_e4m3fn).view(torch.uint8)
    return codes, scales


def paged_decode_fp8_workload(*, batch=64, heads=64, kv_heads=8, head_dim=128, block_size=16,
                              physical_blocks=131072, min_len=32768, max_len=32768, seed=BASE_SEED + 5,
                              device="cuda", seq_lens=None, chunk_blocks=8192, portable=False,
                              name="paged_decode_fp8") -> PagedDecodeFp8Workload:
    """Long-context decode with an fp8 KV cache (values ~ N(0, 1) before quantisation)."""
    source = _source(portable, seed, device, name)
    if seq_lens is None:
        seq_lens = source.integers("seq_lens", min_len, max_len, batch).astype(np.int32)
    else:
        seq_lens = np.asarray(seq_lens, dtype=np.int32)
    table, stride = paged_block_table(source.rng if not portable else source, seq_lens, block_size, physical_blocks)
    query = source.normal("query", (batch, heads, head_dim)).to(torch.bfloat16)
    shape = (physical_blocks, block_size, kv_heads, head_dim)
    block_elements = block_size * kv_heads * head_dim
    caches, scales = [], []
    for tensor in ("key_cache", "value_cache"):
        codes = torch.empty(shape, device=device, dtype=torch.uint8)
        scale = torch.empty((physical_blocks, kv_heads), device=device, dtype=torch.float32)
        for first in range(0, physical_blocks, chunk_blocks):
            count = min(chunk_blocks, physical_blocks - first)
            values = source.normal(tensor, (count, block_size, kv_heads, head_dim), first * block_elements)
            codes[first:first + count], scale[first:first + count] = quantize_fp8_blocks(values)
        caches.append(codes)
        scales.append(scale)
    return PagedDecodeFp8Workload(batch, heads, kv_heads, head_dim, block_size, physical_blocks, stride,
                                  float(1.0 / np.sqrt(np.float32(head_dim))), seq_lens, table, query, caches[0],
                                  caches[1], scales[0], scales[1])


@dataclass
class ChunkedPrefillWorkload:
    """Chunked paged prefill in FlashInfer form: each sequence appends `new_tokens` queries to a cached
    prefix (singe surface, bottom-right causal)."""
    sequences: int
    new_tokens: int
    heads: int
    kv_heads: int
    head_dim: int
    page_size: int
    prefix: np.ndarray             # [sequences] int64
    query_offsets: np.ndarray      # [sequences + 1]
    page_offsets: np.ndarray       # [sequences + 1]
    pages: np.ndarray              # [sum pages]
    last_page_lengths: np.ndarray  # [sequences]
    query: torch.Tensor            # [sequences * new_tokens, heads, dim]
    key_cache: torch.Tensor        # [pool, page_size, kv_heads, dim]
    value_cache: torch.Tensor

    def algorithmic_flops(self) -> int:
        """4 * dim flops per unmasked (query row, key) pair: a query at offset i of a chunk sees
        prefix + i + 1 keys."""
        new = self.new_tokens
        pairs = self.heads * sum(int(new * p + new * (new + 1) // 2) for p in self.prefix)
        return 4 * self.head_dim * pairs

    def algorithmic_bytes(self) -> int:
        """Every operand element once: the keys and values of prefix + new tokens per sequence, the queries, the
        outputs, one f32 log-sum-exp per (token, head), the paging vectors (i32)."""
        tokens = self.sequences * self.new_tokens
        keys = int(sum(int(p) + self.new_tokens for p in self.prefix))
        cache = 2 * keys * self.kv_heads * self.head_dim * 2
        rows = 2 * tokens * self.heads * self.head_dim * 2 + tokens * self.heads * 4
        paging = 4 * (len(self.query_offsets) + len(self.page_offsets) + len(self.pages) + len(self.last_page_lengths))
        return cache + rows + paging


def chunked_prefill_workload(*, sequences=8, new_tokens=512, heads=64, kv_heads=8, head_dim=128, page_size=16,
                             pool_pages=16384, min_prefix=1024, max_prefix=16384, seed=BASE_SEED + 4,
                             device="cuda", dtype=torch.bfloat16, portable=False,
                             name="chunked_prefill") -> ChunkedPrefillWorkload:
    source = _source(portable, seed, device, name)
    prefix = source.integers("prefix", min_prefix, max_prefix, sequences).astype(np.int64)
    keys = prefix + new_tokens
    counts = (keys + page_size - 1) // page_size
    if int(counts.sum()) > pool_pages:
        raise ValueError("page pool too small")
    pages = source.permutation("pages", pool_pages)[: int(counts.sum())].astype(np.int64)
    query_offsets = np.arange(sequences + 1, dtype=np.int64) * new_tokens
    page_offsets = np.concatenate([[0], np.cumsum(counts)]).astype(np.int64)
    last = keys - (counts - 1) * page_size
    query = source.normal("query", (sequences * new_tokens, heads, head_dim)).to(dtype)
    shape = (pool_pages, page_size, kv_heads, head_dim)
    key_cache = source.normal("key_cache", shape).to(dtype)
    value_cache = source.normal("value_cache", shape).to(dtype)
    return ChunkedPrefillWorkload(sequences, new_tokens, heads, kv_heads, head_dim, page_size, prefix, query_offsets,
                                  page_offsets, pages, last, query, key_cache, value_cache)


def portable_normal(name: str, shape, dtype=torch.float32, device="cuda", seed=BASE_SEED) -> torch.Tensor:
    """One N(0, 1) tensor from the counter stream seed(seed, name), rounded to `dtype` on the device."""
    return _PortableSource(seed, device, name).normal("", shape).to(dtype)
