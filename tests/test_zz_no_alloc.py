"""The decode entry point that allocates nothing (singe_hip_paged_kv_decode_attention_no_alloc_bf16) against the
entry point it is a variant of (singe_hip_paged_kv_decode_attention_bf16), through the C ABI.  Both run the same
kernels with the same work split, so the outputs must agree bit for bit; they are also held to the oracle at the
bf16 tolerance (max-abs 2e-2, mean-abs 2e-3).  Two calls in a row share the library's fixed scratch, the second on a
smaller input, so anything the first call left behind would show."""
import ctypes

import numpy as np
import pytest
import torch

import oracle
from singe_amd import _native, error, synthetic
from singe_amd.kernel import attention as A

pytestmark = pytest.mark.gpu


def _config(work):
    return A.PagedKvDecodeAttentionConfig.contiguous(work.batch, work.heads, work.kv_heads, work.head_dim, work.block_size,
                                                     work.physical_blocks, work.block_table_batch_stride, work.scale)


def _both(work):
    config = _config(work)
    lens = torch.from_numpy(work.seq_lens).cuda()
    table = torch.from_numpy(work.block_table.view(np.int32)).cuda()
    shape = (work.batch, work.heads, work.head_dim)
    want = torch.full(shape, float("nan"), device="cuda", dtype=torch.bfloat16)
    got = torch.full(shape, float("nan"), device="cuda", dtype=torch.bfloat16)
    A.paged_kv_decode_attention_bf16(None, want, work.query, work.key_cache, work.value_cache, lens, table, config)
    torch.cuda.synchronize()
    # A warm first call (the array's address is resolved and the kernels' modules are loaded on first use), then the
    # call that is held to the device's own free-memory figure: torch's counters would not see a hipMalloc inside the
    # library, hipMemGetInfo does.
    A.paged_kv_decode_attention_no_alloc_bf16(None, got, work.query, work.key_cache, work.value_cache, lens, table, config)
    torch.cuda.synchronize()
    got.fill_(float("nan"))
    torch.cuda.synchronize()
    before, reserved = torch.cuda.mem_get_info()[0], torch.cuda.memory_reserved()
    A.paged_kv_decode_attention_no_alloc_bf16(None, got, work.query, work.key_cache, work.value_cache, lens, table, config)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == before and torch.cuda.memory_reserved() == reserved
    return want, got


def _oracle(work):
    return oracle.paged_kv_decode_attention_f32(
        work.query.float().cpu().numpy(), work.key_cache.float().cpu().numpy(), work.value_cache.float().cpu().numpy(),
        work.seq_lens, work.block_table, batch=work.batch, heads=work.heads, kv_heads=work.kv_heads,
        head_dim=work.head_dim, block_size=work.block_size, block_table_batch_stride=work.block_table_batch_stride,
        scale=work.scale, threads=8)


def test_no_alloc_decode_equals_the_workspace_entry_point_twice_in_a_row():
    big = synthetic.paged_decode_workload(batch=24, heads=32, kv_heads=8, physical_blocks=2048,
                                          seq_lens=[int(n) for n in np.random.default_rng(5).integers(0, 1200, 24)], seed=71)
    small = synthetic.paged_decode_workload(batch=3, heads=32, kv_heads=8, physical_blocks=256, seq_lens=[77, 1, 300], seed=72)
    for work in (big, small):
        print(f"no-alloc decode: batch {work.batch} lens {work.seq_lens.tolist()}", flush=True)
        want, got = _both(work)
        assert torch.equal(want.view(torch.int16), got.view(torch.int16))
        gap = np.abs(got.float().cpu().numpy() - _oracle(work))
        assert np.isfinite(gap).all() and gap.max() <= 2e-2 and gap.mean() <= 2e-3, (gap.max(), gap.mean())


def test_no_alloc_decode_refuses_a_config_beyond_the_fixed_scratch():
    work = synthetic.paged_decode_workload(batch=2, heads=32, kv_heads=8, physical_blocks=64, seq_lens=[5, 9], seed=3)
    lens = torch.from_numpy(work.seq_lens).cuda()
    table = torch.from_numpy(work.block_table.view(np.int32)).cuda()
    # 4000 sequences need more partial rows than the fixed scratch holds; refused before any pointer is read.
    config = A.PagedKvDecodeAttentionConfig.contiguous(4000, work.heads, work.kv_heads, work.head_dim, work.block_size,
                                                       work.physical_blocks, work.block_table_batch_stride, work.scale)
    assert config.workspace_bytes() > A.STATIC_SCRATCH_BYTES
    out = torch.zeros((2, work.heads, work.head_dim), device="cuda", dtype=torch.bfloat16)
    with pytest.raises(error.LengthTooShort) as caught:
        A.paged_kv_decode_attention_no_alloc_bf16(None, out, work.query, work.key_cache, work.value_cache, lens, table, config)
    assert "static scratch" in str(caught.value)
    detail = _native.ErrorDetail()
    _native.lib().singe_hip_last_error(ctypes.byref(detail))
    assert detail.actual == A.STATIC_SCRATCH_BYTES and detail.minimum == config.workspace_bytes()
