"""f16 operands on the matrix-core kernels (head_dim 128) against the CPU oracle: the paged attention op with every
option, key splits, both index types and page paths, and the dense prefill of the singe-kernel surface
(fmha_prefill_f16 / fmha_prefill_lse_f16).  f16 carries three more mantissa bits than bf16, so the bounds are the
reference's own for f16, 3e-3 on outputs (kernel_plan/source/tests.rs:1299-1303), and 2e-3 on either LSE."""
import numpy as np
import pytest
import torch

import oracle
from singe_amd import _native, neural
from singe_amd.kernel import attention as A

pytestmark = pytest.mark.gpu

MAX_ABS, LSE_ABS = 3e-3, 2e-3


def paged_case(sequences, heads, kv_heads, page_size, options, index_dtype, seed, splits=0, dim=128):
    query_offsets, page_offsets, last = [0], [0], []
    for queries, keys in sequences:
        query_offsets.append(query_offsets[-1] + queries)
        pages = (keys + page_size - 1) // page_size
        page_offsets.append(page_offsets[-1] + pages)
        last.append(0 if keys == 0 else keys - (pages - 1) * page_size)
    needed = page_offsets[-1]
    page_count = needed + 3
    table = np.random.default_rng(seed).permutation(page_count)[:needed].tolist()
    gen = torch.Generator(device="cuda")
    gen.manual_seed(seed)
    q = torch.randn((query_offsets[-1], heads, dim), generator=gen, device="cuda").to(torch.float16)
    kc = torch.randn((page_count, page_size, kv_heads, dim), generator=gen, device="cuda").to(torch.float16)
    vc = torch.randn((page_count, page_size, kv_heads, dim), generator=gen, device="cuda").to(torch.float16)
    index = lambda values: torch.tensor(values, dtype=index_dtype, device="cuda")
    paging = neural.Paging(index(query_offsets), index(page_offsets), index(table), index(last))
    _native.lib().singe_hip_set_paged_attention_splits(splits)
    try:
        out, lse = neural.paged_attention(q, kc, vc, paging, options)
        torch.cuda.synchronize()
    finally:
        _native.lib().singe_hip_set_paged_attention_splits(0)
    status, want, want_lse = oracle.paged_attention_f32(
        q.float().cpu().numpy(), kc.float().cpu().numpy(), vc.float().cpu().numpy(), query_offsets, page_offsets, table, last,
        scale=options.scale, causal=options.causal, window=options.window, softcap=options.softcap, threads=8)
    assert status == 0
    got, got_lse = out.float().cpu().numpy(), lse.cpu().numpy()
    assert np.isfinite(got).all()
    assert np.abs(got - want).max() <= MAX_ABS, np.abs(got - want).max()
    empty = np.isneginf(want_lse)
    assert np.array_equal(np.isneginf(got_lse), empty) and not got[empty].any()
    assert np.abs(got_lse[~empty] - want_lse[~empty]).max(initial=0.0) <= LSE_ABS


SEQUENCES = [(1, 150), (70, 70), (20, 90), (3, 0), (9, 4), (130, 300)]
OPTIONS = [neural.AttentionOptions(), neural.AttentionOptions(causal=True), neural.AttentionOptions(causal=True, window=16, softcap=30.0),
           neural.AttentionOptions(scale=0.05, softcap=5.0)]


@pytest.mark.parametrize("options", OPTIONS)
@pytest.mark.parametrize("heads,kv_heads,page_size,index_dtype", [(8, 2, 1, torch.int32), (8, 1, 16, torch.int64), (4, 4, 7, torch.int64),
                                                                  (64, 8, 32, torch.int32)])
def test_paged_attention_f16(heads, kv_heads, page_size, index_dtype, options):
    paged_case(SEQUENCES, heads, kv_heads, page_size, options, index_dtype, seed=heads + page_size)


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("dim", [128, 64, 96, 112, 80, 48, 32, 16])
@pytest.mark.parametrize("heads,kv_heads,page_size,index_dtype", [(8, 1, 16, torch.int32), (64, 8, 16, torch.int64), (8, 2, 64, torch.int32)])
def test_paged_attention_f16_two_tiles_a_wave(heads, kv_heads, page_size, index_dtype, causal, dim):
    # the f16 builds of the kernel that gives a wave two 32-row tiles: chunks of several 256-row tiles, key counts either
    # side of a tile's end, sequences without keys or with more queries than keys
    _native.lib().singe_hip_set_paged_attention_rows_per_wave(64)
    try:
        paged_case(SEQUENCES + [(300, 1000), (257, 513), (64, 1024)], heads, kv_heads, page_size, neural.AttentionOptions(causal=causal),
                   index_dtype, seed=heads + page_size + 3, dim=dim)
    finally:
        _native.lib().singe_hip_set_paged_attention_rows_per_wave(0)


@pytest.mark.parametrize("splits", [3, 16])
def test_paged_attention_f16_key_splits(splits):
    paged_case([(1, 1500), (1, 40), (5, 700), (2, 0)], 8, 2, 16, neural.AttentionOptions(causal=True), torch.int32, seed=splits,
               splits=splits)


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("batch,query_len,key_len,heads,kv_heads", [(2, 256, 256, 4, 2), (1, 100, 100, 3, 1), (1, 33, 97, 2, 1),
                                                                      (1, 640, 1000, 4, 1), (1, 1, 1, 1, 1)])
def test_dense_prefill_f16(batch, query_len, key_len, heads, kv_heads, causal):
    gen = torch.Generator(device="cuda")
    gen.manual_seed(query_len + key_len)
    q = torch.randn((batch, query_len, heads, 128), generator=gen, device="cuda").to(torch.float16)
    k = torch.randn((batch, key_len, kv_heads, 128), generator=gen, device="cuda").to(torch.float16)
    v = torch.randn((batch, key_len, kv_heads, 128), generator=gen, device="cuda").to(torch.float16)
    scale = float(1.0 / np.sqrt(np.float32(128)))
    config = A.FmhaPrefillConfig.contiguous(batch, query_len, key_len, heads, kv_heads, 128, scale, causal)
    out = torch.full_like(q, float("nan"))
    lse = torch.full((batch, heads, query_len), float("nan"), device="cuda", dtype=torch.float32)
    A.fmha_prefill_lse_f16(None, out, lse, q, k, v, config)
    plain = torch.full_like(q, float("nan"))
    A.fmha_prefill_f16(None, plain, q, k, v, config)
    torch.cuda.synchronize()
    want, want_lse = oracle.fmha_prefill_lse_f32(q.float().cpu().numpy(), k.float().cpu().numpy(), v.float().cpu().numpy(), batch=batch,
                                                 query_len=query_len, key_len=key_len, heads=heads, kv_heads=kv_heads, head_dim=128,
                                                 scale=scale, causal=causal, threads=8)
    assert np.abs(out.float().cpu().numpy() - want).max() <= MAX_ABS
    assert np.abs(lse.cpu().numpy() - want_lse).max() <= LSE_ABS
    assert torch.equal(out, plain)


def test_dense_op_f16_takes_the_matrix_core_kernel_and_matches():
    gen = torch.Generator(device="cuda")
    gen.manual_seed(2)
    q = torch.randn((2, 4, 300, 128), generator=gen, device="cuda").to(torch.float16)
    k = torch.randn((2, 2, 300, 128), generator=gen, device="cuda").to(torch.float16)
    v = torch.randn((2, 2, 300, 128), generator=gen, device="cuda").to(torch.float16)
    got = neural.scaled_dot_product_attention(q, k, v, causal=True)
    want = oracle.scaled_dot_product_attention_f32(q.float().cpu().numpy(), k.float().cpu().numpy(), v.float().cpu().numpy(), causal=True)
    assert np.abs(got.float().cpu().numpy() - want).max() <= MAX_ABS
