"""Seeded random shapes for the bf16 matrix-core kernels against the CPU oracle: what a hand-picked list of cases
misses (odd groupings, page sizes on both sides of the scalar page path, sequences of any mix of query and key
counts, key splits on and off, every option at once).  Same tolerances as the hand-picked cases."""
import numpy as np
import pytest
import torch

import oracle
from singe_amd import _native, neural
from singe_amd.kernel import attention as A

pytestmark = pytest.mark.gpu

MAX_ABS, MEAN_ABS, LSE_ABS = 2e-2, 2e-3, 2e-3


@pytest.mark.parametrize("seed", range(16))
def test_paged_attention_random_shapes_on_the_two_tile_kernel(seed):
    # plain calls (no window, no cap, no key shares) with page sizes the kernel takes and longer chunks, sent to the kernel
    # that gives a wave two 32-row tiles whatever their size
    rng = np.random.default_rng(3000 + seed)
    _native.lib().singe_hip_set_paged_attention_rows_per_wave(64)
    try:
        paged_attention_random_shape(seed, rng, two_tiles=True)
    finally:
        _native.lib().singe_hip_set_paged_attention_rows_per_wave(0)


@pytest.mark.parametrize("seed", range(24))
def test_paged_attention_random_shapes(seed):
    paged_attention_random_shape(seed, np.random.default_rng(1000 + seed), two_tiles=False)


def paged_attention_random_shape(seed, rng, two_tiles):
    kv_heads = int(rng.choice([1, 2, 3, 4, 8]))
    heads = kv_heads * int(rng.choice([1, 2, 4, 5, 8]))
    page_size = int(rng.choice([16, 16, 32, 64, 128, 256] if two_tiles else [1, 2, 3, 8, 16, 16, 32, 64, 128, 24]))
    count = int(rng.integers(1, 7))
    sequences = []
    for _ in range(count):
        keys = int(rng.choice([0, 1, int(rng.integers(1, 64)), int(rng.integers(64, 700)), int(rng.integers(700, 2500))]))
        queries = int(rng.choice([0, 1, 1, int(rng.integers(1, 40)), int(rng.integers(40, 900 if two_tiles else 300))]))
        sequences.append((queries, keys))
    if sum(q for q, _ in sequences) == 0:
        sequences[0] = (3, sequences[0][1])
    options = neural.AttentionOptions(causal=bool(rng.integers(0, 2)),
                                      window=None if two_tiles or rng.integers(0, 3) else int(rng.integers(1, 300)),
                                      softcap=None if two_tiles or rng.integers(0, 4) else float(rng.uniform(2.0, 40.0)),
                                      scale=None if rng.integers(0, 2) else float(rng.uniform(0.02, 0.2)))
    index_dtype = torch.int64 if rng.integers(0, 2) else torch.int32
    splits = 1 if two_tiles else int(rng.choice([0, 0, 1, 2, 5, 16]))

    query_offsets, page_offsets, last = [0], [0], []
    for queries, keys in sequences:
        query_offsets.append(query_offsets[-1] + queries)
        pages = (keys + page_size - 1) // page_size
        page_offsets.append(page_offsets[-1] + pages)
        last.append(0 if keys == 0 else keys - (pages - 1) * page_size)
    needed = page_offsets[-1]
    page_count = needed + int(rng.integers(1, 5))
    table = rng.permutation(page_count)[:needed].tolist()
    tokens = query_offsets[-1]
    gen = torch.Generator(device="cuda")
    gen.manual_seed(seed)
    dim = (128, 64, 96, 112, 80, 48, 32, 16)[seed % 8] if two_tiles else 128  # (every build of the two-tile kernel)
    q = torch.randn((tokens, heads, dim), generator=gen, device="cuda").to(torch.bfloat16)
    kc = torch.randn((page_count, page_size, kv_heads, dim), generator=gen, device="cuda").to(torch.bfloat16)
    vc = torch.randn((page_count, page_size, kv_heads, dim), generator=gen, device="cuda").to(torch.bfloat16)
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
    case = (sequences, heads, kv_heads, page_size, options, splits)
    assert np.isfinite(got).all(), case
    gap = np.abs(got - want)
    assert gap.max(initial=0.0) <= MAX_ABS and (gap.size == 0 or gap.mean() <= MEAN_ABS), (case, gap.max(initial=0.0))
    empty = np.isneginf(want_lse)
    assert np.array_equal(np.isneginf(got_lse), empty), case
    assert np.abs(got_lse[~empty] - want_lse[~empty]).max(initial=0.0) <= LSE_ABS, case


@pytest.mark.parametrize("rows_per_wave,dim", [(0, 128), (64, 128), (64, 64), (64, 96), (64, 112), (64, 80), (64, 48), (64, 32), (64, 16)])
@pytest.mark.parametrize("seed", range(12))
def test_dense_prefill_random_shapes(seed, rows_per_wave, dim):
    # (64 rows a wave: the kernel that gives a wave two 32-row tiles, whatever the shape; larger shapes there, so that
    # several 256-row tiles and key tiles on both sides of the masks are met)
    rng = np.random.default_rng(2000 + seed + 100 * rows_per_wave + dim)
    _native.lib().singe_hip_set_dense_prefill_rows_per_wave(rows_per_wave)
    try:
        dense_prefill_random_shape(seed, rng, dim, 3 if rows_per_wave else 1)
    finally:
        _native.lib().singe_hip_set_dense_prefill_rows_per_wave(0)


def dense_prefill_random_shape(seed, rng, dim, stretch):
    batch = int(rng.integers(1, 4))
    kv_heads = int(rng.choice([1, 2, 4]))
    heads = kv_heads * int(rng.choice([1, 2, 4]))
    query_len = int(rng.choice([1, int(rng.integers(2, 130)), int(rng.integers(130, 700 * stretch))]))
    key_len = query_len if rng.integers(0, 2) else int(rng.choice([1, int(rng.integers(2, 130)), int(rng.integers(130, 900 * stretch))]))
    causal = bool(rng.integers(0, 2))
    scale = float(rng.uniform(0.03, 0.15)) * (-1.0 if rng.integers(0, 6) == 0 else 1.0)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(seed)
    q = torch.randn((batch, query_len, heads, dim), generator=gen, device="cuda").to(torch.bfloat16)
    k = torch.randn((batch, key_len, kv_heads, dim), generator=gen, device="cuda").to(torch.bfloat16)
    v = torch.randn((batch, key_len, kv_heads, dim), generator=gen, device="cuda").to(torch.bfloat16)
    config = A.FmhaPrefillConfig.contiguous(batch, query_len, key_len, heads, kv_heads, dim, scale, causal)
    out = torch.full_like(q, float("nan"))
    lse = torch.full((batch, heads, query_len), float("nan"), device="cuda", dtype=torch.float32)
    A.fmha_prefill_lse_bf16(None, out, lse, q, k, v, config)
    torch.cuda.synchronize()
    want, want_lse = oracle.fmha_prefill_lse_f32(q.float().cpu().numpy(), k.float().cpu().numpy(), v.float().cpu().numpy(), batch=batch,
                                                 query_len=query_len, key_len=key_len, heads=heads, kv_heads=kv_heads, head_dim=dim,
                                                 scale=scale, causal=causal, threads=8)
    got = out.float().cpu().numpy()
    case = (batch, query_len, key_len, heads, kv_heads, causal, scale, dim)
    assert np.isfinite(got).all(), case
    gap = np.abs(got - want)
    assert gap.max() <= MAX_ABS and gap.mean() <= MEAN_ABS, (case, gap.max())
    assert np.abs(lse.cpu().numpy() - want_lse).max() <= LSE_ABS, case


@pytest.mark.parametrize("seed", range(32))
def test_decode_steps_through_the_op_random_shapes(seed):
    """Random decode steps (no more tokens than sequences: mostly a token a sequence, some sequences with none, a few
    with two or three) through the paged attention op, which runs them on the block-table decode kernels: against the
    oracle, both head dimensions, both index types, bf16 and f16, causal or not, with and without a window, up to 16 query
    heads a kv head."""
    rng = np.random.default_rng(5000 + seed)
    kv_heads = int(rng.choice([1, 2, 4, 8]))
    heads = kv_heads * int(rng.choice([1, 2, 3, 4, 5, 8, 12, 16]))
    dim = int(rng.choice([128, 128, 64]))
    page_size = int(rng.choice([1, 3, 8, 16, 16, 32, 64, 24]))
    dtype = torch.bfloat16 if rng.integers(0, 3) else torch.float16
    count = int(rng.choice([1, 2, 5, 17, 70, 130]))
    sequences, spare = [], 0
    for _ in range(count):
        keys = int(rng.choice([0, 1, int(rng.integers(1, 64)), int(rng.integers(64, 700)), int(rng.integers(700, 3000)), int(rng.integers(2048, 4500))]))
        queries = int(rng.choice([1, 1, 1, 1, 0, 2, 3]))
        if queries > 1 and spare < queries - 1:
            queries = 1
        spare += 1 - queries
        sequences.append((queries, keys))
    if sum(q for q, _ in sequences) == 0:
        sequences[0] = (1, sequences[0][1])
    options = neural.AttentionOptions(causal=bool(rng.integers(0, 2)), scale=None if rng.integers(0, 2) else float(rng.uniform(0.02, 0.2)),
                                      window=None if rng.integers(0, 2) else int(rng.choice([1, 100, 2048, 2300, 2999, 5000])))
    index_dtype = torch.int64 if rng.integers(0, 2) else torch.int32
    query_offsets, page_offsets, last = [0], [0], []
    for queries, keys in sequences:
        query_offsets.append(query_offsets[-1] + queries)
        pages = (keys + page_size - 1) // page_size
        page_offsets.append(page_offsets[-1] + pages)
        last.append(0 if keys == 0 else keys - (pages - 1) * page_size)
    needed = page_offsets[-1]
    page_count = needed + int(rng.integers(1, 5))
    table = rng.permutation(page_count)[:needed].tolist()
    tokens = query_offsets[-1]
    assert 0 < tokens <= len(sequences)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(seed)
    rand = lambda *shape: torch.randn(shape, generator=gen, device="cuda").to(dtype)
    q, kc, vc = rand(tokens, heads, dim), rand(page_count, page_size, kv_heads, dim), rand(page_count, page_size, kv_heads, dim)
    index = lambda values: torch.tensor(values, dtype=index_dtype, device="cuda")
    paging = neural.Paging(index(query_offsets), index(page_offsets), index(table), index(last))
    out, lse = neural.paged_attention(q, kc, vc, paging, options)
    torch.cuda.synchronize()
    status, want, want_lse = oracle.paged_attention_f32(q.float().cpu().numpy(), kc.float().cpu().numpy(), vc.float().cpu().numpy(), query_offsets,
                                                        page_offsets, table, last, scale=options.scale, causal=options.causal,
                                                        window=options.window, threads=8)
    assert status == 0
    got, got_lse = out.float().cpu().numpy(), lse.cpu().numpy()
    gap = np.abs(got - want)
    assert gap.max() <= MAX_ABS and gap.mean() <= MEAN_ABS, (gap.max(), gap.mean())
    empty = np.isneginf(want_lse)
    assert np.array_equal(np.isneginf(got_lse), empty) and not got[empty].any()
    assert np.abs(got_lse[~empty] - want_lse[~empty]).max(initial=0.0) <= LSE_ABS
