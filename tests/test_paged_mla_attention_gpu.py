"""Latent (MLA) attention over paged caches on the GPU against the CPU oracle (paged_mla_attention restated, f64),
through the C ABI.  Inputs, shapes and tolerances are those of the reference's own device-against-CPU test
(singe/src/backend/cuda/kernel_plan/source/tests.rs:1191-1316): values ((index * 37 + seed * 11) % 41) / 40 - 0.5,
scale 0.07, output within 0.02 (bf16) / 0.003 (f16), LSE within 1e-3 relative; f32 within 1e-4 here."""
import numpy as np
import pytest
import torch

import oracle
from singe_amd import error, neural

pytestmark = pytest.mark.gpu


def values(shape, seed):
    count = int(np.prod(shape))
    index = np.arange(count, dtype=np.int64)
    return (((index * 37 + seed * 11) % 41).astype(np.float32) / 40.0 - 0.5).reshape(shape)


MANY = [(int(q), 0 if s % 17 == 5 else int(q) + s % 23) for s, q in enumerate(np.random.default_rng(2).choice([0, 1, 1, 2, 3, 7], size=100))]
BATCHES = [
    MANY,                                  # more sequences than one wave's prefix sum covers, some without queries or keys
    [(1, 150), (9, 9), (5, 70), (2, 0)],   # decode over a long cache, a whole prefill, a chunk, a sequence with no keys
    [(1, 2000), (2, 1500)],                # few long sequences
    [(1, 300), (1, 40), (1, 0)],           # decoding alone
]
TOLERANCE = {torch.bfloat16: 0.02, torch.float16: 0.003, torch.float32: 1e-4}


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("heads,latent,positional,page_size", [(16, 512, 64, 1), (8, 128, 32, 5)])
@pytest.mark.parametrize("sequences", BATCHES)
def test_matches_the_cpu_over_ragged_sequences(sequences, heads, latent, positional, page_size, causal, dtype):
    query_offsets, page_offsets, last, needed = [0], [0], [], 0
    for queries, keys in sequences:
        query_offsets.append(query_offsets[-1] + queries)
        pages = (keys + page_size - 1) // page_size
        needed += pages
        page_offsets.append(needed)
        last.append(0 if keys == 0 else keys - (pages - 1) * page_size)
    page_count = needed + 3
    table = [(page * 7 + 2) % page_count for page in range(needed)]
    tokens = query_offsets[-1]
    host = [values((tokens, heads, latent), 1), values((tokens, heads, positional), 2), values((page_count, page_size, latent), 3),
            values((page_count, page_size, positional), 4)]
    device = [torch.tensor(array).to(dtype).cuda() for array in host]
    rounded = [tensor.float().cpu().numpy() for tensor in device]
    index = lambda entries: torch.tensor(entries, dtype=torch.int32, device="cuda")
    paging = neural.Paging(index(query_offsets), index(page_offsets), index(table), index(last))
    out, lse = neural.paged_mla_attention(*device, paging, neural.AttentionOptions(causal=causal, scale=0.07))
    torch.cuda.synchronize()
    status, want, want_lse = oracle.paged_mla_attention(*rounded, query_offsets, page_offsets, table, last, scale=0.07, causal=causal,
                                                        threads=8)
    assert status == 0
    got, got_lse = out.float().cpu().numpy(), lse.cpu().numpy()
    assert np.abs(got - want).max() <= TOLERANCE[dtype]
    empty = np.isneginf(want_lse)
    assert np.array_equal(np.isneginf(got_lse), empty) and not got[empty].any()
    assert (np.abs(got_lse[~empty] - want_lse[~empty]) <= 1e-3 * np.maximum(np.abs(want_lse[~empty]), 1.0)).all()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("heads,page_size,index_dtype", [(128, 16, torch.int32), (24, 5, torch.int64), (1, 64, torch.int32), (40, 1, torch.int32)])
def test_matrix_core_shape_on_random_data(heads, page_size, index_dtype, causal, dtype):
    """Latent width 512 with positional width 64 runs on the matrix cores, 128 (token, head) rows to a workgroup:
    head counts that fill a workgroup exactly, leave waves empty, or let one wave's rows span several tokens;
    decode rows, chunks, whole prefills, more queries than keys, a sequence without keys."""
    sequences = [(1, 700), (37, 37), (20, 333), (3, 0), (9, 4), (1, 65)]
    query_offsets, page_offsets, last, needed = [0], [0], [], 0
    for queries, keys in sequences:
        query_offsets.append(query_offsets[-1] + queries)
        pages = (keys + page_size - 1) // page_size
        needed += pages
        page_offsets.append(needed)
        last.append(0 if keys == 0 else keys - (pages - 1) * page_size)
    page_count = needed + 2
    rng = np.random.default_rng(heads + page_size)
    table = [int(page) for page in rng.permutation(page_count)[:needed]]
    tokens = query_offsets[-1]
    gen = torch.Generator(device="cuda")
    gen.manual_seed(heads)
    rand = lambda *shape: torch.randn(shape, generator=gen, device="cuda").to(dtype)
    device = [rand(tokens, heads, 512), rand(tokens, heads, 64), rand(page_count, page_size, 512), rand(page_count, page_size, 64)]
    index = lambda entries: torch.tensor(entries, dtype=index_dtype, device="cuda")
    paging = neural.Paging(index(query_offsets), index(page_offsets), index(table), index(last))
    out, lse = neural.paged_mla_attention(*device, paging, neural.AttentionOptions(causal=causal))
    torch.cuda.synchronize()
    status, want, want_lse = oracle.paged_mla_attention(*[tensor.float().cpu().numpy() for tensor in device], query_offsets, page_offsets, table,
                                                        last, causal=causal, threads=8)
    assert status == 0
    got, got_lse = out.float().cpu().numpy(), lse.cpu().numpy()
    gap = np.abs(got - want)
    assert gap.max() <= 2e-2 and gap.mean() <= 2e-3, (gap.max(), gap.mean())
    empty = np.isneginf(want_lse)
    assert np.array_equal(np.isneginf(got_lse), empty) and not got[empty].any()
    assert np.abs(got_lse[~empty] - want_lse[~empty]).max() <= 5e-3


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("latent,positional", [(128, 32), (256, 64), (384, 16), (32, 16), (96, 32), (480, 48), (512, 32), (256, 0), (64, 64)])
@pytest.mark.parametrize("splits", [0, 5])
def test_matrix_cores_at_the_reference_plan_s_other_widths(latent, positional, causal, dtype, splits):
    """The widths the reference's tensor-core plan takes beside 512 + 64 (latent a multiple of 32 up to 512, positional a
    multiple of 8 that makes the key width a multiple of 16: mla.rs:75, 140-146; positional parts up to 64 here) run on
    the matrix cores too, with and without key splits, against the oracle on random data."""
    import ctypes
    from singe_amd import _native
    sequences, heads, page_size = [(1, 700), (37, 37), (20, 333), (3, 0), (9, 4), (1, 65)], 24, 16
    query_offsets, page_offsets, last, needed = [0], [0], [], 0
    for queries, keys in sequences:
        query_offsets.append(query_offsets[-1] + queries)
        pages = (keys + page_size - 1) // page_size
        needed += pages
        page_offsets.append(needed)
        last.append(0 if keys == 0 else keys - (pages - 1) * page_size)
    page_count = needed + 2
    rng = np.random.default_rng(latent + positional)
    table = [int(page) for page in rng.permutation(page_count)[:needed]]
    tokens = query_offsets[-1]
    gen = torch.Generator(device="cuda")
    gen.manual_seed(latent)
    rand = lambda *shape: torch.randn(shape, generator=gen, device="cuda").to(dtype)
    device = [rand(tokens, heads, latent), rand(tokens, heads, positional), rand(page_count, page_size, latent), rand(page_count, page_size, positional)]
    index = lambda entries: torch.tensor(entries, dtype=torch.int64, device="cuda")
    paging = neural.Paging(index(query_offsets), index(page_offsets), index(table), index(last))
    _native.lib().singe_hip_set_paged_mla_attention_splits(splits)
    try:
        out, lse = neural.paged_mla_attention(*device, paging, neural.AttentionOptions(causal=causal))
        torch.cuda.synchronize()
    finally:
        _native.lib().singe_hip_set_paged_mla_attention_splits(0)
    status, want, want_lse = oracle.paged_mla_attention(*[tensor.float().cpu().numpy() for tensor in device], query_offsets, page_offsets, table,
                                                        last, causal=causal, threads=8)
    assert status == 0
    got, got_lse = out.float().cpu().numpy(), lse.cpu().numpy()
    assert np.isfinite(got).all()
    gap = np.abs(got - want)
    worst, mean = (2e-2, 2e-3) if dtype == torch.bfloat16 else (5e-3, 5e-4)
    assert gap.max() <= worst and gap.mean() <= mean, (gap.max(), gap.mean())
    empty = np.isneginf(want_lse)
    assert np.array_equal(np.isneginf(got_lse), empty) and not got[empty].any()
    assert np.abs(got_lse[~empty] - want_lse[~empty]).max() <= 5e-3


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("splits", [2, 3, 16, 64])
@pytest.mark.parametrize("causal", [False, True])
def test_key_splits_match_the_cpu_and_the_unsplit_kernel(splits, causal, dtype):
    """With scratch lent, a row tile's keys are shared out over workgroups and merged by a second kernel: decode rows
    over long and short caches, a chunk, a sequence without keys, more shares than a sequence has tiles."""
    import ctypes
    from singe_amd import _native
    sequences, heads, page_size = [(1, 1500), (1, 40), (5, 700), (2, 0), (1, 65), (3, 300)], 24, 16
    query_offsets, page_offsets, last, needed = [0], [0], [], 0
    for queries, keys in sequences:
        query_offsets.append(query_offsets[-1] + queries)
        pages = (keys + page_size - 1) // page_size
        needed += pages
        page_offsets.append(needed)
        last.append(0 if keys == 0 else keys - (pages - 1) * page_size)
    rng = np.random.default_rng(splits)
    table = [int(page) for page in rng.permutation(needed + 2)[:needed]]
    tokens = query_offsets[-1]
    gen = torch.Generator(device="cuda")
    gen.manual_seed(splits)
    rand = lambda *shape: torch.randn(shape, generator=gen, device="cuda").to(dtype)
    device = [rand(tokens, heads, 512), rand(tokens, heads, 64), rand(needed + 2, page_size, 512), rand(needed + 2, page_size, 64)]
    index = lambda entries: torch.tensor(entries, dtype=torch.int32, device="cuda")
    paging = neural.Paging(index(query_offsets), index(page_offsets), index(table), index(last))
    options = neural.AttentionOptions(causal=causal)
    whole, whole_lse = neural.paged_mla_attention(*device, paging, options, scratch=False)
    _native.lib().singe_hip_set_paged_mla_attention_splits(splits)
    try:
        out, lse = neural.paged_mla_attention(*device, paging, options)
    finally:
        _native.lib().singe_hip_set_paged_mla_attention_splits(0)
    torch.cuda.synchronize()
    status, want, want_lse = oracle.paged_mla_attention(*[tensor.float().cpu().numpy() for tensor in device], query_offsets, page_offsets, table,
                                                        last, causal=causal, threads=8)
    assert status == 0
    got, got_lse = out.float().cpu().numpy(), lse.cpu().numpy()
    gap = np.abs(got - want)
    assert gap.max() <= 2e-2 and gap.mean() <= 2e-3, (gap.max(), gap.mean())
    empty = np.isneginf(want_lse)
    assert np.array_equal(np.isneginf(got_lse), empty) and not got[empty].any()
    assert np.abs(got_lse[~empty] - want_lse[~empty]).max() <= 5e-3
    assert (out.float() - whole.float()).abs().max().item() <= 2e-2
    assert np.abs(got_lse[~empty] - whole_lse.cpu().numpy()[~empty]).max() <= 2e-3


@pytest.mark.parametrize("sequences, heads", [([(1, 9000)], 128), ([(1, 5000), (1, 3000), (1, 16)], 16), ([(2, 4100)] * 5, 40)])
def test_few_long_sequences_share_their_keys_out_over_the_chip(sequences, heads):
    """The shares the library picks by itself for a decode step over few, long sequences (up to 64 of them a row
    tile, spread round the XCDs, merged a wave per row): the scratch it asks for says how many, and the result
    matches the CPU."""
    import ctypes
    from singe_amd import _native
    page_size = 64
    query_offsets, page_offsets, last, needed = [0], [0], [], 0
    for queries, keys in sequences:
        query_offsets.append(query_offsets[-1] + queries)
        pages = (keys + page_size - 1) // page_size
        needed += pages
        page_offsets.append(needed)
        last.append(keys - (pages - 1) * page_size)
    table = [int(page) for page in np.random.default_rng(11).permutation(needed)]
    tokens = query_offsets[-1]
    problem = _native.PagedMlaAttentionProblemC(tokens, heads, 512, 64, page_size, len(sequences), needed, needed, 1, 0, 1, 0, 0.0)
    shares = _native.lib().singe_hip_paged_mla_attention_scratch_bytes(ctypes.byref(problem)) // (tokens * heads * 513 * 4)
    assert 16 < shares <= 64
    gen = torch.Generator(device="cuda")
    gen.manual_seed(len(sequences))
    rand = lambda *shape: torch.randn(shape, generator=gen, device="cuda").to(torch.bfloat16)
    device = [rand(tokens, heads, 512), rand(tokens, heads, 64), rand(needed, page_size, 512), rand(needed, page_size, 64)]
    index = lambda entries: torch.tensor(entries, dtype=torch.int32, device="cuda")
    paging = neural.Paging(index(query_offsets), index(page_offsets), index(table), index(last))
    out, lse = neural.paged_mla_attention(*device, paging, neural.AttentionOptions(causal=True))
    torch.cuda.synchronize()
    status, want, want_lse = oracle.paged_mla_attention(*[tensor.float().cpu().numpy() for tensor in device], query_offsets, page_offsets, table,
                                                        last, causal=True, threads=8)
    assert status == 0
    gap = np.abs(out.float().cpu().numpy() - want)
    assert gap.max() <= 2e-2 and gap.mean() <= 2e-3, (gap.max(), gap.mean())
    assert np.abs(lse.cpu().numpy() - want_lse).max() <= 5e-3


@pytest.mark.parametrize("bad_page", [-1, 9])
def test_matrix_core_kernel_reports_a_bad_page_and_leaves_other_sequences_right(bad_page):
    """A page id outside the cache sets the status word (its keys are read as zeros); the other sequence's rows are
    what they are without it."""
    heads, page_size, pages = 16, 16, 9
    gen = torch.Generator(device="cuda")
    gen.manual_seed(5)
    rand = lambda *shape: torch.randn(shape, generator=gen, device="cuda").to(torch.bfloat16)
    device = [rand(3, heads, 512), rand(3, heads, 64), rand(pages, page_size, 512), rand(pages, page_size, 64)]
    index = lambda entries: torch.tensor(entries, dtype=torch.int32, device="cuda")
    good = neural.Paging(index([0, 1, 3]), index([0, 4, 8]), index([8, 0, 3, 5, 1, 2, 6, 7]), index([10, 16]))
    bad = neural.Paging(index([0, 1, 3]), index([0, 4, 8]), index([8, 0, 3, 5, 1, bad_page, 6, 7]), index([10, 16]))
    want, want_lse = neural.paged_mla_attention(*device, good, neural.AttentionOptions(causal=True))
    with pytest.raises(error.IndexOutOfBounds):
        neural.paged_mla_attention(*device, bad, neural.AttentionOptions(causal=True))
    status = torch.zeros(1, device="cuda", dtype=torch.int32)
    out, lse = neural.paged_mla_attention(*device, bad, neural.AttentionOptions(causal=True), status=status, check=False)
    torch.cuda.synchronize()
    assert int(status.item()) == 1
    assert torch.equal(out[:1], want[:1]) and torch.equal(lse[:1], want_lse[:1])
    assert torch.isfinite(out.float()).all()


def test_decode_at_full_size_splits_on_its_own_and_agrees_with_the_unsplit_kernel_and_a_torch_reference():
    """64 sequences of 2048 to 4096 keys, 128 heads: too large for the CPU oracle in a test, so the split and unsplit
    kernels are held to each other and to a plain torch f32 evaluation of the same rows on the device."""
    import ctypes
    heads, page_size = 128, 64
    rng = np.random.default_rng(3)
    lengths = [int(n) for n in rng.integers(2048, 4097, size=64)]
    query_offsets, page_offsets, last, needed = list(range(65)), [0], [], 0
    for keys in lengths:
        pages = (keys + page_size - 1) // page_size
        needed += pages
        page_offsets.append(needed)
        last.append(keys - (pages - 1) * page_size)
    table = [int(page) for page in rng.permutation(needed)]
    gen = torch.Generator(device="cuda")
    gen.manual_seed(13)
    rand = lambda *shape: torch.randn(shape, generator=gen, device="cuda").to(torch.bfloat16)
    q, qp, lc, pc = rand(64, heads, 512), rand(64, heads, 64), rand(needed, page_size, 512), rand(needed, page_size, 64)
    index = lambda entries: torch.tensor(entries, dtype=torch.int32, device="cuda")
    paging = neural.Paging(index(query_offsets), index(page_offsets), index(table), index(last))
    options = neural.AttentionOptions(causal=True)
    whole, whole_lse = neural.paged_mla_attention(q, qp, lc, pc, paging, options, scratch=False)
    out, lse = neural.paged_mla_attention(q, qp, lc, pc, paging, options)  # 64 workgroups for 256 compute units: it splits
    assert (out.float() - whole.float()).abs().max().item() <= 1e-2
    assert (lse - whole_lse).abs().max().item() <= 1e-3
    scale = 1.0 / np.sqrt(576.0)
    for sequence in (0, 31, 63):
        pages = torch.tensor(table[page_offsets[sequence]:page_offsets[sequence + 1]], device="cuda")
        keys = lengths[sequence]
        latent = lc[pages].reshape(-1, 512)[:keys].float()
        positional = pc[pages].reshape(-1, 64)[:keys].float()
        scores = (q[sequence].float() @ latent.T + qp[sequence].float() @ positional.T) * scale
        want = torch.softmax(scores, dim=-1) @ latent
        gap = (out[sequence].float() - want).abs()
        assert gap.max().item() <= 2e-2 and gap.mean().item() <= 2e-3
        want_lse = torch.logsumexp(scores, dim=-1) / np.log(2.0)
        assert (lse[sequence] - want_lse).abs().max().item() <= 5e-3


def test_default_scale_counts_the_whole_key_width_and_int64_indices():
    gen = torch.Generator(device="cuda")
    gen.manual_seed(1)
    rand = lambda *shape: torch.randn(shape, generator=gen, device="cuda").to(torch.bfloat16)
    q, qp, lc, pc = rand(7, 4, 192), rand(7, 4, 24), rand(9, 4, 192), rand(9, 4, 24)
    index = lambda entries: torch.tensor(entries, dtype=torch.int64, device="cuda")
    qo, po, table, last = [0, 3, 7], [0, 4, 7], [8, 0, 3, 5, 1, 2, 6], [2, 4]
    out, lse = neural.paged_mla_attention(q, qp, lc, pc, neural.Paging(index(qo), index(po), index(table), index(last)),
                                          neural.AttentionOptions(causal=True))
    host = lambda tensor: tensor.float().cpu().numpy()
    status, want, want_lse = oracle.paged_mla_attention(host(q), host(qp), host(lc), host(pc), qo, po, table, last, causal=True)
    assert status == 0
    assert np.abs(host(out) - want).max() <= 0.02 and np.abs(lse.cpu().numpy() - want_lse).max() <= 2e-3


TOKENS, HEADS, LATENT, POSITIONAL, SLOTS, PAGES = 2, 2, 32, 8, 4, 2
VALID = dict(query_offsets=[0, 2], page_offsets=[0, 1], pages=[0], last_page_lengths=[2])
INVALID = [dict(query_offsets=[0, 3]), dict(query_offsets=[-1, 2]), dict(query_offsets=[2, 0]), dict(page_offsets=[0, 2]),
           dict(page_offsets=[-1, 1]), dict(pages=[PAGES]), dict(pages=[-1]), dict(last_page_lengths=[SLOTS + 1]),
           dict(last_page_lengths=[-1])]


def attend_mla(paging_values, dtype):
    # singe/tests/nn/paged_attention.rs:127-161
    q = torch.zeros((TOKENS, HEADS, LATENT), device="cuda", dtype=torch.bfloat16)
    qp = torch.zeros((TOKENS, HEADS, POSITIONAL), device="cuda", dtype=torch.bfloat16)
    lc = torch.zeros((PAGES, SLOTS, LATENT), device="cuda", dtype=torch.bfloat16)
    pc = torch.zeros((PAGES, SLOTS, POSITIONAL), device="cuda", dtype=torch.bfloat16)
    entries = {**VALID, **paging_values}
    index = lambda v: torch.tensor(v, dtype=dtype, device="cuda")
    paging = neural.Paging(index(entries["query_offsets"]), index(entries["page_offsets"]), index(entries["pages"]),
                           index(entries["last_page_lengths"]))
    return neural.paged_mla_attention(q, qp, lc, pc, paging, neural.AttentionOptions(causal=True))


@pytest.mark.parametrize("dtype", [torch.int32, torch.int64])
def test_paging_values_outside_their_buffers_are_refused(dtype):
    attend_mla({}, dtype)
    for bad in INVALID:
        with pytest.raises(error.IndexOutOfBounds):
            attend_mla(bad, dtype)


def test_shapes_the_op_does_not_take():
    zeros = lambda *shape: torch.zeros(shape, device="cuda", dtype=torch.bfloat16)
    index = lambda v: torch.tensor(v, dtype=torch.int32, device="cuda")
    paging = neural.Paging(index([0, 2]), index([0, 1]), index([0]), index([2]))
    with pytest.raises(error.InvalidArgument):   # positional cache of another width
        neural.paged_mla_attention(zeros(2, 2, 32), zeros(2, 2, 8), zeros(2, 4, 32), zeros(2, 4, 16), paging)
    with pytest.raises(error.UnsupportedWidth):  # beyond the widths this kernel holds
        neural.paged_mla_attention(zeros(2, 2, 576), zeros(2, 2, 8), zeros(2, 4, 576), zeros(2, 4, 8), paging)


def random_latent_case(seed):
    """Random sequences over pages that hold whole 32-key tiles (the kernel then takes one page id a tile) or do not,
    at the built widths or others, with or without key shares, against the CPU oracle."""
    rng = np.random.default_rng(4000 + seed)
    page_size = int(rng.choice([32, 64, 128, 32, 64, 16, 48]))
    latent, positional = [(512, 64), (512, 64), (256, 64), (128, 32), (384, 16)][int(rng.integers(0, 5))]
    heads = int(rng.choice([1, 8, 16, 40, 128]))
    dtype = torch.bfloat16 if rng.integers(0, 2) else torch.float16
    index_dtype = torch.int64 if rng.integers(0, 2) else torch.int32
    causal = bool(rng.integers(0, 2))
    sequences = []
    for _ in range(int(rng.integers(1, 6))):
        keys = int(rng.choice([0, 1, int(rng.integers(1, 33)), int(rng.integers(33, 400)), int(rng.integers(400, 1500))]))
        queries = int(rng.choice([0, 1, 1, int(rng.integers(1, 30)), int(rng.integers(30, 200))]))
        sequences.append((queries, keys))
    if sum(q for q, _ in sequences) == 0:
        sequences[0] = (2, sequences[0][1])
    query_offsets, page_offsets, last, needed = [0], [0], [], 0
    for queries, keys in sequences:
        query_offsets.append(query_offsets[-1] + queries)
        pages = (keys + page_size - 1) // page_size
        needed += pages
        page_offsets.append(needed)
        last.append(0 if keys == 0 else keys - (pages - 1) * page_size)
    page_count = needed + int(rng.integers(1, 4))
    table = [int(page) for page in rng.permutation(page_count)[:needed]]
    tokens = query_offsets[-1]
    gen = torch.Generator(device="cuda")
    gen.manual_seed(seed)
    rand = lambda *shape: torch.randn(shape, generator=gen, device="cuda").to(dtype)
    device = [rand(tokens, heads, latent), rand(tokens, heads, positional), rand(page_count, page_size, latent), rand(page_count, page_size, positional)]
    index = lambda entries: torch.tensor(entries, dtype=index_dtype, device="cuda")
    paging = neural.Paging(index(query_offsets), index(page_offsets), index(table), index(last))
    from singe_amd import _native
    splits = int(rng.choice([0, 0, 1, 3, 8]))
    _native.lib().singe_hip_set_paged_mla_attention_splits(splits)
    try:
        out, lse = neural.paged_mla_attention(*device, paging, neural.AttentionOptions(causal=causal))
        torch.cuda.synchronize()
    finally:
        _native.lib().singe_hip_set_paged_mla_attention_splits(0)
    status, want, want_lse = oracle.paged_mla_attention(*[tensor.float().cpu().numpy() for tensor in device], query_offsets, page_offsets, table,
                                                        last, causal=causal, threads=8)
    assert status == 0
    case = (sequences, heads, latent, positional, page_size, causal, dtype, index_dtype, splits)
    got, got_lse = out.float().cpu().numpy(), lse.cpu().numpy()
    gap = np.abs(got - want)
    assert gap.max(initial=0.0) <= 2e-2 and (gap.size == 0 or gap.mean() <= 2e-3), (case, gap.max(initial=0.0))
    empty = np.isneginf(want_lse)
    assert np.array_equal(np.isneginf(got_lse), empty) and not got[empty].any(), case
    assert np.abs(got_lse[~empty] - want_lse[~empty]).max(initial=0.0) <= 5e-3, case


@pytest.mark.parametrize("seed", range(24))
def test_random_shapes_over_pages_of_whole_tiles_and_others(seed):
    random_latent_case(seed)
