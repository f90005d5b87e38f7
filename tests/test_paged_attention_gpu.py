"""The singe paged-attention op (FlashInfer form, bottom-right causal) on the GPU against the CPU oracle
(attend_paged restated), through the C ABI.  bf16 outputs within max-abs 2e-2 / mean-abs 2e-3, base-two
LSE within 2e-3; the paging error contract bit for bit."""
import numpy as np
import pytest
import torch

import oracle
from singe_amd import _native, error, neural

pytestmark = pytest.mark.gpu

MAX_ABS, MEAN_ABS, LSE_ABS = 2e-2, 2e-3, 2e-3


def layout(sequences, page_size, extra_pages=3):
    query_offsets, page_offsets, last, needed = [0], [0], [], 0
    for queries, keys in sequences:
        query_offsets.append(query_offsets[-1] + queries)
        pages = (keys + page_size - 1) // page_size
        needed += pages
        page_offsets.append(needed)
        last.append(0 if keys == 0 else keys - (pages - 1) * page_size)
    page_count = needed + extra_pages
    table = [(p * 7 + 2) % page_count for p in range(needed)] if np.gcd(7, page_count) == 1 else \
        list(np.random.default_rng(page_count).permutation(page_count)[:needed])
    return query_offsets, page_offsets, table, last, page_count


def run_case(sequences, heads, kv_heads, page_size, options, index_dtype=torch.int32, seed=0, dim=128):
    query_offsets, page_offsets, table, last, page_count = layout(sequences, page_size)
    tokens = query_offsets[-1]
    gen = torch.Generator(device="cuda")
    gen.manual_seed(seed)
    q = torch.randn((tokens, heads, dim), generator=gen, device="cuda").to(torch.bfloat16)
    kc = torch.randn((page_count, page_size, kv_heads, dim), generator=gen, device="cuda").to(torch.bfloat16)
    vc = torch.randn((page_count, page_size, kv_heads, dim), generator=gen, device="cuda").to(torch.bfloat16)
    index = lambda values: torch.tensor(values, dtype=index_dtype, device="cuda")
    paging = neural.Paging(index(query_offsets), index(page_offsets), index(table), index(last))
    out, lse = neural.paged_attention(q, kc, vc, paging, options)
    torch.cuda.synchronize()
    status, want, want_lse = oracle.paged_attention_f32(
        q.float().cpu().numpy(), kc.float().cpu().numpy(), vc.float().cpu().numpy(), query_offsets, page_offsets, table,
        last, scale=options.scale, causal=options.causal, window=options.window, softcap=options.softcap, threads=8)
    assert status == 0
    got, got_lse = out.float().cpu().numpy(), lse.cpu().numpy()
    assert np.isfinite(got).all()
    gap = np.abs(got - want)
    assert gap.max() <= MAX_ABS, gap.max()
    assert gap.mean() <= MEAN_ABS, gap.mean()
    empty = np.isneginf(want_lse)
    assert np.array_equal(np.isneginf(got_lse), empty)
    assert not got[empty].any()
    assert np.abs(got_lse[~empty] - want_lse[~empty]).max(initial=0.0) <= LSE_ABS


OPTIONS = [neural.AttentionOptions(), neural.AttentionOptions(causal=True),
           neural.AttentionOptions(causal=True, window=16, softcap=30.0),
           neural.AttentionOptions(causal=True, window=100), neural.AttentionOptions(scale=0.05, softcap=5.0)]


@pytest.mark.parametrize("options", OPTIONS)
@pytest.mark.parametrize("heads,kv_heads,page_size", [(8, 2, 1), (8, 1, 16), (4, 4, 7), (64, 8, 16), (8, 2, 8), (8, 2, 32),
                                                      (4, 1, 64), (8, 2, 128), (6, 3, 48)])
def test_ragged_sequences_match_oracle(heads, kv_heads, page_size, options):
    # decode, full prefill, chunked prefill, no keys (kernel_plan/source/tests.rs:830-889), plus more
    # queries than keys, where the CPU path's saturating position applies
    sequences = [(1, 150), (70, 70), (20, 90), (3, 0), (9, 4), (130, 300)]
    run_case(sequences, heads, kv_heads, page_size, options, seed=heads + page_size)


@pytest.mark.parametrize("index_dtype", [torch.int32, torch.int64])
@pytest.mark.parametrize("heads,kv_heads,page_size,splits", [(8, 2, 16, 0), (4, 4, 16, 0), (16, 1, 8, 3)])
def test_many_ragged_sequences_find_their_row_tiles(heads, kv_heads, page_size, splits, index_dtype):
    # more sequences than one wave's prefix sum covers (64), some without queries, some without keys, query
    # counts from under one row tile to several
    rng = np.random.default_rng(heads * 31 + page_size)
    sequences = []
    for s in range(150):
        queries = int(rng.choice([0, 1, 1, 2, 5, 17, 31, 32, 33, 64, 100, 129, 200]))
        keys = 0 if s % 23 == 7 else queries + int(rng.integers(0, 120))
        sequences.append((queries, keys))
    _native.lib().singe_hip_set_paged_attention_splits(splits)
    try:
        run_case(sequences, heads, kv_heads, page_size, neural.AttentionOptions(causal=True), index_dtype=index_dtype, seed=heads)
        run_case(sequences[:70], heads, kv_heads, page_size, neural.AttentionOptions(window=40, causal=True), index_dtype=index_dtype, seed=3)
    finally:
        _native.lib().singe_hip_set_paged_attention_splits(0)


@pytest.mark.parametrize("index_dtype", [torch.int32, torch.int64])
@pytest.mark.parametrize("heads,kv_heads,page_size,splits", [(8, 2, 16, 0), (16, 1, 8, 2), (4, 4, 3, 0)])
def test_up_to_64_sequences_with_tiles_to_spare_are_taken_longest_first(heads, kv_heads, page_size, splits, index_dtype):
    # few sequences with several row tiles each: the grid lists them by pages held, longest first, ties by index;
    # equal lengths, sequences without queries or without keys, and one much longer than the rest
    groups = heads // kv_heads
    base = 128 // groups  # queries of one row tile
    sequences = [(3 * base, 700), (3 * base, 700), (0, 300), (5 * base + 1, 5 * base + 1), (2 * base, 0), (base, 2000),
                 (4 * base, 700), (1, 64), (6 * base, 1100), (2 * base + 7, 333)]
    assert sum(q for q, _ in sequences) * groups // 128 >= 2 * len(sequences)
    _native.lib().singe_hip_set_paged_attention_splits(splits)
    try:
        run_case(sequences, heads, kv_heads, page_size, neural.AttentionOptions(causal=True), index_dtype=index_dtype, seed=heads + 9)
        run_case(sequences[::-1], heads, kv_heads, page_size, neural.AttentionOptions(causal=True, window=90), index_dtype=index_dtype, seed=2)
        run_case(sequences * 6, heads, kv_heads, page_size, neural.AttentionOptions(causal=True), index_dtype=index_dtype, seed=5)  # 60 of them
    finally:
        _native.lib().singe_hip_set_paged_attention_splits(0)


@pytest.mark.parametrize("options", [neural.AttentionOptions(causal=True, softcap=-4.0), neural.AttentionOptions(scale=-0.06, softcap=5.0),
                                     neural.AttentionOptions(scale=-0.06, softcap=-5.0, causal=True, window=50)])
@pytest.mark.parametrize("heads,kv_heads,page_size", [(8, 2, 16), (4, 4, 7)])
def test_negative_caps_and_scales(heads, kv_heads, page_size, options):
    # cap * tanh(score / cap) does not care about the sign of the cap; a negative scale turns the scores round
    run_case([(1, 150), (70, 70), (20, 90)], heads, kv_heads, page_size, options, seed=heads)


@pytest.mark.parametrize("options", [neural.AttentionOptions(causal=True, window=300), neural.AttentionOptions(causal=True, window=200, softcap=8.0),
                                     neural.AttentionOptions(causal=True, window=64), neural.AttentionOptions(causal=True, softcap=6.0),
                                     neural.AttentionOptions(window=500), neural.AttentionOptions(softcap=3.0, scale=-0.05)])
@pytest.mark.parametrize("heads,kv_heads,page_size", [(8, 2, 16), (4, 4, 16), (16, 1, 5)])
def test_long_windows_and_caps(heads, kv_heads, page_size, options):
    """Sequences long enough that a wave meets tiles reaching back past the window, tiles wholly inside it (which,
    like the capped ones, take the straight-line path) and tiles on the causal edge."""
    run_case([(300, 1100), (700, 700), (1, 1300), (40, 64)], heads, kv_heads, page_size, options, seed=heads + 3)


def test_int64_indices_and_chunked_prefill_shape():
    # one sequence of the chunked-prefill shape: 512 new queries over a cached prefix, 64 query / 8 kv heads
    run_case([(512, 1536 + 512), (512, 1024 + 512)], 64, 8, 16, neural.AttentionOptions(causal=True),
             index_dtype=torch.int64, seed=4)


@pytest.mark.parametrize("rows_per_wave", [0, 64])
def test_a_bad_page_in_a_large_page_table_is_refused_and_the_rest_is_right(rows_per_wave):
    """Page sizes of 16 keys and more look their pages up on the scalar unit (the two-tile kernel: in the lanes that
    fetched them): the same error contract."""
    _native.lib().singe_hip_set_paged_attention_rows_per_wave(rows_per_wave)
    try:
        a_bad_page_is_refused_and_the_rest_is_right()
    finally:
        _native.lib().singe_hip_set_paged_attention_rows_per_wave(0)


def a_bad_page_is_refused_and_the_rest_is_right():
    gen = torch.Generator(device="cuda")
    gen.manual_seed(8)
    q = torch.randn((40, 4, 128), generator=gen, device="cuda").to(torch.bfloat16)
    cache = torch.randn((6, 32, 2, 128), generator=gen, device="cuda").to(torch.bfloat16)
    index = lambda v: torch.tensor(v, dtype=torch.int32, device="cuda")
    good = neural.Paging(index([0, 20, 40]), index([0, 3, 5]), index([4, 1, 0, 2, 5]), index([7, 32]))
    want, _ = neural.paged_attention(q, cache, cache, good, neural.AttentionOptions(causal=True))
    bad = neural.Paging(index([0, 20, 40]), index([0, 3, 5]), index([4, 1, 0, 2, 6]), index([7, 32]))  # page 6 of 6
    status = torch.zeros(1, dtype=torch.int32, device="cuda")
    got, _ = neural.paged_attention(q, cache, cache, bad, neural.AttentionOptions(causal=True), status=status, check=False)
    assert status.item() == 1
    assert torch.equal(got[:20], want[:20])  # the sequence with good pages is untouched by its neighbour's error
    with pytest.raises(error.IndexOutOfBounds):
        neural.paged_attention(q, cache, cache, bad, neural.AttentionOptions(causal=True))


TOKENS, HEADS, DIM, SLOTS, PAGES = 2, 2, 128, 4, 2
VALID = dict(query_offsets=[0, 2], page_offsets=[0, 1], pages=[0], last_page_lengths=[2])
INVALID = [dict(query_offsets=[0, 3]), dict(query_offsets=[-1, 2]), dict(query_offsets=[2, 0]), dict(page_offsets=[0, 2]),
           dict(page_offsets=[-1, 1]), dict(pages=[PAGES]), dict(pages=[-1]), dict(last_page_lengths=[SLOTS + 1]),
           dict(last_page_lengths=[-1])]


def attend(paging_values, dtype=torch.int64):
    # singe/tests/nn/paged_attention.rs:96-127 (head_dim 128 here: the width this build's kernel takes)
    q = torch.zeros((TOKENS, HEADS, DIM), device="cuda", dtype=torch.bfloat16)
    cache = torch.zeros((PAGES, SLOTS, HEADS, DIM), device="cuda", dtype=torch.bfloat16)
    values = {**VALID, **paging_values}
    index = lambda v: torch.tensor(v, dtype=dtype, device="cuda")
    paging = neural.Paging(index(values["query_offsets"]), index(values["page_offsets"]), index(values["pages"]),
                           index(values["last_page_lengths"]))
    return neural.paged_attention(q, cache, cache, paging, neural.AttentionOptions(causal=True))


@pytest.mark.parametrize("dtype", [torch.int32, torch.int64])
def test_paging_values_outside_their_buffers_are_refused(dtype):
    # singe/tests/nn/paged_attention.rs:24-73, 141-186
    attend({}, dtype)
    for bad in INVALID:
        with pytest.raises(error.IndexOutOfBounds):
            attend(bad, dtype)
        attend({}, dtype)  # the next valid launch succeeds
    attend(dict(last_page_lengths=[SLOTS]), dtype)
    attend(dict(query_offsets=[0, 0], page_offsets=[0, 0], pages=[PAGES + 7], last_page_lengths=[-1]), dtype)
    for bad in INVALID:
        assert oracle.check_paged_values(**{**VALID, **bad}, tokens=TOKENS, cache_pages=PAGES, page_size=SLOTS) == 1


def test_paged_equals_dense_prefill():
    # paged == dense invariant (singe/tests/nn/cross_attention.rs:120-198): one sequence whose queries
    # are all of its tokens is plain causal attention over the gathered keys.
    from singe_amd.kernel import attention as A

    length, heads, kv_heads, page_size, dim = 300, 8, 2, 16, 128
    query_offsets, page_offsets, table, last, page_count = layout([(length, length)], page_size)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(12)
    q = torch.randn((length, heads, dim), generator=gen, device="cuda").to(torch.bfloat16)
    kc = torch.randn((page_count, page_size, kv_heads, dim), generator=gen, device="cuda").to(torch.bfloat16)
    vc = torch.randn((page_count, page_size, kv_heads, dim), generator=gen, device="cuda").to(torch.bfloat16)
    index = lambda v: torch.tensor(v, dtype=torch.int32, device="cuda")
    out, lse = neural.paged_attention(q, kc, vc, neural.Paging(index(query_offsets), index(page_offsets), index(table), index(last)),
                                      neural.AttentionOptions(causal=True))
    rows = torch.tensor([table[k // page_size] * page_size + k % page_size for k in range(length)], device="cuda")
    k_dense = kc.view(-1, kv_heads, dim)[rows].unsqueeze(0).contiguous()
    v_dense = vc.view(-1, kv_heads, dim)[rows].unsqueeze(0).contiguous()
    dense = torch.empty((1, length, heads, dim), device="cuda", dtype=torch.bfloat16)
    dense_lse = torch.empty((1, heads, length), device="cuda")
    A.fmha_prefill_lse_bf16(None, dense, dense_lse, q.unsqueeze(0).contiguous(), k_dense, v_dense,
                            A.FmhaPrefillConfig.contiguous(1, length, length, heads, kv_heads, dim, dim ** -0.5, True))
    torch.cuda.synchronize()
    assert (out.float() - dense[0].float()).abs().max().item() <= 2 ** -6
    assert (lse - dense_lse[0].T / np.log(2.0)).abs().max().item() <= 2e-3


@pytest.mark.parametrize("splits", [2, 3, 7, 16, 64])
@pytest.mark.parametrize("options", [neural.AttentionOptions(causal=True), neural.AttentionOptions(),
                                     neural.AttentionOptions(causal=True, window=100, softcap=20.0)])
def test_key_splits_match_oracle(splits, options):
    """With scratch lent, a row tile's keys are shared out over workgroups and merged by a second kernel: decode rows
    over long and short caches, a chunk, a sequence without keys, more shares than a sequence has tiles."""
    from singe_amd import _native
    _native.lib().singe_hip_set_paged_attention_splits(splits)
    try:
        run_case([(1, 1500), (1, 40), (5, 700), (2, 0), (1, 65), (130, 300)], 8, 2, 16, options, seed=splits)
        run_case([(1, 333), (3, 64)], 8, 1, 7, options, index_dtype=torch.int64, seed=splits + 1)
    finally:
        _native.lib().singe_hip_set_paged_attention_splits(0)


def test_decode_shaped_calls_split_on_their_own_and_agree_with_the_unsplit_kernel():
    gen = torch.Generator(device="cuda")
    gen.manual_seed(21)
    lens = [4096, 512, 1000, 2047, 16, 3000, 1, 777]
    pages_of = [(n + 15) // 16 for n in lens]
    page_count = sum(pages_of) + 5
    q = torch.randn((len(lens), 32, 128), generator=gen, device="cuda").to(torch.bfloat16)
    kc = torch.randn((page_count, 16, 8, 128), generator=gen, device="cuda").to(torch.bfloat16)
    vc = torch.randn((page_count, 16, 8, 128), generator=gen, device="cuda").to(torch.bfloat16)
    index = lambda values: torch.tensor(values, dtype=torch.int32, device="cuda")
    table = np.random.default_rng(3).permutation(page_count)[:sum(pages_of)]
    paging = neural.Paging(index(list(range(len(lens) + 1))), index(np.concatenate([[0], np.cumsum(pages_of)])), index(table),
                           index([n - (p - 1) * 16 for n, p in zip(lens, pages_of)]))
    apart, apart_lse = neural.paged_attention(q, kc, vc, paging, neural.AttentionOptions(causal=True), scratch=False)
    split, split_lse = neural.paged_attention(q, kc, vc, paging, neural.AttentionOptions(causal=True))
    assert (apart.float() - split.float()).abs().max().item() <= 4e-3
    assert (apart_lse - split_lse).abs().max().item() <= 1e-3


def test_a_stream_that_is_not_torchs_current_one_orders_the_fills_and_the_status_word():
    """The wrapper fills the output, the log-sum-exp and the status word and reads the word back: all of it has to
    run on the stream the kernel is launched on, also when that is not torch's current stream.  The current stream
    is kept busy meanwhile, so work queued on it by mistake would land after the kernel's."""
    gen = torch.Generator(device="cuda")
    gen.manual_seed(9)
    q = torch.randn((40, 4, 128), generator=gen, device="cuda").to(torch.bfloat16)
    cache = torch.randn((6, 32, 2, 128), generator=gen, device="cuda").to(torch.bfloat16)
    index = lambda v: torch.tensor(v, dtype=torch.int32, device="cuda")
    good = neural.Paging(index([0, 20, 40]), index([0, 3, 5]), index([4, 1, 0, 2, 5]), index([7, 32]))
    bad = neural.Paging(index([0, 20, 40]), index([0, 3, 5]), index([4, 1, 0, 2, 6]), index([7, 32]))
    want, want_lse = neural.paged_attention(q, cache, cache, good, neural.AttentionOptions(causal=True))
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    busy = torch.randn((4096, 4096), device="cuda")
    for _ in range(3):
        for _ in range(20):
            busy = busy @ busy * 1e-3  # the current stream stays busy while the side stream works
        got, got_lse = neural.paged_attention(q, cache, cache, good, neural.AttentionOptions(causal=True), stream=side)
        side.synchronize()
        assert torch.equal(got, want) and torch.equal(got_lse, want_lse)
        with pytest.raises(error.IndexOutOfBounds):
            neural.paged_attention(q, cache, cache, bad, neural.AttentionOptions(causal=True), stream=side)
    torch.cuda.synchronize()


# A decode step (no more tokens than sequences, no window or cap) runs on the block-table decode kernels,
# token by token: (queries, keys) per sequence.
DECODE_STEPS = [
    [(1, 700), (1, 1), (1, 4096), (1, 33), (1, 16), (1, 2049), (1, 5003)], # a token a sequence, ragged
    [(1, 300), (0, 500), (1, 0), (1, 64), (0, 0), (1, 1500)],             # sequences without a token, a token without keys
    [(2, 2900), (0, 40), (1, 17), (0, 2000)],                             # two tokens of one sequence, as many tokens as sequences
    [(3, 2), (0, 5), (0, 7), (1, 129)],                                   # more queries than keys
    [(1, 128 * (b % 5) + b) for b in range(1, 70)],                       # more sequences than a wave has lanes
]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("heads, kv_heads, page_size, dim", [(8, 2, 16, 128), (32, 4, 8, 128), (16, 1, 64, 128), (4, 4, 1, 128), (8, 2, 32, 64), (6, 1, 7, 64)])
@pytest.mark.parametrize("step", range(len(DECODE_STEPS)))
@pytest.mark.parametrize("index_dtype", [torch.int32, torch.int64])
def test_a_decode_step_through_the_op_matches_the_oracle_and_the_row_tile_kernel(step, heads, kv_heads, page_size, dim, dtype, index_dtype):
    import ctypes
    sequences = DECODE_STEPS[step]
    query_offsets, page_offsets, table, last, page_count = layout(sequences, page_size)
    tokens = query_offsets[-1]
    gen = torch.Generator(device="cuda")
    gen.manual_seed(100 * step + heads)
    rand = lambda *shape: torch.randn(shape, generator=gen, device="cuda").to(dtype)
    q, kc, vc = rand(tokens, heads, dim), rand(page_count, page_size, kv_heads, dim), rand(page_count, page_size, kv_heads, dim)
    index = lambda values: torch.tensor(values, dtype=index_dtype, device="cuda")
    paging = neural.Paging(index(query_offsets), index(page_offsets), index(table), index(last))
    # (windows from 2048 keys on take the decode kernels too: whole pages before the window are left out of a token's row,
    # the keys of its first page before the window are masked; shorter ones stay on the row-tile kernel)
    windows = (neural.AttentionOptions(causal=True, window=2048), neural.AttentionOptions(causal=True, window=2500), neural.AttentionOptions(window=2077),
               neural.AttentionOptions(causal=True, window=100), neural.AttentionOptions(causal=True, window=1 << 40))
    for options in (neural.AttentionOptions(causal=True), neural.AttentionOptions(scale=0.05)) + (windows if dtype == torch.bfloat16 else ()):
        # the scratch the op asks for covers the decode kernels' rows and partials
        problem = neural._problem(q, kc, vc, paging, options)
        if options.window is None or options.window >= 2048:
            assert _native.lib().singe_hip_paged_attention_scratch_bytes(ctypes.byref(problem)) >= 2 * 256 + 4 * tokens * heads * (dim + 1)
        out, lse = neural.paged_attention(q, kc, vc, paging, options)
        tiled, tiled_lse = neural.paged_attention(q, kc, vc, paging, options, scratch=False)
        torch.cuda.synchronize()
        status, want, want_lse = oracle.paged_attention_f32(q.float().cpu().numpy(), kc.float().cpu().numpy(), vc.float().cpu().numpy(), query_offsets,
                                                            page_offsets, table, last, scale=options.scale, causal=options.causal,
                                                            window=options.window, threads=8)
        assert status == 0
        got, got_lse = out.float().cpu().numpy(), lse.cpu().numpy()
        gap = np.abs(got - want)
        assert gap.max() <= MAX_ABS and gap.mean() <= MEAN_ABS, (options, gap.max(), gap.mean())
        empty = np.isneginf(want_lse)
        assert np.array_equal(np.isneginf(got_lse), empty) and not got[empty].any(), options
        assert np.abs(got_lse[~empty] - want_lse[~empty]).max(initial=0.0) <= LSE_ABS
        assert (out.float() - tiled.float()).abs().max().item() <= 8e-3
        assert np.array_equal(np.isneginf(tiled_lse.cpu().numpy()), empty)


@pytest.mark.parametrize("index_dtype", [torch.int32, torch.int64])
def test_a_decode_step_keeps_the_error_contract_and_leaves_unowned_tokens_alone(index_dtype):
    gen = torch.Generator(device="cuda")
    gen.manual_seed(4)
    q = torch.randn((3, 4, 128), generator=gen, device="cuda").to(torch.bfloat16)
    cache = torch.randn((6, 16, 2, 128), generator=gen, device="cuda").to(torch.bfloat16)
    index = lambda v: torch.tensor(v, dtype=index_dtype, device="cuda")
    options = neural.AttentionOptions(causal=True)
    good = neural.Paging(index([0, 1, 2, 3]), index([0, 2, 3, 5]), index([4, 1, 0, 2, 5]), index([7, 16, 3]))
    want, want_lse = neural.paged_attention(q, cache, cache, good, options)
    for pages, last in (([4, 1, 0, 2, 6], [7, 16, 3]), ([4, 1, 0, -1, 5], [7, 16, 3]), ([4, 1, 0, 2, 5], [7, 16, 17])):
        bad = neural.Paging(index([0, 1, 2, 3]), index([0, 2, 3, 5]), index(pages), index(last))
        status = torch.zeros(1, dtype=torch.int32, device="cuda")
        got, got_lse = neural.paged_attention(q, cache, cache, bad, options, status=status, check=False)
        assert status.item() == 1
        assert torch.equal(got[:2], want[:2]) and torch.equal(got_lse[:2], want_lse[:2])  # the sequences with good paging are right
        with pytest.raises(error.IndexOutOfBounds):
            neural.paged_attention(q, cache, cache, bad, options)
    # a page id outside the cache that no sequence with a token reads is not looked at
    unread = neural.Paging(index([0, 1, 2, 2]), index([0, 2, 3, 5]), index([4, 1, 0, 77, -3]), index([7, 16, 3]))
    got, _ = neural.paged_attention(q[:2], cache, cache, unread, options)
    assert torch.equal(got, want[:2])
    # tokens before the first sequence's and after the last one's belong to nobody: their rows stay as they were
    edges = neural.Paging(index([1, 2, 2, 2]), index([0, 2, 3, 3]), index([4, 1, 0]), index([7, 16, 0]))
    got, got_lse = neural.paged_attention(q, cache, cache, edges, options)
    tiled, tiled_lse = neural.paged_attention(q, cache, cache, edges, options, scratch=False)
    assert (got[1].float() - tiled[1].float()).abs().max().item() <= 8e-3 and (got_lse[1] - tiled_lse[1]).abs().max().item() <= 2e-3
    assert not got[0].any() and not got[2].any() and torch.isneginf(got_lse[0]).all() and torch.isneginf(got_lse[2]).all()


@pytest.mark.parametrize("count, heads, kv_heads", [(7900, 4, 2), (3000, 16, 2), (2300, 16, 2)])
def test_a_decode_step_of_thousands_of_sequences(count, heads, kv_heads):
    """The decode kernels keep three words a token in LDS on this route: 7900 tokens fill it beside the one-hot form's
    staging; with eight heads a kv head 3000 tokens no longer fit beside the dense form's and take the one-hot form, 2300 do."""
    rng = np.random.default_rng(count)
    sequences = [(1, int(n)) for n in rng.integers(0, 40, count)]
    query_offsets, page_offsets, table, last, page_count = layout(sequences, 16)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(count)
    rand = lambda *shape: torch.randn(shape, generator=gen, device="cuda").to(torch.bfloat16)
    q, kc, vc = rand(count, heads, 128), rand(page_count, 16, kv_heads, 128), rand(page_count, 16, kv_heads, 128)
    index = lambda values: torch.tensor(values, dtype=torch.int64, device="cuda")
    paging = neural.Paging(index(query_offsets), index(page_offsets), index(table), index(last))
    out, lse = neural.paged_attention(q, kc, vc, paging, neural.AttentionOptions(causal=True))
    torch.cuda.synchronize()
    status, want, want_lse = oracle.paged_attention_f32(q.float().cpu().numpy(), kc.float().cpu().numpy(), vc.float().cpu().numpy(), query_offsets,
                                                        page_offsets, table, last, causal=True, threads=8)
    assert status == 0
    gap = np.abs(out.float().cpu().numpy() - want)
    assert gap.max() <= MAX_ABS and gap.mean() <= MEAN_ABS, (gap.max(), gap.mean())
    empty = np.isneginf(want_lse)
    assert np.array_equal(np.isneginf(lse.cpu().numpy()), empty)
    assert np.abs(lse.cpu().numpy()[~empty] - want_lse[~empty]).max() <= LSE_ABS


@pytest.fixture
def two_tiles_a_wave():
    """Sends every paged call that has the form to the kernel that gives a wave two 32-row tiles."""
    _native.lib().singe_hip_set_paged_attention_rows_per_wave(64)
    yield
    _native.lib().singe_hip_set_paged_attention_rows_per_wave(0)


@pytest.mark.parametrize("index_dtype", [torch.int32, torch.int64])
@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("heads,kv_heads,page_size,dim", [(8, 1, 16, 128), (64, 8, 16, 128), (8, 2, 32, 128), (4, 1, 64, 128), (8, 2, 128, 128),
                                                          (4, 4, 16, 128), (8, 1, 16, 64), (64, 8, 16, 64), (8, 2, 64, 64), (4, 4, 32, 64),
                                                          (8, 1, 16, 96), (64, 8, 16, 96), (8, 2, 64, 96), (4, 4, 32, 96),
                                                          (8, 1, 16, 112), (8, 2, 64, 112), (64, 8, 16, 80), (4, 4, 32, 80), (8, 1, 16, 48),
                                                          (8, 2, 128, 48), (64, 8, 16, 32), (4, 1, 64, 32), (8, 2, 16, 16), (4, 4, 256, 16)])
def test_two_tiles_a_wave_ragged_sequences_match_oracle(two_tiles_a_wave, heads, kv_heads, page_size, dim, causal, index_dtype):
    # the shapes of the ragged test (decode, full prefill, chunked prefill, no keys, more queries than keys) and
    # chunks long enough for several 256-row tiles, several key tiles ahead of the mask and key counts either side of
    # a tile's and a page's end
    sequences = [(1, 150), (70, 70), (20, 90), (3, 0), (9, 4), (130, 300), (300, 1000), (257, 513), (64, 1024), (512, 512)]
    run_case(sequences, heads, kv_heads, page_size, neural.AttentionOptions(causal=causal), index_dtype=index_dtype,
             seed=heads + page_size + 1, dim=dim)


def test_two_tiles_a_wave_equals_the_four_wave_kernel_at_the_chunked_prefill_shape():
    # The fourth benchmark configuration fills the chip with 256-row tiles, so the default choice is this kernel: its
    # answer against the 32-row kernel's, within the rounding of the output.
    from singe_amd import synthetic
    work = synthetic.chunked_prefill_workload(portable=True)
    index = lambda values: torch.from_numpy(np.asarray(values, dtype=np.int32)).cuda()
    paging = neural.Paging(index(work.query_offsets), index(work.page_offsets), index(work.pages), index(work.last_page_lengths))
    options = neural.AttentionOptions(causal=True)
    chosen, chosen_lse = neural.paged_attention(work.query, work.key_cache, work.value_cache, paging, options)
    _native.lib().singe_hip_set_paged_attention_rows_per_wave(32)
    try:
        narrow, narrow_lse = neural.paged_attention(work.query, work.key_cache, work.value_cache, paging, options)
    finally:
        _native.lib().singe_hip_set_paged_attention_rows_per_wave(0)
    torch.cuda.synchronize()
    assert (chosen.float() - narrow.float()).abs().max().item() <= 2 ** -6
    assert (chosen_lse - narrow_lse).abs().max().item() <= 1e-4


@pytest.mark.parametrize("rows_per_wave", [64, 32])
@pytest.mark.parametrize("index_dtype", [torch.int32, torch.int64])
def test_pages_beyond_two_and_four_gib_of_a_cache_read_the_same_as_the_first_pages(rows_per_wave, index_dtype):
    # 150 000 pages of 32 KiB: a page's first byte lies past 2^31 from id 65 536 and past 2^32 from id 131 072.  The
    # same page contents under small ids in a small cache must give the same bits.
    heads, kv_heads, page_size, cache_pages = 32, 8, 16, 150_000
    sequences = [(300, 700), (256, 512)]
    gen = torch.Generator(device="cuda")
    gen.manual_seed(77)
    page_counts = [-(-keys // page_size) for _, keys in sequences]
    used = sum(page_counts)
    high = torch.tensor([65_536 + 3, 131_072 + 5, cache_pages - 1, 70_001, 140_002, 100_000], dtype=torch.int64)
    ids_high = torch.cat([high, 90_000 + 7 * torch.arange(used - len(high))])
    ids_low = torch.randperm(used)
    small_k = torch.randn((used, page_size, kv_heads, 128), generator=gen, device="cuda").to(torch.bfloat16)
    small_v = torch.randn((used, page_size, kv_heads, 128), generator=gen, device="cuda").to(torch.bfloat16)
    big_k = torch.zeros((cache_pages, page_size, kv_heads, 128), device="cuda", dtype=torch.bfloat16)
    big_v = torch.zeros((cache_pages, page_size, kv_heads, 128), device="cuda", dtype=torch.bfloat16)
    big_k[ids_high.cuda()] = small_k[ids_low.cuda()]
    big_v[ids_high.cuda()] = small_v[ids_low.cuda()]
    tokens = sum(queries for queries, _ in sequences)
    q = torch.randn((tokens, heads, 128), generator=gen, device="cuda").to(torch.bfloat16)
    query_offsets = np.concatenate([[0], np.cumsum([queries for queries, _ in sequences])])
    page_offsets = np.concatenate([[0], np.cumsum(page_counts)])
    last = [keys - (count - 1) * page_size for (_, keys), count in zip(sequences, page_counts)]
    index = lambda values: torch.as_tensor(np.asarray(values), dtype=index_dtype).cuda()
    options = neural.AttentionOptions(causal=True)
    _native.lib().singe_hip_set_paged_attention_rows_per_wave(rows_per_wave)
    try:
        far, far_lse = neural.paged_attention(q, big_k, big_v, neural.Paging(index(query_offsets), index(page_offsets), index(ids_high.numpy()), index(last)), options)
        near, near_lse = neural.paged_attention(q, small_k, small_v, neural.Paging(index(query_offsets), index(page_offsets), index(ids_low.numpy()), index(last)), options)
    finally:
        _native.lib().singe_hip_set_paged_attention_rows_per_wave(0)
    torch.cuda.synchronize()
    assert torch.equal(far, near) and torch.equal(far_lse, near_lse)
    assert far.float().abs().max().item() > 0.1
