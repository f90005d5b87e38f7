"""The attention entry points only enqueue work on the caller's stream (the contract of the reference's launchers,
singe-kernel/src/cuda/mod.rs:3-12: legal under stream capture).  Each op is recorded into a HIP graph on a side stream
and replayed several times; between the replays the CONTENTS of its inputs change (lengths, tables, queries), with
eager launches and synchronisations in between, and every replay must give the bits of an eager launch on the same
inputs.  One case per op is also held to the oracle, so the eager side of the comparison is pinned too."""
import ctypes

import numpy as np
import pytest
import torch

import oracle
from singe_amd import _native, neural, synthetic
from singe_amd.kernel import attention as A

pytestmark = pytest.mark.gpu


def _bits(tensor):
    return tensor.contiguous().view(torch.int16 if tensor.element_size() == 2 else torch.int32)


def _replays_equal_eager(run, changes, outputs):
    """run(stream) enqueues the op; changes rewrite its inputs in place, one per replay."""
    changes[0]()
    run(None)  # eager once: whatever the library sets up on first use happens outside the capture
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        run(torch.cuda.current_stream())
    for number, change in enumerate(changes):
        print(f"graph replay {number}", flush=True)
        change()
        for output in outputs:
            output.fill_(float("nan"))
        run(None)
        torch.cuda.synchronize()
        want = [output.clone() for output in outputs]
        for output in outputs:
            output.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for expected, output in zip(want, outputs):
            assert torch.equal(_bits(expected), _bits(output)), f"replay {number} differs from the eager launch"
    return want


def _decode_case(fp8=False):
    lengths = [[700, 33, 0, 1500, 64, 257], [1, 1499, 800, 16, 0, 31], [1500, 1500, 1500, 1500, 1500, 1500]]
    make = synthetic.paged_decode_fp8_workload if fp8 else synthetic.paged_decode_workload
    work = make(batch=6, heads=32, kv_heads=8, physical_blocks=1024, seq_lens=[1500] * 6, seed=11)
    config = A.PagedKvDecodeAttentionConfig.contiguous(work.batch, work.heads, work.kv_heads, work.head_dim, work.block_size,
                                                       work.physical_blocks, work.block_table_batch_stride, work.scale)
    lens = torch.from_numpy(work.seq_lens).cuda()
    table = torch.from_numpy(work.block_table.view(np.int32)).cuda()
    out = torch.empty((work.batch, work.heads, work.head_dim), device="cuda", dtype=torch.bfloat16)
    queries = [torch.randn(work.query.shape, device="cuda", generator=torch.Generator("cuda").manual_seed(40 + i)).to(torch.bfloat16)
               for i in range(len(lengths))]
    orders = [torch.randperm(work.batch, generator=torch.Generator().manual_seed(50 + i)).cuda() for i in range(len(lengths))]
    first_table = table.clone()

    def change(i):
        def apply():
            lens.copy_(torch.tensor(lengths[i], dtype=torch.int32))
            work.query.copy_(queries[i])
            table.copy_(first_table[orders[i]])  # sequences swap their page lists
        return apply

    return work, config, lens, table, out, [change(i) for i in range(len(lengths))], lengths, orders


def _decode_oracle(work, query, lens, table, cache=None):
    key_cache, value_cache = cache if cache is not None else (work.key_cache.float().cpu().numpy(), work.value_cache.float().cpu().numpy())
    return oracle.paged_kv_decode_attention_f32(
        query.float().cpu().numpy(), key_cache, value_cache, lens.cpu().numpy(), table.cpu().numpy().view(np.uint32),
        batch=work.batch, heads=work.heads, kv_heads=work.kv_heads, head_dim=work.head_dim, block_size=work.block_size,
        block_table_batch_stride=work.block_table_batch_stride, scale=work.scale, threads=8)


def test_decode_with_a_workspace_replays():
    work, config, lens, table, out, changes, _, _ = _decode_case()
    workspace = torch.empty(config.workspace_bytes(), dtype=torch.uint8, device="cuda")
    run = lambda stream: A.paged_kv_decode_attention_bf16(stream, out, work.query, work.key_cache, work.value_cache, lens, table,
                                                          config, workspace)
    (last,) = _replays_equal_eager(run, changes, [out])
    gap = np.abs(last.float().cpu().numpy() - _decode_oracle(work, work.query, lens, table))
    assert gap.max() <= 2e-2 and gap.mean() <= 2e-3, (gap.max(), gap.mean())


def test_decode_on_the_fixed_scratch_replays():
    work, config, lens, table, out, changes, _, _ = _decode_case()
    run = lambda stream: A.paged_kv_decode_attention_no_alloc_bf16(stream, out, work.query, work.key_cache, work.value_cache, lens,
                                                                   table, config)
    (last,) = _replays_equal_eager(run, changes, [out])
    gap = np.abs(last.float().cpu().numpy() - _decode_oracle(work, work.query, lens, table))
    assert gap.max() <= 2e-2 and gap.mean() <= 2e-3, (gap.max(), gap.mean())


def test_a_captured_decode_survives_the_module_scratch_growing():
    """A decode recorded without a workspace of its own holds a pointer to this layer's per-device scratch.  A bigger
    config that makes that scratch grow afterwards must not free what the graph points at: replays after the growth
    (and after eager calls on the new buffer) still match eager launches; and growing under capture is refused."""
    from singe_amd import error

    work, config, lens, table, out, changes, _, _ = _decode_case()
    config.reserve_workspace()
    run = lambda stream: A.paged_kv_decode_attention_bf16(stream, out, work.query, work.key_cache, work.value_cache, lens, table, config)
    changes[0]()
    run(None)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        run(torch.cuda.current_stream())
    held = A._workspaces.get(out.device, 1)

    # (earlier tests may have grown the module's scratch already: the bigger config is sized against what is held now)
    sized = lambda batch: A.PagedKvDecodeAttentionConfig.contiguous(batch, 32, 8, 128, 16, 4 * batch, 3, 0.1).workspace_bytes()
    many = 96
    while sized(many) <= held.numel():
        many *= 2
    big = synthetic.paged_decode_workload(batch=many, heads=32, kv_heads=8, physical_blocks=4 * many, seq_lens=[40] * many, seed=12)
    big_config = A.PagedKvDecodeAttentionConfig.contiguous(big.batch, big.heads, big.kv_heads, big.head_dim, big.block_size,
                                                           big.physical_blocks, big.block_table_batch_stride, big.scale)
    assert big_config.workspace_bytes() > held.numel()
    big_out = torch.empty((big.batch, big.heads, big.head_dim), device="cuda", dtype=torch.bfloat16)
    big_lens, big_table = torch.from_numpy(big.seq_lens).cuda(), torch.from_numpy(big.block_table.view(np.int32)).cuda()
    A.paged_kv_decode_attention_bf16(None, big_out, big.query, big.key_cache, big.value_cache, big_lens, big_table, big_config)
    torch.cuda.synchronize()
    grown = A._workspaces.get(out.device, 1)
    assert grown.data_ptr() != held.data_ptr() and grown.numel() >= big_config.workspace_bytes()
    filler = [torch.full((held.numel(),), 0xA5, dtype=torch.uint8, device="cuda") for _ in range(4)]  # would land on a freed buffer

    for number, change in enumerate(changes):
        print(f"graph replay {number} after the scratch grew", flush=True)
        change()
        workspace = torch.empty(config.workspace_bytes(), dtype=torch.uint8, device="cuda")
        out.fill_(float("nan"))
        A.paged_kv_decode_attention_bf16(None, out, work.query, work.key_cache, work.value_cache, lens, table, config, workspace)
        torch.cuda.synchronize()
        want = out.clone()
        out.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(_bits(want), _bits(out)), f"replay {number} differs from the eager launch"
    del filler

    other = torch.cuda.CUDAGraph()
    with pytest.raises(error.UnsupportedConfiguration):
        with torch.cuda.graph(other, stream=side):
            A._workspaces.get(out.device, grown.numel() + 1)


def test_fp8_decode_replays():
    work, config, lens, table, out, changes, _, _ = _decode_case(fp8=True)
    workspace = torch.empty(config.workspace_bytes(), dtype=torch.uint8, device="cuda")
    run = lambda stream: A.paged_kv_decode_attention_f8e4m3kv_bf16(stream, out, work.query, work.key_cache, work.value_cache,
                                                                   work.key_scales, work.value_scales, lens, table, config, workspace)
    _replays_equal_eager(run, changes, [out])


def test_block_table_prefill_replays():
    batch, heads, kv_heads, dim, block, blocks = 3, 8, 2, 128, 16, 256
    rng = np.random.default_rng(21)
    tokens = 3 * 96
    cases = [([96, 96, 96], [300, 96, 1000]), ([10, 180, 96], [10, 400, 97]), ([0, 96, 150], [55, 96, 150])]
    stride = 64
    table = torch.from_numpy(rng.permutation(blocks)[: batch * stride].reshape(batch, stride).astype(np.int32)).cuda()
    query = torch.randn((tokens, heads, dim), device="cuda").to(torch.bfloat16)
    key_cache = torch.randn((blocks, block, kv_heads, dim), device="cuda").to(torch.bfloat16)
    value_cache = torch.randn((blocks, block, kv_heads, dim), device="cuda").to(torch.bfloat16)
    q_lens = torch.zeros(batch, dtype=torch.int32, device="cuda")
    kv_lens = torch.zeros(batch, dtype=torch.int32, device="cuda")
    offsets = torch.zeros(batch, dtype=torch.int32, device="cuda")
    out = torch.empty_like(query)
    lse = torch.empty((tokens, heads), device="cuda", dtype=torch.float32)
    config = A.PagedKvPrefillAttentionConfig.contiguous(batch, tokens, heads, kv_heads, dim, block, blocks, stride, True,
                                                        float(1.0 / np.sqrt(dim)))

    def change(i):
        def apply():
            q, kv = cases[i]
            q_lens.copy_(torch.tensor(q, dtype=torch.int32))
            kv_lens.copy_(torch.tensor(kv, dtype=torch.int32))
            offsets.copy_(torch.tensor(np.concatenate([[0], np.cumsum(q)[:-1]]), dtype=torch.int32))
            query.copy_(torch.randn(query.shape, device="cuda", generator=torch.Generator("cuda").manual_seed(60 + i)).to(torch.bfloat16))
        return apply

    run = lambda stream: A.paged_kv_prefill_attention_bf16(stream, out, lse, query, key_cache, value_cache, q_lens, kv_lens, offsets,
                                                           table, config)
    # rows no sequence owns are not written: compare the owned rows only, which the NaN fill leaves recognisable
    changes = [change(i) for i in range(len(cases))]
    changes[0]()
    run(None)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        run(torch.cuda.current_stream())
    for number, apply in enumerate(changes):
        print(f"prefill graph replay {number}", flush=True)
        apply()
        out.fill_(float("nan"))
        lse.fill_(float("nan"))
        run(None)
        torch.cuda.synchronize()
        want_out, want_lse = out.clone(), lse.clone()
        out.fill_(float("nan"))
        lse.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(_bits(want_out), _bits(out)) and torch.equal(_bits(want_lse), _bits(lse))
        owned = sum(cases[number][0])
        assert torch.isfinite(out[:owned].float()).all()


@pytest.mark.parametrize("shares", [0, 4])
def test_paged_attention_with_key_splits_replays(shares):
    """The FlashInfer-form op in decode shape, by itself (the kernel that checks the paging vectors and gives every token
    its row, then the block-table decode kernels) and held to its row-tile kernel by a fixed number of shares (the
    attention kernel leaves partials in caller scratch and a second kernel merges them): every launch recorded."""
    _native.lib().singe_hip_set_paged_attention_splits(shares)
    try:
        _paged_attention_replays()
    finally:
        _native.lib().singe_hip_set_paged_attention_splits(0)


def _paged_attention_replays():
    sequences, heads, kv_heads, dim, page, cache_pages = 5, 32, 8, 128, 16, 640
    rng = np.random.default_rng(31)
    cases = [[900, 16, 2000, 333, 1], [2000, 2000, 2000, 2000, 2000], [17, 1999, 64, 0, 700]]
    capacity = 5 * 125
    query = torch.randn((sequences, heads, dim), device="cuda").to(torch.bfloat16)
    key_cache = torch.randn((cache_pages, page, kv_heads, dim), device="cuda").to(torch.bfloat16)
    value_cache = torch.randn((cache_pages, page, kv_heads, dim), device="cuda").to(torch.bfloat16)
    query_offsets = torch.arange(sequences + 1, dtype=torch.int32, device="cuda")
    page_offsets = torch.zeros(sequences + 1, dtype=torch.int32, device="cuda")
    pages = torch.zeros(capacity, dtype=torch.int32, device="cuda")
    last = torch.zeros(sequences, dtype=torch.int32, device="cuda")
    paging = neural.Paging(query_offsets, page_offsets, pages, last)
    problem = neural._problem(query, key_cache, value_cache, paging, neural.AttentionOptions(causal=True))
    out = torch.empty_like(query)
    lse = torch.empty((sequences, heads), device="cuda", dtype=torch.float32)
    status = torch.zeros(1, device="cuda", dtype=torch.int32)
    scratch_bytes = int(_native.lib().singe_hip_paged_attention_scratch_bytes(ctypes.byref(problem)))
    assert scratch_bytes > 0, "this shape is meant to take key splits"
    scratch = torch.empty(scratch_bytes, device="cuda", dtype=torch.uint8)

    def change(i):
        def apply():
            counts = [(n + page - 1) // page for n in cases[i]]
            page_offsets.copy_(torch.tensor(np.concatenate([[0], np.cumsum(counts)]), dtype=torch.int32))
            listed = np.zeros(capacity, dtype=np.int32)
            listed[: sum(counts)] = rng.permutation(cache_pages)[: sum(counts)]
            pages.copy_(torch.from_numpy(listed))
            last.copy_(torch.tensor([n - (c - 1) * page if c else 0 for n, c in zip(cases[i], counts)], dtype=torch.int32))
            query.copy_(torch.randn(query.shape, device="cuda", generator=torch.Generator("cuda").manual_seed(70 + i)).to(torch.bfloat16))
        return apply

    def run(stream):
        handle = int((stream or torch.cuda.current_stream()).cuda_stream)
        _native.check(_native.lib().singe_hip_paged_attention_scratch_bf16(
            handle, query.data_ptr(), key_cache.data_ptr(), value_cache.data_ptr(), query_offsets.data_ptr(), page_offsets.data_ptr(),
            pages.data_ptr(), last.data_ptr(), out.data_ptr(), lse.data_ptr(), status.data_ptr(), scratch.data_ptr(), scratch.numel(),
            ctypes.byref(problem)), "paged_attention")

    want_out, want_lse = _replays_equal_eager(run, [change(i) for i in range(len(cases))], [out, lse])
    assert int(status.item()) == 0
    # the last case against the oracle (base-two log-sum-exp, -inf for the sequence without keys)
    code, reference, reference_lse = oracle.paged_attention_f32(
        query.float().cpu().numpy(), key_cache.float().cpu().numpy(), value_cache.float().cpu().numpy(),
        query_offsets.cpu().numpy(), page_offsets.cpu().numpy(), pages.cpu().numpy(), last.cpu().numpy(), causal=True, threads=8)
    assert code == 0
    gap = np.abs(want_out.float().cpu().numpy() - reference)
    assert gap.max() <= 2e-2 and gap.mean() <= 2e-3, (gap.max(), gap.mean())
    live = np.isfinite(reference_lse)
    assert np.array_equal(live, np.isfinite(want_lse.cpu().numpy()))
    assert np.abs(want_lse.cpu().numpy()[live] - reference_lse[live]).max() <= 2e-3


@pytest.mark.parametrize("rows_per_wave,length", [(0, 320), (64, 320), (64, 417)])
def test_dense_prefill_replays(rows_per_wave, length):
    # (64 rows a wave: the kernel that gives a wave two 32-row tiles, with whole key tiles and with a last tile that is not)
    _native.lib().singe_hip_set_dense_prefill_rows_per_wave(rows_per_wave)
    try:
        _dense_prefill_replays(length)
    finally:
        _native.lib().singe_hip_set_dense_prefill_rows_per_wave(0)


def _dense_prefill_replays(length):
    batch, heads, kv_heads, dim = 2, 8, 2, 128
    query = torch.empty((batch, length, heads, dim), device="cuda", dtype=torch.bfloat16)
    key = torch.empty((batch, length, kv_heads, dim), device="cuda", dtype=torch.bfloat16)
    value = torch.empty_like(key)
    out = torch.empty_like(query)
    config = A.FmhaPrefillConfig.contiguous(batch, length, length, heads, kv_heads, dim, float(1.0 / np.sqrt(dim)), True)

    def change(i):
        def apply():
            generator = torch.Generator("cuda").manual_seed(80 + i)
            for tensor in (query, key, value):
                tensor.copy_(torch.randn(tensor.shape, device="cuda", generator=generator).to(torch.bfloat16))
        return apply

    run = lambda stream: A.fmha_prefill_bf16(stream, out, query, key, value, config)
    _replays_equal_eager(run, [change(i) for i in range(3)], [out])


def test_prefill_shaped_paged_attention_replays_on_the_two_tile_kernel():
    """Chunks of new tokens over cached prefixes, on the kernel that gives a wave two 32-row tiles: the page lists, the
    prefix lengths and the queries change between replays."""
    sequences, chunk, heads, kv_heads, dim, page, cache_pages = 3, 300, 16, 2, 128, 16, 400
    rng = np.random.default_rng(37)
    cases = [[700, 300, 1500], [300, 2000, 301], [1024, 513, 999]]  # keys of each sequence (its chunk included)
    capacity = 3 * 130
    query = torch.empty((sequences * chunk, heads, dim), device="cuda", dtype=torch.bfloat16)
    key_cache = torch.randn((cache_pages, page, kv_heads, dim), device="cuda").to(torch.bfloat16)
    value_cache = torch.randn((cache_pages, page, kv_heads, dim), device="cuda").to(torch.bfloat16)
    query_offsets = torch.arange(0, (sequences + 1) * chunk, chunk, dtype=torch.int32, device="cuda")
    page_offsets = torch.zeros(sequences + 1, dtype=torch.int32, device="cuda")
    pages = torch.zeros(capacity, dtype=torch.int32, device="cuda")
    last = torch.zeros(sequences, dtype=torch.int32, device="cuda")
    paging = neural.Paging(query_offsets, page_offsets, pages, last)
    problem = neural._problem(query, key_cache, value_cache, paging, neural.AttentionOptions(causal=True))
    out = torch.empty_like(query)
    lse = torch.empty((sequences * chunk, heads), device="cuda", dtype=torch.float32)
    status = torch.zeros(1, device="cuda", dtype=torch.int32)

    def change(i):
        def apply():
            counts = [(n + page - 1) // page for n in cases[i]]
            page_offsets.copy_(torch.tensor(np.concatenate([[0], np.cumsum(counts)]), dtype=torch.int32))
            listed = np.zeros(capacity, dtype=np.int32)
            listed[: sum(counts)] = rng.permutation(cache_pages)[: sum(counts)]
            pages.copy_(torch.from_numpy(listed))
            last.copy_(torch.tensor([n - (c - 1) * page for n, c in zip(cases[i], counts)], dtype=torch.int32))
            query.copy_(torch.randn(query.shape, device="cuda", generator=torch.Generator("cuda").manual_seed(90 + i)).to(torch.bfloat16))
        return apply

    def run(stream):
        handle = int((stream or torch.cuda.current_stream()).cuda_stream)
        _native.check(_native.lib().singe_hip_paged_attention_bf16(
            handle, query.data_ptr(), key_cache.data_ptr(), value_cache.data_ptr(), query_offsets.data_ptr(), page_offsets.data_ptr(),
            pages.data_ptr(), last.data_ptr(), out.data_ptr(), lse.data_ptr(), status.data_ptr(), ctypes.byref(problem)), "paged_attention")

    _native.lib().singe_hip_set_paged_attention_rows_per_wave(64)
    try:
        want_out, want_lse = _replays_equal_eager(run, [change(i) for i in range(len(cases))], [out, lse])
    finally:
        _native.lib().singe_hip_set_paged_attention_rows_per_wave(0)
    assert int(status.item()) == 0
    code, reference, reference_lse = oracle.paged_attention_f32(
        query.float().cpu().numpy(), key_cache.float().cpu().numpy(), value_cache.float().cpu().numpy(),
        query_offsets.cpu().numpy(), page_offsets.cpu().numpy(), pages.cpu().numpy(), last.cpu().numpy(), causal=True, threads=8)
    assert code == 0
    gap = np.abs(want_out.float().cpu().numpy() - reference)
    assert gap.max() <= 2e-2 and gap.mean() <= 2e-3, (gap.max(), gap.mean())
    assert np.abs(want_lse.cpu().numpy() - reference_lse).max() <= 2e-3
