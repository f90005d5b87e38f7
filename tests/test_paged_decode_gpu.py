"""Paged decode on the GPU against the CPU oracle, through the C ABI (ctypes -> libsinge_hip_attention.so
-> hipModuleLaunchKernel).  Tolerance for bf16 outputs: max-abs 2e-2 and mean-abs 2e-3 against the
oracle run on the same bf16-rounded inputs widened to f32; gather indices and lengths bit-exact."""
import math

import numpy as np
import pytest
import torch

import oracle
from singe_amd import error, synthetic
from singe_amd.kernel import attention as A

pytestmark = pytest.mark.gpu

MAX_ABS, MEAN_ABS = 2e-2, 2e-3


def compact(work):
    """The referenced blocks only, renumbered, as f32 on the host (the oracle is invariant under a
    permutation of physical blocks, which tests/test_oracle.py pins)."""
    counts = (work.seq_lens.astype(np.int64) + work.block_size - 1) // work.block_size
    used = np.concatenate([work.block_table[b, :n] for b, n in enumerate(counts)] + [np.zeros(0, np.uint32)]).astype(np.int64)
    if len(used) == 0:
        used = np.zeros(1, dtype=np.int64)
    remap = np.zeros(work.physical_blocks, dtype=np.uint32)
    remap[used] = np.arange(len(used), dtype=np.uint32)
    table = np.zeros_like(work.block_table)
    for b, n in enumerate(counts):
        table[b, :n] = remap[work.block_table[b, :n]]
    index = torch.from_numpy(used).to(work.key_cache.device)
    kc = work.key_cache[index].float().cpu().numpy()
    vc = work.value_cache[index].float().cpu().numpy()
    return kc, vc, table


def run_gpu(work, workers=0, dtype=torch.bfloat16):
    A._native.lib().singe_hip_set_decode_workers(workers)
    try:
        if dtype == torch.float16:
            config = A.PagedKvDecodeAttentionConfig.contiguous(work.batch, work.heads, work.kv_heads, work.head_dim,
                                                               work.block_size, work.physical_blocks,
                                                               work.block_table_batch_stride, work.scale)
            out = torch.full((work.batch, work.heads, work.head_dim), float("nan"), device="cuda", dtype=dtype)
            A.paged_kv_decode_attention_f16(None, out, work.query.to(dtype), work.key_cache.to(dtype), work.value_cache.to(dtype),
                                            torch.from_numpy(work.seq_lens).cuda(),
                                            torch.from_numpy(work.block_table.view(np.int32)).cuda(), config)
            torch.cuda.synchronize()
            return out.float().cpu().numpy()
        config = A.PagedKvDecodeAttentionConfig.contiguous(work.batch, work.heads, work.kv_heads, work.head_dim,
                                                           work.block_size, work.physical_blocks,
                                                           work.block_table_batch_stride, work.scale)
        out = torch.full((work.batch, work.heads, work.head_dim), float("nan"), device="cuda", dtype=torch.bfloat16)
        lens = torch.from_numpy(work.seq_lens).cuda()
        table = torch.from_numpy(work.block_table.view(np.int32)).cuda()
        A.paged_kv_decode_attention_bf16(None, out, work.query, work.key_cache, work.value_cache, lens, table, config)
        torch.cuda.synchronize()
    finally:
        A._native.lib().singe_hip_set_decode_workers(0)
    return out.float().cpu().numpy()


def run_oracle(work):
    kc, vc, table = compact(work)
    return oracle.paged_kv_decode_attention_f32(
        work.query.float().cpu().numpy(), kc, vc, work.seq_lens, table, batch=work.batch, heads=work.heads,
        kv_heads=work.kv_heads, head_dim=work.head_dim, block_size=work.block_size,
        block_table_batch_stride=work.block_table_batch_stride, scale=work.scale, threads=8)


def assert_close(got, want, label=""):
    assert np.isfinite(got).all(), f"{label}: non-finite output"
    gap = np.abs(got - want)
    assert gap.max() <= MAX_ABS, f"{label}: max-abs {gap.max()}"
    assert gap.mean() <= MEAN_ABS, f"{label}: mean-abs {gap.mean()}"


def test_decode_headline_shape_matches_oracle():
    # batch 32, 32 query / 8 kv heads, dim 128, block 16, context U[512, 4096], 16384-block pool
    work = synthetic.paged_decode_workload(fill="used")
    print(f"total keys {work.total_keys}", flush=True)
    assert_close(run_gpu(work), run_oracle(work), "headline")


@pytest.mark.parametrize("heads,kv_heads", [(8, 8), (8, 4), (12, 4), (8, 2), (6, 1), (8, 1), (16, 1), (24, 2)])
def test_decode_group_sizes(heads, kv_heads):
    lens = [0, 1, 15, 16, 17, 31, 32, 33, 100, 257, 300, 64]
    work = synthetic.paged_decode_workload(batch=len(lens), heads=heads, kv_heads=kv_heads, physical_blocks=256,
                                           seq_lens=lens, seed=100 + heads * 31 + kv_heads)
    got, want = run_gpu(work), run_oracle(work)
    assert not got[0].any()  # an empty sequence keeps a zero row (cpu/attention.rs:1213-1215)
    assert_close(got, want, f"{heads}/{kv_heads}")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("block_size", [16, 7, 32, 1])
@pytest.mark.parametrize("heads,kv_heads", [(40, 8), (64, 8), (7, 1), (24, 2), (48, 3)])
def test_five_to_sixteen_query_heads_per_kv_head(heads, kv_heads, block_size, dtype):
    # more than four query heads per kv head: the dense form of the decode kernel at head_dim 128 (every head a
    # column of one product, values through LDS); sixteen and twelve heads take two waves per kv head
    lens = [300, 0, 1, 31, 32, 33, 1000, 64, 17, 555]
    work = synthetic.paged_decode_workload(batch=len(lens), heads=heads, kv_heads=kv_heads, block_size=block_size,
                                           physical_blocks=max(256, 16 * 2400 // block_size), seq_lens=lens, seed=7 * heads + block_size)
    if dtype == torch.float16:  # the oracle reads what the kernel reads: bf16 values that f16 holds too
        work.query, work.key_cache, work.value_cache = (x.to(torch.float16).to(torch.bfloat16)
                                                        for x in (work.query, work.key_cache, work.value_cache))
    got, want = run_gpu(work, dtype=dtype), run_oracle(work)
    assert not got[1].any()
    assert_close(got, want, f"{heads}/{kv_heads} block {block_size} {dtype}")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("head_dim", [128, 64])
@pytest.mark.parametrize("lens", [[9000], [0, 7777], [33, 5000, 1, 0, 2048], [16] * 3])
def test_few_sequences_fold_their_many_slots_with_a_workgroup_per_row(lens, head_dim, dtype):
    # a row of a lone long sequence has a slot per worker: the merge takes a workgroup of eight waves per row then
    work = synthetic.paged_decode_workload(batch=len(lens), heads=8, kv_heads=2, head_dim=head_dim, physical_blocks=1024,
                                           seq_lens=lens, seed=len(lens) + head_dim)
    if dtype == torch.float16:
        work.query, work.key_cache, work.value_cache = (x.to(torch.float16).to(torch.bfloat16)
                                                        for x in (work.query, work.key_cache, work.value_cache))
    got, want = run_gpu(work, dtype=dtype), run_oracle(work)
    assert_close(got, want, f"lens {lens} head_dim {head_dim} {dtype}")
    for b, n in enumerate(lens):
        if n == 0:
            assert not got[b].any()


def test_the_dense_form_steps_aside_for_batches_whose_prefix_sums_do_not_fit():
    # 1600 sequences: their prefix sums (12.8 KB of LDS) no longer fit beside the dense form's staging
    rng = np.random.default_rng(12)
    lens = [int(n) for n in rng.integers(0, 40, 1600)]
    work = synthetic.paged_decode_workload(batch=len(lens), heads=16, kv_heads=2, physical_blocks=8192, seq_lens=lens, seed=9, fill="used")
    assert_close(run_gpu(work), run_oracle(work), "1600 sequences, 8 heads per kv head")


@pytest.mark.parametrize("block_size", [1, 7, 16, 32, 48, 5])
@pytest.mark.parametrize("workers", [0, 1, 3, 50, 4096])
def test_decode_block_sizes_and_splits(block_size, workers):
    lens = [200, 1, 333, 0, 97, 160, 31, 512]
    blocks = sum((l + block_size - 1) // block_size for l in lens) + 9
    work = synthetic.paged_decode_workload(batch=len(lens), heads=8, kv_heads=2, block_size=block_size,
                                           physical_blocks=blocks, seq_lens=lens, seed=7 + block_size)
    assert_close(run_gpu(work, workers), run_oracle(work), f"block {block_size} split {workers}")


def test_decode_table_stride_wider_than_needed_and_poisoned_tail():
    # Entries past a sequence's blocks hold an out-of-range block id and every cache row that no key
    # owns is NaN: a single read outside the gather set would poison the output.
    lens = np.array([130, 16, 47, 0, 255, 1], dtype=np.int32)
    work = synthetic.paged_decode_workload(batch=len(lens), heads=8, kv_heads=2, physical_blocks=128,
                                           seq_lens=lens, seed=11)
    wide = np.full((work.batch, work.block_table_batch_stride + 5), 0xFFFFFFFF, dtype=np.uint32)
    owned = torch.zeros((work.physical_blocks, work.block_size), dtype=torch.bool)
    for b, length in enumerate(lens):
        n = (int(length) + 15) // 16
        wide[b, :n] = work.block_table[b, :n]
        for key in range(int(length)):
            owned[int(work.block_table[b, key // 16]), key % 16] = True
    work.block_table, work.block_table_batch_stride = wide, wide.shape[1]
    poison = (~owned).cuda()
    work.key_cache[poison] = float("nan")
    work.value_cache[poison] = float("nan")
    got = run_gpu(work)
    clean_k, clean_v = work.key_cache.clone(), work.value_cache.clone()
    clean_k[poison], clean_v[poison] = 0, 0
    work.key_cache, work.value_cache = clean_k, clean_v
    work.block_table = np.where(wide == 0xFFFFFFFF, 0, wide).astype(np.uint32)
    assert_close(got, run_oracle(work), "poisoned tail")


def test_decode_gather_indices_are_bit_exact():
    # Each cache row carries its own (block, slot) in bf16-exact integers and one key per sequence
    # dominates the softmax, so the output row IS the gathered row: its index must equal the oracle's.
    rng = np.random.default_rng(5)
    batch, heads, kv_heads, dim, bs, blocks = 16, 8, 2, 128, 16, 4096
    lens = rng.integers(1, 700, size=batch).astype(np.int32)
    lens[:3] = [1, 16, 17]
    work = synthetic.paged_decode_workload(batch=batch, heads=heads, kv_heads=kv_heads, block_size=bs,
                                           physical_blocks=blocks, seq_lens=lens, seed=21)
    ident = torch.zeros((blocks, bs, kv_heads, dim), dtype=torch.float32)
    block_id = torch.arange(blocks).view(-1, 1, 1)
    ident[..., 0] = (block_id % 256).float()
    ident[..., 1] = (block_id // 256).float()
    ident[..., 2] = torch.arange(bs).view(1, -1, 1).float()
    ident[..., 3] = torch.arange(kv_heads).view(1, 1, -1).float()
    work.value_cache = ident.to(torch.bfloat16).cuda()
    for which in ("first", "last", "random"):
        target = {"first": np.zeros(batch, np.int64), "last": lens.astype(np.int64) - 1,
                  "random": rng.integers(0, lens)}[which]
        keys = torch.zeros((blocks, bs, kv_heads, dim), dtype=torch.float32)
        query = torch.ones((batch, heads, dim), dtype=torch.float32)
        for b in range(batch):
            blk = int(work.block_table[b, target[b] // bs])
            keys[blk, target[b] % bs] = 8.0  # score 8 * 128 * scale ~ 90 above the zero rows
        work.key_cache, work.query = keys.to(torch.bfloat16).cuda(), query.to(torch.bfloat16).cuda()
        got = run_gpu(work)
        for g in range(kv_heads):
            offsets = oracle.paged_gather_offsets(lens, work.block_table, kv_heads=kv_heads, head_dim=dim,
                                                  block_size=bs, block_table_batch_stride=work.block_table_batch_stride,
                                                  kv_head=g)
            starts = np.concatenate([[0], np.cumsum(lens.astype(np.int64))])
            for b in range(batch):
                want = int(offsets[starts[b] + target[b]])
                for h in range(g * (heads // kv_heads), (g + 1) * (heads // kv_heads)):
                    row = got[b, h]
                    seen = (((int(row[0]) + 256 * int(row[1])) * bs + int(row[2])) * kv_heads + int(row[3])) * dim
                    assert seen == want, (which, b, h, seen, want)


def test_decode_lengths_are_exact():
    # Uniform scores: the row is the mean of exactly seq_len value rows.  The key right after the
    # last one holds a huge value, the last one a distinctive one: one key too many or too few shows.
    lens = np.array([1, 2, 16, 17, 31, 33, 255, 256, 257, 1000], dtype=np.int32)
    work = synthetic.paged_decode_workload(batch=len(lens), heads=4, kv_heads=1, physical_blocks=512,
                                           seq_lens=lens, seed=31)
    work.query = torch.zeros_like(work.query)
    values = torch.zeros_like(work.value_cache, dtype=torch.float32)
    for b, length in enumerate(lens):
        last = int(length) - 1
        values[int(work.block_table[b, last // 16]), last % 16] = float(length)
        nxt = int(length)
        if nxt // 16 < work.block_table_batch_stride and nxt % 16 != 0:
            values[int(work.block_table[b, nxt // 16]), nxt % 16] = 3.0e4
    work.value_cache = values.to(torch.bfloat16).cuda()
    got = run_gpu(work)
    assert np.abs(got - 1.0).max() <= 2 ** -8  # mean = length / length, rounded once to bf16


def test_decode_validation_errors_match_the_reference():
    good = dict(batch=2, heads=8, kv_heads=2, head_dim=128, block_size=16, physical_blocks=8,
                block_table_batch_stride=4, scale=0.1)
    for bad in (dict(batch=0), dict(heads=7), dict(scale=float("nan")), dict(block_size=0)):
        with pytest.raises(error.InvalidLength):
            A.PagedKvDecodeAttentionConfig.contiguous(**{**good, **bad})
    with pytest.raises(error.LengthExceedsI32):
        A.PagedKvDecodeAttentionConfig.contiguous(**{**good, "physical_blocks": 2**31})
    config = A.PagedKvDecodeAttentionConfig.contiguous(**good)
    out = torch.zeros((2, 8, 128), device="cuda", dtype=torch.bfloat16)
    cache = torch.zeros((8, 16, 2, 128), device="cuda", dtype=torch.bfloat16)
    lens = torch.zeros(2, device="cuda", dtype=torch.int32)
    table = torch.zeros((2, 4), device="cuda", dtype=torch.int32)
    with pytest.raises(error.LengthTooShort) as caught:
        A.paged_kv_decode_attention_bf16(None, out, out.clone(), cache[:7], cache, lens, table, config)
    assert caught.value.minimum == 8 * 16 * 2 * 128 and caught.value.actual == 7 * 16 * 2 * 128
    wide_out = torch.zeros((2, 8, 320), device="cuda", dtype=torch.bfloat16)
    wide_cache = torch.zeros((8, 16, 2, 320), device="cuda", dtype=torch.bfloat16)
    with pytest.raises(error.UnsupportedWidth):  # head dimensions past 256 have no kernel
        A.paged_kv_decode_attention_bf16(None, wide_out, wide_out.clone(), wide_cache, wide_cache, lens, table,
                                         A.PagedKvDecodeAttentionConfig.contiguous(**{**good, "head_dim": 320, "heads": 8}))
    A.paged_kv_decode_attention_bf16(None, out, out.clone(), cache, cache, lens, table, config)
    torch.cuda.synchronize()


def test_decode_phases_and_scratch_reuse():
    """The one-call form and the split + reduce phases run apart give the same rows, also on repeated
    calls of different shapes that share one caller-owned scratch buffer, which carries no state."""
    shapes = [dict(batch=12, heads=16, kv_heads=4, seq_lens=[0, 700, 33, 1, 2048, 16, 90, 513, 64, 300, 5, 1000]),
              dict(batch=3, heads=8, kv_heads=8, seq_lens=[4000, 0, 129]),
              dict(batch=40, heads=8, kv_heads=2, seq_lens=list(range(1, 400, 10)))]
    works = [synthetic.paged_decode_workload(physical_blocks=1024, seed=900 + i, **shape) for i, shape in enumerate(shapes)]
    configs = [A.PagedKvDecodeAttentionConfig.contiguous(w.batch, w.heads, w.kv_heads, w.head_dim, w.block_size,
                                                         w.physical_blocks, w.block_table_batch_stride, w.scale) for w in works]
    size = max(c.workspace_bytes() for c in configs)
    scratch = torch.randint(1, 255, (size,), dtype=torch.uint8, device="cuda")  # dirty on purpose
    for _ in range(2):
        for work, config in zip(works, configs):
            want = run_oracle(work)
            lens = torch.from_numpy(work.seq_lens).cuda()
            table = torch.from_numpy(work.block_table.view(np.int32)).cuda()
            both = torch.full((work.batch, work.heads, work.head_dim), float("nan"), device="cuda", dtype=torch.bfloat16)
            A.paged_kv_decode_attention_bf16(None, both, work.query, work.key_cache, work.value_cache, lens, table, config, scratch)
            apart = torch.full_like(both, float("nan"))
            A.paged_kv_decode_attention_bf16(None, apart, work.query, work.key_cache, work.value_cache, lens, table, config, scratch, 1)
            A.paged_kv_decode_attention_bf16(None, apart, work.query, work.key_cache, work.value_cache, lens, table, config, scratch, 2)
            torch.cuda.synchronize()
            assert_close(both.float().cpu().numpy(), want, "both phases")
            assert torch.equal(both.view(torch.int16), apart.view(torch.int16))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("head_dim", [128, 64])
def test_no_more_workers_than_sequences_fold_rows_four_slots_at_a_time(head_dim, dtype):
    """With no more workers than sequences the reduce fetches a row's slots four at a time: most rows have one or two,
    and the one long sequence here has one in nearly every worker's range."""
    lens = [3000, 1, 40, 0, 17, 5, 64, 33, 2, 90]
    work = synthetic.paged_decode_workload(batch=len(lens), heads=8, kv_heads=2, head_dim=head_dim, physical_blocks=256, seq_lens=lens,
                                           seed=31)
    for workers in (10, 7):
        got, want = run_gpu(work, workers, dtype=dtype), run_oracle(work)
        assert not got[3].any()
        gap = np.abs(got - want)
        assert gap.max() <= MAX_ABS and gap.mean() <= MEAN_ABS, (workers, gap.max(), gap.mean())


def test_decode_one_long_sequence_spans_more_than_64_ranges():
    """A single sequence cut into more key ranges than a wave has lanes: the reduce walks its slots in
    chunks."""
    work = synthetic.paged_decode_workload(batch=1, heads=8, kv_heads=8, physical_blocks=640, seq_lens=[10000], seed=77)
    assert_close(run_gpu(work), run_oracle(work), "one long sequence")
    assert_close(run_gpu(work, workers=200), run_oracle(work), "one long sequence, 200 ranges")


@pytest.mark.parametrize("heads,kv_heads,block_size", [(8, 2, 16), (8, 8, 16), (16, 1, 16), (12, 4, 7), (32, 8, 32)])
def test_f16_decode_matches_oracle(heads, kv_heads, block_size):
    # bf16 values are f16 values here (N(0,1) magnitudes), so the same inputs and the same oracle serve both; the
    # f16 bounds are the bf16 ones scaled as the reference scales its own (0.03 -> 0.005, tests.rs:549-553)
    lens = [0, 1, 15, 16, 17, 100, 257, 1300, 64]
    blocks = sum((l + block_size - 1) // block_size for l in lens) + 5
    work = synthetic.paged_decode_workload(batch=len(lens), heads=heads, kv_heads=kv_heads, block_size=block_size,
                                           physical_blocks=blocks, seq_lens=lens, seed=200 + heads)
    got, want = run_gpu(work, dtype=torch.float16), run_oracle(work)
    assert not got[0].any()
    gap = np.abs(got - want)
    assert gap.max() <= MAX_ABS / 6 and gap.mean() <= MEAN_ABS / 6, (gap.max(), gap.mean())
    # and the f16 kernel against the bf16 one on the same values: they differ by the weights' rounding only
    assert np.abs(got - run_gpu(work)).max() <= MAX_ABS


def test_f16_decode_headline_shape():
    work = synthetic.paged_decode_workload(fill="used")
    got, want = run_gpu(work, dtype=torch.float16), run_oracle(work)
    gap = np.abs(got - want)
    assert gap.max() <= MAX_ABS / 6 and gap.mean() <= MEAN_ABS / 6, (gap.max(), gap.mean())


@pytest.mark.parametrize("magnitude", [20.0, 0.01])
def test_decode_peaked_and_flat_softmax(magnitude):
    # Queries twenty times larger give scores of standard deviation twenty (one or two keys carry a row and the
    # running maximum keeps jumping); a hundred times smaller give a flat average of the values.
    lens = [700, 33, 1024, 5]
    work = synthetic.paged_decode_workload(batch=len(lens), heads=8, kv_heads=2, physical_blocks=160, seq_lens=lens, seed=77)
    work.query.mul_(magnitude)
    got, want = run_gpu(work), run_oracle(work)
    assert_close(got, want, f"magnitude {magnitude}")


def random_decode_case(seed):
    """Random batches for the block-table decode kernels, bf16 or f16 or fp8 caches: block sizes whose 16-key halves lie
    whole in a block (located without per-key tests) and others, lengths that end anywhere in a half, empty sequences,
    worker counts that cut sequences anywhere."""
    import test_paged_decode_fp8_gpu as fp8
    rng = np.random.default_rng(6000 + seed)
    kv_heads = int(rng.choice([1, 2, 4, 8]))
    heads = kv_heads * int(rng.choice([1, 2, 4, 4, 8]))
    block_size = int(rng.choice([16, 16, 32, 64, 48, 7]))
    lens = [int(rng.choice([0, 1, int(rng.integers(1, 40)), int(rng.integers(40, 700)), int(rng.integers(700, 3000))]))
            for _ in range(int(rng.integers(1, 12)))]
    blocks = sum((length + block_size - 1) // block_size for length in lens) + int(rng.integers(1, 9))
    workers = int(rng.choice([0, 0, 1, 5, 37, 300]))
    kind = int(rng.integers(0, 3))
    label = (seed, heads, kv_heads, block_size, lens, workers, kind)
    if kind == 2:
        work = synthetic.paged_decode_fp8_workload(batch=len(lens), heads=heads, kv_heads=kv_heads, block_size=block_size,
                                                   physical_blocks=blocks, seq_lens=lens, seed=seed)
        fp8.assert_close(fp8.run_gpu(work, False, workers), fp8.run_oracle(work), str(label))
    else:
        dtype = torch.bfloat16 if kind == 0 else torch.float16
        work = synthetic.paged_decode_workload(batch=len(lens), heads=heads, kv_heads=kv_heads, block_size=block_size,
                                               physical_blocks=blocks, seq_lens=lens, seed=seed)
        assert_close(run_gpu(work, workers, dtype), run_oracle(work), str(label))


@pytest.mark.parametrize("seed", range(24))
def test_decode_random_batches(seed):
    random_decode_case(seed)
