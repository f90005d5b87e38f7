"""paged_kv_prefill_attention_bf16 (block-table paging, queries aligned with the first keys, natural-log
LSE) on the GPU against the CPU oracle, through the C ABI.  bf16 outputs within max-abs 2e-2 /
mean-abs 2e-3, LSE within 2e-3; the reference's own validation cases
(singe-kernel/src/cuda/attention/tests.rs:349-375) for the length checks."""
import numpy as np
import pytest
import torch

import oracle
from singe_amd import error
from singe_amd.kernel import attention as A

pytestmark = pytest.mark.gpu

MAX_ABS, MEAN_ABS, LSE_ABS = 2e-2, 2e-3, 2e-3
DIM = 128


def build(sequences, heads, kv_heads, block_size, seed, gap_tokens=0, extra_blocks=5, dim=DIM):
    """sequences: (query tokens, keys) pairs.  Tokens are packed in order with `gap_tokens` unowned
    rows between sequences; table rows are slices of a seeded permutation of the pool."""
    rng = np.random.default_rng(seed)
    lens_q = np.array([q for q, _ in sequences], dtype=np.int32)
    lens_kv = np.array([k for _, k in sequences], dtype=np.int32)
    offsets, at = [], 0
    for q, _ in sequences:
        offsets.append(at)
        at += q + gap_tokens
    total = max(at, 1)
    counts = (lens_kv.astype(np.int64) + block_size - 1) // block_size
    stride = max(int(counts.max()), 1) + 1
    blocks = int(counts.sum()) + extra_blocks
    perm = rng.permutation(blocks)
    table = np.zeros((len(sequences), stride), dtype=np.uint32)
    used = 0
    for b, n in enumerate(counts):
        table[b, :n] = perm[used:used + n]
        used += int(n)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(seed)
    query = torch.randn((total, heads, dim), generator=gen, device="cuda").to(torch.bfloat16)
    kc = torch.randn((blocks, block_size, kv_heads, dim), generator=gen, device="cuda").to(torch.bfloat16)
    vc = torch.randn((blocks, block_size, kv_heads, dim), generator=gen, device="cuda").to(torch.bfloat16)
    return lens_q, lens_kv, np.array(offsets, dtype=np.int32), table, stride, blocks, total, query, kc, vc


def run_case(sequences, heads, kv_heads, block_size, causal, seed=0, gap_tokens=0, scale=None, dtype=torch.bfloat16, dim=DIM):
    DIM = dim
    lens_q, lens_kv, offsets, table, stride, blocks, total, query, kc, vc = build(sequences, heads, kv_heads, block_size,
                                                                                seed, gap_tokens, dim=dim)
    query, kc, vc = query.to(dtype), kc.to(dtype), vc.to(dtype)
    scale = DIM ** -0.5 if scale is None else scale
    config = A.PagedKvPrefillAttentionConfig.contiguous(len(sequences), total, heads, kv_heads, DIM, block_size, blocks,
                                                        stride, causal, scale)
    sentinel = 7.0
    out = torch.full((total, heads, DIM), sentinel, device="cuda", dtype=dtype)
    lse = torch.full((total, heads), sentinel, device="cuda", dtype=torch.float32)
    op = A.paged_kv_prefill_attention_bf16 if dtype == torch.bfloat16 else A.paged_kv_prefill_attention_f16
    op(None, out, lse, query, kc, vc, torch.from_numpy(lens_q).cuda(),
                                      torch.from_numpy(lens_kv).cuda(), torch.from_numpy(offsets).cuda(),
                                      torch.from_numpy(table.view(np.int32)).cuda(), config)
    torch.cuda.synchronize()
    want, want_lse = oracle.paged_kv_prefill_attention_f32(
        query.float().cpu().numpy(), kc.float().cpu().numpy(), vc.float().cpu().numpy(), lens_q, lens_kv, offsets, table,
        batch=len(sequences), total_query_tokens=total, heads=heads, kv_heads=kv_heads, head_dim=DIM,
        block_size=block_size, block_table_batch_stride=stride, causal=causal, scale=scale, threads=8)
    got, got_lse = out.float().cpu().numpy(), lse.cpu().numpy()
    owned = np.zeros(total, dtype=bool)
    for start, count in zip(offsets, lens_q):
        owned[start:start + count] = True
    # Rows no sequence owns are not written.
    assert (got[~owned] == sentinel).all() and (got_lse[~owned] == sentinel).all()
    got, got_lse, want, want_lse = got[owned], got_lse[owned], want[owned], want_lse[owned]
    if got.size == 0:
        return
    assert np.isfinite(got).all()
    gap = np.abs(got - want)
    # f16 carries three more mantissa bits than bf16: the reference's own bounds are 0.03 and 0.005
    # (kernel_plan/source/tests.rs:549-553); the same ratio is applied to the bf16 bounds here.
    tighter = 1.0 if dtype == torch.bfloat16 else 1.0 / 6.0
    assert gap.max() <= MAX_ABS * tighter, gap.max()
    assert gap.mean() <= MEAN_ABS * tighter, gap.mean()
    empty = want_lse == np.float32(-1.0e20)
    assert np.array_equal(got_lse == np.float32(-1.0e20), empty)
    assert not got[empty].any()
    assert np.abs(got_lse[~empty] - want_lse[~empty]).max(initial=0.0) <= LSE_ABS


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("case", [
    dict(sequences=[(5, 5), (2, 40)], heads=4, kv_heads=2, block_size=3),          # the reference's validation shape
    dict(sequences=[(130, 130), (1, 1), (33, 200), (64, 10)], heads=8, kv_heads=2, block_size=16),
    dict(sequences=[(300, 257)], heads=2, kv_heads=2, block_size=7),
    dict(sequences=[(70, 70), (0, 12), (9, 0), (20, 90)], heads=16, kv_heads=2, block_size=16, gap_tokens=2),
    dict(sequences=[(100, 300), (7, 33), (64, 64)], heads=8, kv_heads=2, block_size=32),
    dict(sequences=[(40, 200), (129, 129)], heads=4, kv_heads=1, block_size=128),
])
def test_matches_oracle(case, causal):
    run_case(causal=causal, seed=11, **case)


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("case", [
    dict(sequences=[(130, 130), (1, 1), (33, 200), (64, 10)], heads=8, kv_heads=2, block_size=16),
    dict(sequences=[(300, 257)], heads=2, kv_heads=2, block_size=7),
    dict(sequences=[(70, 70), (0, 12), (9, 0), (20, 90)], heads=16, kv_heads=2, block_size=16, gap_tokens=2),
])
def test_f16_matches_oracle(case, causal):
    run_case(causal=causal, seed=12, dtype=torch.float16, **case)


@pytest.mark.parametrize("dtype,dim", [(torch.bfloat16, 128), (torch.bfloat16, 64), (torch.float16, 96)])
def test_many_ragged_sequences_find_their_row_tiles(dtype, dim):
    # more sequences than one wave's prefix sum covers (64), query counts from none to several 128-row tiles,
    # unowned rows between sequences; 96 takes the one-wave-per-row kernel's list of workgroups
    rng = np.random.default_rng(dim)
    sequences = []
    for s in range(130):
        queries = int(rng.choice([0, 1, 2, 7, 31, 32, 33, 70, 150]))
        sequences.append((queries, 0 if s % 29 == 4 else queries + int(rng.integers(0, 90))))
    run_case(sequences, 8, 2, 16, True, seed=dim, gap_tokens=1, dtype=dtype, dim=dim)
    run_case(sequences[:70], 4, 4, 7, False, seed=dim + 1, dtype=dtype, dim=dim)


def test_more_queries_than_keys_causal_and_full():
    """Queries past the last key see every key when causal (key <= query index) and when not."""
    run_case([(48, 5)], 4, 1, 4, True, seed=3)
    run_case([(48, 5)], 4, 1, 4, False, seed=3)


def test_negative_scale():
    run_case([(40, 77)], 4, 4, 16, True, seed=5, scale=-0.09)


def test_chunk_of_a_long_sequence():
    run_case([(256, 1500), (256, 700)], 8, 1, 16, True, seed=9)


def test_validation_mirrors_reference_cases():
    config = A.PagedKvPrefillAttentionConfig.contiguous(2, 7, 4, 2, 8, 3, 5, 4, True, 0.5)
    assert config.output_len() == 224 and config.lse_len() == 28
    with pytest.raises(error.InvalidLength):
        A.PagedKvPrefillAttentionConfig.contiguous(2, 7, 3, 2, 8, 3, 5, 4, True, 0.5)
    # A short lse is refused before anything is launched (tests.rs:356-366); a head dimension past 256 has no
    # kernel and is reported as an unsupported width after the length checks.
    bf16 = lambda n: torch.zeros(n, device="cuda", dtype=torch.bfloat16)
    i32 = lambda n: torch.zeros(n, device="cuda", dtype=torch.int32)
    with pytest.raises(error.LengthTooShort) as caught:
        A.paged_kv_prefill_attention_bf16(None, bf16(224), torch.zeros(27, device="cuda"), bf16(224), bf16(240), bf16(240),
                                          i32(2), i32(2), i32(2), i32(8), config)
    assert caught.value.name == "lse" and caught.value.minimum == 28 and caught.value.actual == 27
    A.paged_kv_prefill_attention_bf16(None, bf16(224), torch.zeros(28, device="cuda"), bf16(224), bf16(240), bf16(240),
                                      i32(2), i32(2), i32(2), i32(8), config)  # the reference's own shape runs
    wide = A.PagedKvPrefillAttentionConfig.contiguous(2, 7, 4, 2, 320, 3, 5, 4, True, 0.5)
    with pytest.raises(error.UnsupportedWidth):
        A.paged_kv_prefill_attention_bf16(None, bf16(7 * 4 * 320), torch.zeros(28, device="cuda"), bf16(7 * 4 * 320),
                                          bf16(5 * 3 * 2 * 320), bf16(5 * 3 * 2 * 320), i32(2), i32(2), i32(2), i32(8), wide)


def test_out_of_range_sequence_is_skipped():
    """Offsets or lengths that would address outside the buffers leave the sequence's rows unwritten and
    read nothing through them."""
    heads, kv_heads, block_size = 4, 2, 16
    lens_q, lens_kv, offsets, table, stride, blocks, total, query, kc, vc = build([(8, 20), (8, 20)], heads, kv_heads,
                                                                                block_size, 21)
    config = A.PagedKvPrefillAttentionConfig.contiguous(2, total, heads, kv_heads, DIM, block_size, blocks, stride, True,
                                                        DIM ** -0.5)
    bad_lens_kv = lens_kv.copy()
    bad_lens_kv[1] = stride * block_size + 1
    out = torch.full((total, heads, DIM), 7.0, device="cuda", dtype=torch.bfloat16)
    lse = torch.full((total, heads), 7.0, device="cuda", dtype=torch.float32)
    A.paged_kv_prefill_attention_bf16(None, out, lse, query, kc, vc, torch.from_numpy(lens_q).cuda(),
                                      torch.from_numpy(bad_lens_kv).cuda(), torch.from_numpy(offsets).cuda(),
                                      torch.from_numpy(table.view(np.int32)).cuda(), config)
    torch.cuda.synchronize()
    assert (out[8:].float() == 7.0).all() and not (out[:8].float() == 7.0).all()
