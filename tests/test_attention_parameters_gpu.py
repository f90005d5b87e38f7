"""Every candidate of AttentionParameters gives what the default gives, within 0.1, on the reference's own operands
(singe/src/backend/cuda/kernel_plan/source/parameter_tests.rs:150-276) and on decode-shaped problems where the
threshold really changes how many workgroups share a row tile's keys; and the dense op's key splits against the CPU
oracle (attention.rs:283-292, 420-452, 588-654), sinks, key lengths, window, cap and mask included.
bf16 max-abs 2e-2 / mean-abs 2e-3, f16 max-abs 5e-3 against the oracle."""
import ctypes

import numpy as np
import pytest
import torch

import oracle
from singe_amd import _native, neural
from test_general_attention_gpu import close, host, tensors

pytestmark = pytest.mark.gpu


def reference_tensor(shape, dtype, seed):
    # the reference fills its test operands with ((i * 37 + seed * 11) % 41) / 20 - 1 (kernel_plan/source/tests.rs:443-563)
    count = int(np.prod(shape))
    values = ((np.arange(count, dtype=np.int64) * 37 + seed * 11) % 41) / 20.0 - 1.0
    return torch.tensor(values.reshape(shape), dtype=torch.float32, device="cuda").to(dtype)


def index(values, dtype=torch.int32):
    return torch.tensor(values, dtype=dtype, device="cuda")


def every_candidate(run):
    """run() under the default and under every candidate: all within 0.1 of the default (parameter_tests.rs:100-112)."""
    neural.set_attention_parameters(None)
    expected = [t.float().clone() for t in run()]
    candidates = neural.attention_candidates()
    assert len(candidates) > 1
    try:
        for candidate in candidates:
            neural.set_attention_parameters(candidate)
            for actual, wanted in zip(run(), expected):
                actual = actual.float()
                both_empty = torch.isneginf(actual) & torch.isneginf(wanted)
                gap = torch.where(both_empty, torch.zeros_like(actual), (actual - wanted).abs())
                assert torch.isfinite(gap).all() and gap.max().item() <= 0.1, (candidate, gap.max().item())
    finally:
        neural.set_attention_parameters(None)


def test_every_paged_attention_parameter_matches_the_default():
    # parameter_tests.rs:244-276: query [5, 4, 16], caches [4, 32, 2, 16], offsets [0, 3, 5], [0, 2, 4], pages [0, 1, 3, 2], last [8, 4]
    q = reference_tensor((5, 4, 16), torch.bfloat16, 8)
    kc, vc = reference_tensor((4, 32, 2, 16), torch.bfloat16, 9), reference_tensor((4, 32, 2, 16), torch.bfloat16, 10)
    paging = neural.Paging(index([0, 3, 5]), index([0, 2, 4]), index([0, 1, 3, 2]), index([8, 4]))
    every_candidate(lambda: neural.paged_attention(q, kc, vc, paging, neural.AttentionOptions(causal=True)))
    # parameter_tests.rs:226-241: query [3, 1, 128], caches [4, 32, 1, 128], one sequence of two pages
    q = reference_tensor((3, 1, 128), torch.bfloat16, 14)
    kc, vc = reference_tensor((4, 32, 1, 128), torch.bfloat16, 15), reference_tensor((4, 32, 1, 128), torch.bfloat16, 16)
    paging = neural.Paging(index([0, 3]), index([0, 2]), index([0, 1]), index([8]))
    every_candidate(lambda: neural.paged_attention(q, kc, vc, paging, neural.AttentionOptions(causal=True)))


def test_every_attention_parameter_matches_the_default():
    # parameter_tests.rs:150-180 and 208-225: f16 [1, 4, 8, 16] on [1, 2, 96, 16], and [1, 1, 4, 128] on [1, 1, 96, 128], causal
    q, k, v = (reference_tensor(shape, torch.float16, seed) for shape, seed in (((1, 4, 8, 16), 5), ((1, 2, 96, 16), 6), ((1, 2, 96, 16), 7)))
    every_candidate(lambda: (neural.scaled_dot_product_attention(q, k, v, None, True),))
    q, k, v = (reference_tensor(shape, torch.float16, seed) for shape, seed in (((1, 1, 4, 128), 11), ((1, 1, 96, 128), 12), ((1, 1, 96, 128), 13)))
    every_candidate(lambda: (neural.scaled_dot_product_attention(q, k, v, None, True),))


@pytest.mark.parametrize("dim", [128, 64])
def test_candidates_agree_where_the_threshold_changes_the_shares(dim):
    # eight decoding sequences of 8000 to 20000 keys: 16 workgroups unsplit; the candidates' thresholds give 1 to 24
    # shares (a share keeps at least eight key tiles of a sequence of average length)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(dim)
    lens = [8000, 20000, 12400, 8191, 16384, 10000, 13333, 8193]
    pages_of = [(n + 15) // 16 for n in lens]
    page_count = sum(pages_of) + 3
    q = torch.randn((len(lens), 8, dim), generator=gen, device="cuda").to(torch.bfloat16)
    kc = torch.randn((page_count, 16, 2, dim), generator=gen, device="cuda").to(torch.bfloat16)
    vc = torch.randn((page_count, 16, 2, dim), generator=gen, device="cuda").to(torch.bfloat16)
    table = np.random.default_rng(3).permutation(page_count)[:sum(pages_of)]
    paging = neural.Paging(index(list(range(len(lens) + 1))), index(np.concatenate([[0], np.cumsum(pages_of)])), index(table),
                           index([n - (p - 1) * 16 for n, p in zip(lens, pages_of)]))
    # (a score cap keeps this decode step on the row-tile kernel, whose shares the thresholds change; without one the
    # step would run on the block-table decode kernels)
    options = neural.AttentionOptions(causal=True, softcap=50.0)
    problem = neural._problem(q, kc, vc, paging, options)
    wanted = set()
    for candidate in neural.attention_candidates():
        neural.set_attention_parameters(candidate)
        wanted.add(int(_native.lib().singe_hip_paged_attention_scratch_bytes(ctypes.byref(problem))))
    neural.set_attention_parameters(None)
    assert 0 in wanted and len(wanted) >= 3  # no split at all, and at least two different numbers of shares
    every_candidate(lambda: neural.paged_attention(q, kc, vc, paging, options))
    q4, k4, v4 = tensors((2, 8, 4, dim), (2, 2, 3000, dim), (2, 2, 3000, dim), torch.bfloat16, 5)
    every_candidate(lambda: (neural.scaled_dot_product_attention(q4, k4, v4, None, True),))


def dense_splits(q, k):
    batch, heads, query_len, dim = q.shape
    problem = _native.AttentionProblemC(batch, heads, k.shape[1], query_len, k.shape[2], dim, dim, (ctypes.c_int64 * 4)(0, 0, 0, 0),
                                        neural._DATA_TYPES[q.dtype], 0, 0, 0, 0, 0.0, 0.0, 0)
    need = int(_native.lib().singe_hip_scaled_dot_product_attention_scratch_bytes(ctypes.byref(problem)))
    return need // (batch * heads * query_len * (dim + 1) * 4)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("dim", [128, 64])
@pytest.mark.parametrize("options", [dict(), dict(causal=True), dict(causal=True, window=700, softcap=8.0), dict(window=1500),
                                     dict(softcap=-3.0, scale=0.05)])
def test_dense_key_splits_match_the_oracle(dim, options, dtype):
    """Few query rows on many keys: the op shares a query tile's keys out over workgroups and merges them."""
    batch, heads, kv_heads, query_len, key_len = 2, 8, 2, 5, 2500
    q, k, v = tensors((batch, heads, query_len, dim), (batch, kv_heads, key_len, dim), (batch, kv_heads, key_len, dim), dtype, 41 + dim)
    assert dense_splits(q, k) > 1
    out = neural.attend(q, k, v, options=neural.AttentionOptions(**options))
    want = oracle.scaled_dot_product_attention_f32(host(q), host(k), host(v), threads=8, **options)
    close(host(out), want, dtype)
    # and the split result stays within the weights' rounding of the unsplit one
    neural.set_attention_parameters(neural.AttentionParameters(split_below_blocks=0))
    try:
        assert dense_splits(q, k) == 0
        apart = neural.attend(q, k, v, options=neural.AttentionOptions(**options))
    finally:
        neural.set_attention_parameters(None)
    assert (out.float() - apart.float()).abs().max().item() <= (8e-3 if dtype == torch.bfloat16 else 2e-3)


@pytest.mark.parametrize("dim", [128, 64])
def test_dense_key_splits_with_sinks_key_lengths_and_a_mask(dim):
    batch, heads, kv_heads, query_len, key_len = 3, 4, 2, 3, 1800
    dtype = torch.bfloat16
    q, k, v = tensors((batch, heads, query_len, dim), (batch, kv_heads, key_len, dim), (batch, kv_heads, key_len, dim), dtype, 77)
    assert dense_splits(q, k) > 1
    gen = torch.Generator(device="cuda")
    gen.manual_seed(9)
    sinks = (torch.randn((heads,), generator=gen, device="cuda") * 3).to(dtype)
    sinks[1] = float("-inf")  # a sink that never counts
    sinks[2] = 30.0           # a sink that takes nearly all of every row
    out = neural.attend(q, k, v, None, sinks, neural.AttentionOptions(causal=True))
    want = oracle.scaled_dot_product_attention_f32(host(q), host(k), host(v), causal=True, sinks=host(sinks), threads=8)
    close(host(out), want, dtype)
    # per-batch key counts: none (zeros), some that leave the later shares empty, all
    lengths = torch.tensor([0, 300, 4000], dtype=torch.int32, device="cuda")
    out = neural.attend_padded(q, k, v, lengths)
    want = oracle.scaled_dot_product_attention_f32(host(q), host(k), host(v), key_lengths=[0, 300, 4000], threads=8)
    close(host(out), want, dtype)
    assert not host(out)[0].any()
    mask = torch.randn((query_len, key_len), generator=gen, device="cuda").to(dtype)
    mask[:, 3] = float("-inf")
    mask[1, :1700] = float("-inf")  # a row whose first shares see nothing
    out = neural.attend(q, k, v, mask, sinks)
    want = oracle.scaled_dot_product_attention_f32(host(q), host(k), host(v), mask=host(mask), sinks=host(sinks), threads=8)
    close(host(out), want, dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("heads, kv_heads, query_len", [(8, 2, 1), (32, 8, 4), (16, 1, 8), (16, 2, 16), (16, 2, 17), (6, 3, 5), (64, 8, 16)])
def test_grouped_heads_of_a_decode_shaped_dense_call_share_a_tile(heads, kv_heads, query_len, dtype):
    """Without a causal mask, query_len * (heads / kv_heads) rows of at most a tile are packed into one tile per kv head
    (17 queries under eight heads a kv head are not, nor is anything under a causal mask): with and without key splits,
    with a mask that differs per head, sinks per head and per-batch key counts, against the oracle."""
    batch, key_len, dim = 2, 1500, 128
    q, k, v = tensors((batch, heads, query_len, dim), (batch, kv_heads, key_len, dim), (batch, kv_heads, key_len, dim), dtype, 3 * heads + query_len)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(heads)
    mask = torch.randn((heads, query_len, key_len), generator=gen, device="cuda").to(dtype)
    mask[heads - 1, query_len - 1, 100:] = float("-inf")
    sinks = torch.randn((heads,), generator=gen, device="cuda").to(dtype)
    lengths = torch.tensor([key_len, 700], dtype=torch.int32, device="cuda")
    for below in (None, 0):
        neural.set_attention_parameters(None if below is None else neural.AttentionParameters(split_below_blocks=below))
        try:
            plain = neural.attend(q, k, v)
            with_mask = neural.attend(q, k, v, mask, sinks, neural.AttentionOptions(softcap=20.0))
            padded = neural.attend_padded(q, k, v, lengths, neural.AttentionOptions(window=900))
        finally:
            neural.set_attention_parameters(None)
        close(host(plain), oracle.scaled_dot_product_attention_f32(host(q), host(k), host(v), threads=8), dtype)
        close(host(with_mask), oracle.scaled_dot_product_attention_f32(host(q), host(k), host(v), mask=host(mask), sinks=host(sinks),
                                                                       softcap=20.0, threads=8), dtype)
        close(host(padded), oracle.scaled_dot_product_attention_f32(host(q), host(k), host(v), key_lengths=[key_len, 700], window=900,
                                                                    threads=8), dtype)
