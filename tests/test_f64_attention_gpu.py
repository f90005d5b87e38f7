"""The paged op and the dense op on f64 tensors (the reference's general kernel and CPU path take f64 and compute it in
f64: singe/src/backend/cuda/kernel_plan/source/paged_general.rs:91-99, singe/src/backend/cpu/normalization/
attention.rs:63-69), against a float64 restatement in numpy that shares no code with the kernels: matrix products
instead of fma chains, so agreement is to rounding order, 1e-12 on outputs of magnitude one and 1e-5 on the f32
log-sum-exp the op returns.  Parity unpinned beyond that: the reference holds no f64 fixture for these ops."""
import math

import numpy as np
import pytest
import torch

from singe_amd import error, neural

pytestmark = pytest.mark.gpu


def softmax_rows_f64(scores, values):
    """scores [L, S] with -inf for hidden keys, values [S, D] -> (out [L, D], lse natural [L])."""
    peak = scores.max(axis=1, keepdims=True, initial=-np.inf)
    peak = np.where(np.isfinite(peak), peak, 0.0)
    weights = np.exp(scores - peak)
    total = weights.sum(axis=1, keepdims=True)
    with np.errstate(divide="ignore", invalid="ignore"):
        out = np.where(total > 0, (weights @ values) / total, 0.0)
        lse = np.where(total[:, 0] > 0, peak[:, 0] + np.log(total[:, 0]), -np.inf)
    return out, lse


@pytest.mark.parametrize("index_dtype", [torch.int32, torch.int64])
@pytest.mark.parametrize("causal,window,softcap", [(False, None, None), (True, None, None), (True, 16, 30.0)])
@pytest.mark.parametrize("heads,kv_heads,dim,page_size", [(8, 2, 64, 1), (8, 1, 128, 16), (4, 4, 64, 7), (4, 2, 200, 5)])
def test_paged_attention_f64(heads, kv_heads, dim, page_size, causal, window, softcap, index_dtype):
    # the reference's ragged recipe (kernel_plan/source/tests.rs:830-889): decode, full prefill, chunked prefill, no keys
    sequences = [(1, 150), (70, 70), (20, 90), (3, 0), (9, 4)]
    query_offsets, page_offsets, last, needed = [0], [0], [], 0
    for queries, keys in sequences:
        query_offsets.append(query_offsets[-1] + queries)
        pages = (keys + page_size - 1) // page_size
        needed += pages
        page_offsets.append(needed)
        last.append(0 if keys == 0 else keys - (pages - 1) * page_size)
    page_count = needed + 3
    table = list(np.random.default_rng(page_count).permutation(page_count)[:needed])
    rng = np.random.default_rng(dim + page_size)
    q = rng.standard_normal((query_offsets[-1], heads, dim))
    kc = rng.standard_normal((page_count, page_size, kv_heads, dim))
    vc = rng.standard_normal((page_count, page_size, kv_heads, dim))
    index = lambda values: torch.tensor(values, dtype=index_dtype, device="cuda")
    paging = neural.Paging(index(query_offsets), index(page_offsets), index(table), index(last))
    options = neural.AttentionOptions(causal=causal, window=window, softcap=softcap)
    device = lambda a: torch.tensor(a, dtype=torch.float64, device="cuda")
    out, lse = neural.paged_attention(device(q), device(kc), device(vc), paging, options)
    assert out.dtype == torch.float64 and lse.dtype == torch.float32
    out, lse = out.cpu().numpy(), lse.cpu().numpy()

    scale, group = 1.0 / math.sqrt(dim), heads // kv_heads
    kflat, vflat = kc.reshape(-1, kv_heads, dim), vc.reshape(-1, kv_heads, dim)
    for s, (queries, keys) in enumerate(sequences):
        slot = np.array([table[page_offsets[s] + key // page_size] * page_size + key % page_size for key in range(keys)], dtype=np.int64)
        position = np.maximum(keys + np.arange(queries) - queries, 0)[:, None]
        key_index = np.arange(keys)[None, :]
        visible = np.ones((queries, keys), bool)
        if causal:
            visible &= key_index <= position
        if window is not None:
            visible &= key_index + window > position
        for h in range(heads):
            rows = q[query_offsets[s]: query_offsets[s + 1], h]
            scores = (rows @ kflat[slot, h // group].T) * scale
            if softcap is not None:
                scores = np.tanh(scores / softcap) * softcap
            want, want_lse = softmax_rows_f64(np.where(visible, scores, -np.inf), vflat[slot, h // group])
            got, got_lse = out[query_offsets[s]: query_offsets[s + 1], h], lse[query_offsets[s]: query_offsets[s + 1], h]
            assert np.abs(got - want).max(initial=0.0) <= 1e-12
            empty = np.isneginf(want_lse)
            assert np.array_equal(np.isneginf(got_lse), empty) and not got[empty].any()
            assert np.abs(got_lse[~empty] - want_lse[~empty] / math.log(2.0)).max(initial=0.0) <= 1e-5


def test_dense_attention_f64_with_every_option():
    rng = np.random.default_rng(5)
    batch, heads, kv_heads, query_len, key_len, dim, value_dim = 2, 4, 2, 37, 53, 48, 80
    q = rng.standard_normal((batch, heads, query_len, dim))
    k = rng.standard_normal((batch, kv_heads, key_len, dim))
    v = rng.standard_normal((batch, kv_heads, key_len, value_dim))
    mask = rng.standard_normal((query_len, key_len))
    mask[:, 3] = -np.inf
    sinks = rng.standard_normal(heads)
    device = lambda a: torch.tensor(a, dtype=torch.float64, device="cuda")
    out = neural.attend(device(q), device(k), device(v), device(mask), device(sinks),
                        neural.AttentionOptions(causal=True, window=30, softcap=5.0, scale=0.2)).cpu().numpy()
    query_index, key_index = np.arange(query_len)[:, None], np.arange(key_len)[None, :]
    visible = (key_index <= query_index) & (key_index + 30 > query_index)
    for b in range(batch):
        for h in range(heads):
            # an explicit scale is an f32 attribute widened to f64 (attention.rs:82-87)
            scores = np.tanh((q[b, h] @ k[b, h // 2].T) * float(np.float32(0.2)) / 5.0) * 5.0 + mask
            scores = np.where(visible, scores, -np.inf)
            # the sink is one more score that weighs no value (attention.rs:255-262)
            joined = np.concatenate([scores, np.full((query_len, 1), sinks[h])], axis=1)
            values = np.concatenate([v[b, h // 2], np.zeros((1, value_dim))], axis=0)
            want, _ = softmax_rows_f64(joined, values)
            assert np.abs(out[b, h] - want).max() <= 1e-12


def test_f64_is_refused_where_the_reference_does_not_take_it():
    latent = torch.zeros((2, 2, 64), device="cuda", dtype=torch.float64)
    index = lambda values: torch.tensor(values, dtype=torch.int32, device="cuda")
    paging = neural.Paging(index([0, 2]), index([0, 1]), index([0]), index([2]))
    with pytest.raises(error.Error):
        neural.paged_mla_attention(latent, latent[..., :16].contiguous(), torch.zeros((2, 4, 64), device="cuda", dtype=torch.float64),
                                   torch.zeros((2, 4, 16), device="cuda", dtype=torch.float64), paging)
