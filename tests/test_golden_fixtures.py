"""The CPU oracle against tests/golden/sdpa_fixtures.npz: answers of a library routine
(torch.nn.functional.scaled_dot_product_attention on the CPU in float32, written by tests/golden/make_sdpa_fixtures.py)
that shares no code with the oracle.  Every oracle function of the attention path is run on the fixtures' inputs
in the layout it takes (dense BHSD and BSHD, paged through CSR tables and through block tables, split and
reduced) and must give the library's output and log-sum-exp."""
import os

import numpy as np
import pytest

import oracle

FIXTURES = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "sdpa_fixtures.npz"), allow_pickle=False)
OUT_TOLERANCE, LSE_TOLERANCE = 3e-6, 1e-5
LN2 = float(np.log(2.0))


def load(name):
    keys = ("query", "key", "value", "out", "lse")
    q, k, v, out, lse = (FIXTURES[f"{name}/{key}"] for key in keys)
    mask = FIXTURES[f"{name}/mask"] if f"{name}/mask" in FIXTURES.files else None
    return q, k, v, out, lse, float(FIXTURES[f"{name}/scale"]), mask


def page(gen, keys, values, page_size):
    """[batch, kv_heads, S, D] -> shuffled paged caches [pages, page_size, kv_heads, D] with their CSR vectors."""
    batch, kv_heads, length, dim = keys.shape
    per = -(-length // page_size)
    total = batch * per + 3
    order = gen.permutation(total)
    kc = gen.normal(size=(total, page_size, kv_heads, dim)).astype(np.float32)  # unread slots hold noise
    vc = gen.normal(size=(total, page_size, kv_heads, dim)).astype(np.float32)
    pages, page_offsets, last = [], [0], []
    for b in range(batch):
        mine = order[b * per:(b + 1) * per]
        for p, index in enumerate(mine):
            rows = slice(p * page_size, min((p + 1) * page_size, length))
            n = rows.stop - rows.start
            kc[index, :n] = keys[b, :, rows].transpose(1, 0, 2)
            vc[index, :n] = values[b, :, rows].transpose(1, 0, 2)
        pages += list(mine)
        page_offsets.append(len(pages))
        last.append(length - (per - 1) * page_size)
    return kc, vc, np.array(pages), np.array(page_offsets), np.array(last), per


@pytest.mark.parametrize("name,causal", [("anchor_causal", True), ("gqa_full", False), ("gqa_causal_square", True),
                                         ("prefix_top_left", True), ("masked", False), ("decode", False)])
def test_dense_op(name, causal):
    q, k, v, out, lse, scale, mask = load(name)
    got = oracle.scaled_dot_product_attention_f32(q, k, v, scale=scale, causal=causal, mask=mask)
    assert np.abs(got - out).max() <= OUT_TOLERANCE


@pytest.mark.parametrize("name,causal", [("anchor_causal", True), ("gqa_full", False), ("gqa_causal_square", True),
                                         ("prefix_top_left", True), ("decode", False)])
def test_dense_prefill_with_lse(name, causal):
    q, k, v, out, lse, scale, _ = load(name)
    batch, heads, query_len, dim = q.shape
    got, got_lse = oracle.fmha_prefill_lse_f32(q.transpose(0, 2, 1, 3), k.transpose(0, 2, 1, 3), v.transpose(0, 2, 1, 3), batch=batch,
                                               query_len=query_len, key_len=k.shape[2], heads=heads, kv_heads=k.shape[1], head_dim=dim,
                                               scale=scale, causal=causal)
    assert np.abs(got.reshape(batch, query_len, heads, dim).transpose(0, 2, 1, 3) - out).max() <= OUT_TOLERANCE
    assert np.abs(got_lse.reshape(batch, heads, query_len) - lse).max() <= LSE_TOLERANCE


@pytest.mark.parametrize("page_size", [1, 4, 7])
@pytest.mark.parametrize("name,causal", [("chunk_bottom_right", True), ("gqa_causal_square", True), ("gqa_full", False), ("decode", False)])
def test_paged_op_through_csr_tables(name, causal, page_size):
    q, k, v, out, lse, scale, _ = load(name)
    batch, heads, query_len, dim = q.shape
    kc, vc, pages, page_offsets, last, _ = page(np.random.default_rng(page_size), k, v, page_size)
    rows = q.transpose(0, 2, 1, 3).reshape(batch * query_len, heads, dim)
    query_offsets = np.arange(batch + 1) * query_len
    status, got, got_lse = oracle.paged_attention_f32(rows, kc, vc, query_offsets, page_offsets, pages, last, scale=scale, causal=causal)
    assert status == 0
    assert np.abs(got.reshape(batch, query_len, heads, dim).transpose(0, 2, 1, 3) - out).max() <= OUT_TOLERANCE
    assert np.abs(got_lse.reshape(batch, query_len, heads).transpose(0, 2, 1) * LN2 - lse).max() <= LSE_TOLERANCE  # base two


@pytest.mark.parametrize("block_size", [1, 5, 16])
def test_block_table_decode(block_size):
    q, k, v, out, lse, scale, _ = load("decode")
    batch, heads, _, dim = q.shape
    kc, vc, pages, _, _, per = page(np.random.default_rng(block_size), k, v, block_size)
    table = pages.reshape(batch, per).astype(np.uint32)
    lengths = np.full(batch, k.shape[2], dtype=np.int32)
    for literal in (False, True):
        got = oracle.paged_kv_decode_attention_f32(q[:, :, 0], kc, vc, lengths, table, batch=batch, heads=heads, kv_heads=k.shape[1],
                                                   head_dim=dim, block_size=block_size, block_table_batch_stride=per, scale=scale,
                                                   literal=literal)
        assert np.abs(got - out[:, :, 0]).max() <= OUT_TOLERANCE


@pytest.mark.parametrize("name,causal", [("prefix_top_left", True), ("anchor_causal", True), ("gqa_full", False)])
def test_block_table_prefill(name, causal):
    q, k, v, out, lse, scale, _ = load(name)
    batch, heads, query_len, dim = q.shape
    kc, vc, pages, _, _, per = page(np.random.default_rng(3), k, v, 4)
    rows = q.transpose(0, 2, 1, 3).reshape(batch * query_len, heads, dim)
    got, got_lse = oracle.paged_kv_prefill_attention_f32(
        rows, kc, vc, np.full(batch, query_len, np.int32), np.full(batch, k.shape[2], np.int32), np.arange(batch, dtype=np.int32) * query_len,
        pages.reshape(batch, per).astype(np.uint32), batch=batch, total_query_tokens=batch * query_len, heads=heads, kv_heads=k.shape[1],
        head_dim=dim, block_size=4, block_table_batch_stride=per, causal=causal, scale=scale)
    assert np.abs(got.reshape(batch, query_len, heads, dim).transpose(0, 2, 1, 3) - out).max() <= OUT_TOLERANCE
    assert np.abs(got_lse.reshape(batch, query_len, heads).transpose(0, 2, 1) - lse).max() <= LSE_TOLERANCE


@pytest.mark.parametrize("splits", [1, 2, 7, 45])
def test_split_decode_and_reduce(splits):
    q, k, v, out, lse, scale, _ = load("decode")
    batch, heads, _, dim = q.shape
    per = -(-k.shape[2] // splits)
    attn, part_lse = oracle.fmha_decode_splitk_f32(q[:, :, 0], k.transpose(0, 2, 1, 3), v.transpose(0, 2, 1, 3), splits=splits,
                                                   kv_len_per_split=per, scale=scale)
    got = oracle.splitk_reduce_f32(attn, part_lse, batch=batch, heads=heads, splits=splits, head_dim=dim)
    assert np.abs(got - out[:, :, 0]).max() <= OUT_TOLERANCE
    if splits == 1:
        assert np.abs(part_lse[:, :, 0] - lse[:, :, 0]).max() <= LSE_TOLERANCE
