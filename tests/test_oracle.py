"""Pins the CPU oracle before anything is checked against it.

Each test uses a vector the reference's own tests hold, or a fact the mathematics fixes
(closed forms, invariants, a float64 restatement that shares no code with the oracle), chosen so a
dropped term, a wrong sign or index, or a transposed operand fails at least one of them.
"""
import math

import numpy as np
import pytest
import torch

import oracle


def rng(seed):
    return np.random.default_rng(seed)


# ---- codecs -----------------------------------------------------------------------------------

def test_f8e4m3_value_known_answers():
    # singe-kernel/src/cpu/quantization.rs:297-316
    cases = [(0x00, 0.0), (0x01, 0.001953125), (0x07, 0.013671875), (0x08, 0.015625), (0x30, 0.5),
             (0x38, 1.0), (0x40, 2.0), (0x76, 224.0), (0x7E, 448.0), (0x81, -0.001953125),
             (0xB8, -1.0), (0xFE, -448.0)]
    for code, expected in cases:
        assert oracle.f8e4m3_value(code) == expected, hex(code)
    assert math.isnan(oracle.f8e4m3_value(0x7F))
    assert math.isnan(oracle.f8e4m3_value(0xFF))
    assert math.copysign(1.0, oracle.f8e4m3_value(0x80)) == -1.0


def test_f8e4m3_encode_known_answers_and_round_trip():
    # singe-codegen/src/interpret/tests.rs:274-312 (the bits torch's float8_e4m3fn cast gives)
    values = [0.0, -0.0, 1.0, 448.0, 449.0, 464.0, 480.0, 1000.0, math.inf, math.nan, 1e-9, 0.0019,
              57344.0, 61440.0, 70000.0]
    bits = [0x00, 0x80, 0x38, 0x7E, 0x7E, 0x7E, 0x7F, 0x7F, 0x7F, 0x7F, 0x00, 0x01, 0x7F, 0x7F, 0x7F]
    for value, expected in zip(values, bits):
        assert oracle.f8e4m3_encode(value) == expected, value
    for code in range(256):
        value = oracle.f8e4m3_value(code)
        if not math.isnan(value):
            assert oracle.f8e4m3_encode(value) == code, hex(code)


def test_f8e4m3_matches_torch_float8_e4m3fn():
    codes = torch.arange(256, dtype=torch.uint8)
    wide = codes.view(torch.float8_e4m3fn).to(torch.float32).numpy()
    table = oracle.f8e4m3_table()
    finite = ~np.isnan(table)
    assert np.array_equal(np.isnan(wide), np.isnan(table))
    assert np.array_equal(wide[finite], table[finite])
    samples = np.concatenate([rng(1).normal(size=4096) * 100, np.linspace(-460, 460, 2001)])
    ours = oracle.f8e4m3_encode_array(samples)
    theirs = torch.tensor(samples, dtype=torch.float64).to(torch.float32)
    # torch rounds through f32 first; keep the samples whose f32 and f64 values agree.
    same = theirs.double().numpy() == samples
    theirs = theirs.to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(ours[same], theirs[same])


def test_bf16_round_to_nearest_even():
    # prelude.rs:100-104, cross-checked with the library cast.
    values = np.concatenate([
        rng(2).normal(size=20000).astype(np.float32),
        np.array([0.0, -0.0, 1.0, 1.00390625, 1.01171875, 3.3895314e38, 1e-40, -1e-40, np.inf, -np.inf],
                 dtype=np.float32),
        # exact ties: odd and even low bits
        (np.arange(0x3F800000, 0x3F800000 + 0x40000, 0x8000, dtype=np.uint32)).view(np.float32),
    ])
    ours = oracle.f32_to_bf16(values)
    theirs = torch.from_numpy(values).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(ours, theirs)
    scalar = np.array([oracle.lib().oracle_f32_to_bf16(float(v)) for v in values[:3000]], dtype=np.uint16)
    assert np.array_equal(scalar, ours[:3000])
    assert np.array_equal(oracle.bf16_to_f32(ours), torch.from_numpy(values).to(torch.bfloat16).float().numpy())
    nan = oracle.f32_to_bf16(np.array([np.nan], dtype=np.float32))
    assert (nan[0] & 0x7FC0) == 0x7FC0


# ---- the reference's closed-form unit tests ---------------------------------------------------

def test_gqa_groups_are_contiguous():
    # singe-kernel/src/cpu/attention.rs:2235-2245: 4 heads over 2 kv heads -> [10, 10, 20, 20]
    out = oracle.sliding_window_attention_f32(
        np.ones(4), np.ones(2), np.array([10.0, 20.0]), batch=1, query_len=1, key_len=1, heads=4,
        kv_heads=2, head_dim=1, query_start=0, key_start=0, window=1, scale=1.0, output_scale=1.0)
    assert out.tolist() == [10.0, 10.0, 20.0, 20.0]
    # the same head map in every function that shares it
    common = dict(batch=1, heads=4, kv_heads=2, head_dim=1)
    q, k, v = np.ones((1, 4, 1)), np.ones((1, 1, 2, 1)), np.array([10.0, 20.0]).reshape(1, 1, 2, 1)
    dec = oracle.paged_kv_decode_attention_f32(q, k, v, [1], [0], block_size=1, block_table_batch_stride=1,
                                               scale=1.0, **common)
    assert dec.ravel().tolist() == [10.0, 10.0, 20.0, 20.0]
    st, pa, _ = oracle.paged_attention_f32(q, k, v, [0, 1], [0, 1], [0], [1], scale=1.0)
    assert st == 0 and pa.ravel().tolist() == [10.0, 10.0, 20.0, 20.0]
    out, _ = oracle.fmha_prefill_lse_f32(np.ones((1, 1, 4, 1)), np.ones((1, 1, 2, 1)),
                                         np.array([10.0, 20.0]).reshape(1, 1, 2, 1), batch=1, query_len=1,
                                         key_len=1, heads=4, kv_heads=2, head_dim=1, scale=1.0, causal=False)
    assert out.ravel().tolist() == [10.0, 10.0, 20.0, 20.0]
    sd = oracle.scaled_dot_product_attention_f32(np.ones((1, 4, 1, 1)), np.ones((1, 2, 1, 1)),
                                                 np.array([10.0, 20.0]).reshape(1, 2, 1, 1), scale=1.0)
    assert sd.ravel().tolist() == [10.0, 10.0, 20.0, 20.0]


def test_window_is_causal_left_not_symmetric():
    # singe-kernel/src/cpu/attention.rs:2247-2281: query at position 1, window 1, keys 0..2 -> [20]
    out = oracle.sliding_window_attention_f32(
        np.ones(1), np.ones(3), np.array([10.0, 20.0, 30.0]), batch=1, query_len=1, key_len=3, heads=1,
        kv_heads=1, head_dim=1, query_start=1, key_start=0, window=1, scale=1.0, output_scale=1.0)
    assert out.tolist() == [20.0]
    # singe's window rule: key + window <= position is hidden (registry/attributes/mod.rs:293-294).
    q = np.ones((1, 1, 3, 1))
    k = np.ones((1, 1, 3, 1))
    v = np.array([10.0, 20.0, 30.0]).reshape(1, 1, 3, 1)
    sd = oracle.scaled_dot_product_attention_f32(q, k, v, scale=1.0, causal=True, window=1)
    assert sd.ravel().tolist() == [10.0, 20.0, 30.0]
    sd = oracle.scaled_dot_product_attention_f32(q, k, v, scale=1.0, causal=True, window=2)
    assert np.allclose(sd.ravel(), [10.0, 15.0, 25.0], rtol=0, atol=1e-6)


def test_softmax_sum_and_lse_known_answer():
    # singe-codegen/src/interpret/tests.rs:217-272: logits [1, 2, -3], values [10, 20, 30].
    keys = np.array([[1.0, 0.0], [0.5, 1.5], [-1.0, -2.0]])
    values = np.array([[10.0, 0.0], [20.0, 0.0], [30.0, 0.0]])
    logits = np.array([1.0, 2.0, -3.0])
    total = np.exp(logits).sum()
    expected = (np.exp(logits) * np.array([10.0, 20.0, 30.0])).sum() / total
    q = np.ones((1, 1, 2))
    dec = oracle.paged_kv_decode_attention_f32(q, keys.reshape(3, 1, 1, 2), values.reshape(3, 1, 1, 2), [3],
                                               [0, 1, 2], batch=1, heads=1, kv_heads=1, head_dim=2,
                                               block_size=1, block_table_batch_stride=3, scale=1.0)
    assert abs(dec[0, 0, 0] - expected) < 1e-5
    out, lse = oracle.paged_kv_prefill_attention_f32(
        q, keys.reshape(3, 1, 1, 2), values.reshape(3, 1, 1, 2), [1], [3], [0], [0, 1, 2], batch=1,
        total_query_tokens=1, heads=1, kv_heads=1, head_dim=2, block_size=1, block_table_batch_stride=3,
        causal=False, scale=1.0)
    assert abs(out[0, 0, 0] - expected) < 1e-5 and abs(lse[0, 0] - math.log(total)) < 1e-5
    st, out, lse2 = oracle.paged_attention_f32(q, keys.reshape(3, 1, 1, 2), values.reshape(3, 1, 1, 2),
                                               [0, 1], [0, 3], [0, 1, 2], [1], scale=1.0)
    assert st == 0 and abs(out[0, 0, 0] - expected) < 1e-5
    assert abs(lse2[0, 0] - math.log(total) / math.log(2.0)) < 1e-5
    out, lse = oracle.fmha_prefill_lse_f32(q.reshape(1, 1, 1, 2), keys.reshape(1, 3, 1, 2),
                                           values.reshape(1, 3, 1, 2), batch=1, query_len=1, key_len=3,
                                           heads=1, kv_heads=1, head_dim=2, scale=1.0, causal=False)
    assert abs(out[0, 0, 0, 0] - expected) < 1e-5 and abs(lse[0, 0, 0] - math.log(total)) < 1e-5


def test_softmax_rows_known_answer():
    # singe-codegen/src/interpret/tests.rs:132-176: rows [1,2,3] and [-1,0,4]; one-hot values read the
    # weights out directly.
    for row in ([1.0, 2.0, 3.0], [-1.0, 0.0, 4.0]):
        keys = np.array(row).reshape(1, 1, 3, 1)
        q = np.ones((1, 1, 1, 1))
        values = np.eye(3).reshape(1, 1, 3, 3)
        out = oracle.scaled_dot_product_attention_f32(q, keys, values, scale=1.0)
        expected = np.exp(np.array(row) - max(row))
        expected /= expected.sum()
        assert np.abs(out.ravel() - expected).max() <= 1e-6


# ---- integer contract -------------------------------------------------------------------------

def test_gather_offsets_brute_force():
    # block = table[b*stride + key//bs]; offset = block*(bs*G*D) + (key%bs)*(G*D) + g*D
    gen = rng(3)
    for block_size, kv_heads, dim in [(1, 2, 4), (16, 8, 128), (7, 4, 64), (3, 1, 8)]:
        batch, stride, blocks = 5, 9, 40
        lens = gen.integers(0, stride * block_size + 1, size=batch)
        table = gen.permutation(blocks)[: batch * stride].reshape(batch, stride) if blocks >= batch * stride \
            else gen.integers(0, blocks, size=(batch, stride))
        for g in range(kv_heads):
            got = oracle.paged_gather_offsets(lens, table, kv_heads=kv_heads, head_dim=dim,
                                              block_size=block_size, block_table_batch_stride=stride, kv_head=g)
            want = [int(table[b, key // block_size]) * block_size * kv_heads * dim
                    + (key % block_size) * kv_heads * dim + g * dim
                    for b in range(batch) for key in range(int(lens[b]))]
            assert got.tolist() == want


def test_flashinfer_slots_known_index_set():
    # scripts/references/suites/conformance.py:1570-1582: cache [7, 4, 2, 16]
    slots, counts = oracle.paged_slots([0, 3, 5, 5], [4, 0, 6, 2, 5], [2, 3, 0], page_size=4)
    assert counts.tolist() == [10, 7, 0]
    assert slots.tolist() == [16, 17, 18, 19, 0, 1, 2, 3, 24, 25, 8, 9, 10, 11, 20, 21, 22]


def test_flashinfer_slots_reference_shuffle_recipe():
    # kernel_plan/source/tests.rs:853-889: pages[p] = (p*7+2) % page_count, sequences below
    sequences = [(1, 150), (70, 70), (20, 90), (3, 0)]
    for page_size in (1, 16, 7):
        page_offsets, last, needed = [0], [], 0
        for _, keys in sequences:
            pages = (keys + page_size - 1) // page_size
            needed += pages
            page_offsets.append(needed)
            last.append(0 if keys == 0 else keys - (pages - 1) * page_size)
        page_count = needed + 3
        table = [(p * 7 + 2) % page_count for p in range(needed)]
        slots, counts = oracle.paged_slots(page_offsets, table, last, page_size=page_size)
        assert counts.tolist() == [keys for _, keys in sequences]
        want = []
        for s, (_, keys) in enumerate(sequences):
            for key in range(keys):
                want.append(table[page_offsets[s] + key // page_size] * page_size + key % page_size)
        assert slots.tolist() == want
        assert len(set(table)) == len(table)  # the shuffle hands out distinct pages


VALID = dict(query_offsets=[0, 2], page_offsets=[0, 1], pages=[0], last_page_lengths=[2])
TOKENS, SLOTS, PAGES = 2, 4, 2


def paging_cases():
    # singe/tests/nn/paged_attention.rs:24-73,161-186
    invalid = [dict(query_offsets=[0, 3]), dict(query_offsets=[-1, 2]), dict(query_offsets=[2, 0]),
               dict(page_offsets=[0, 2]), dict(page_offsets=[-1, 1]), dict(pages=[PAGES]), dict(pages=[-1]),
               dict(last_page_lengths=[SLOTS + 1]), dict(last_page_lengths=[-1])]
    valid = [dict(), dict(last_page_lengths=[SLOTS]),
             dict(query_offsets=[0, 0], page_offsets=[0, 0], pages=[PAGES + 7], last_page_lengths=[-1])]
    return [({**VALID, **c}, 0) for c in valid] + [({**VALID, **c}, 1) for c in invalid]


@pytest.mark.parametrize("paging,expected", paging_cases())
def test_paging_error_contract(paging, expected):
    got = oracle.check_paged_values(paging["query_offsets"], paging["page_offsets"], paging["pages"],
                                    paging["last_page_lengths"], tokens=TOKENS, cache_pages=PAGES,
                                    page_size=SLOTS)
    assert got == expected
    q = np.zeros((TOKENS, 2, 16), dtype=np.float32)
    cache = np.zeros((PAGES, SLOTS, 2, 16), dtype=np.float32)
    status, _, _ = oracle.paged_attention_f32(q, cache, cache, paging["query_offsets"], paging["page_offsets"],
                                              paging["pages"], paging["last_page_lengths"], causal=True)
    assert status == expected


# ---- numerics: closed forms, invariants, an independent float64 restatement ---------------------

def dense_reference_f64(q, k, v, scale, visible):
    """q [L,D], k [S,D], v [S,Dv], visible [L,S] bool -> (out, lse natural); float64, no shared code."""
    s = (q.astype(np.float64) @ k.astype(np.float64).T) * scale
    s = np.where(visible, s, -np.inf)
    m = s.max(axis=1, keepdims=True, initial=-np.inf)
    m = np.where(np.isfinite(m), m, 0.0)
    p = np.exp(s - m)
    total = p.sum(axis=1, keepdims=True)
    with np.errstate(divide="ignore", invalid="ignore"):
        out = np.where(total > 0, (p @ v.astype(np.float64)) / total, 0.0)
        lse = np.where(total[:, 0] > 0, m[:, 0] + np.log(total[:, 0]), -np.inf)
    return out, lse


def make_paged(gen, batch, heads, kv_heads, dim, block_size, max_len, blocks, min_len=0):
    lens = gen.integers(min_len, max_len + 1, size=batch).astype(np.int32)
    stride = (max_len + block_size - 1) // block_size
    perm = gen.permutation(blocks)
    assert blocks >= batch * stride
    table = perm[: batch * stride].reshape(batch, stride).astype(np.uint32)
    q = gen.normal(size=(batch, heads, dim)).astype(np.float32)
    kc = gen.normal(size=(blocks, block_size, kv_heads, dim)).astype(np.float32)
    vc = gen.normal(size=(blocks, block_size, kv_heads, dim)).astype(np.float32)
    return q, kc, vc, lens, table, stride


def gather_dense(cache, table_row, length, block_size, kv_head):
    keys = np.arange(length)
    return cache[table_row[keys // block_size], keys % block_size, kv_head]


@pytest.mark.parametrize("heads,kv_heads,dim,block_size", [(8, 2, 64, 16), (4, 4, 32, 7), (8, 1, 128, 1)])
def test_paged_decode_matches_float64_and_literal(heads, kv_heads, dim, block_size):
    gen = rng(10 + dim + block_size)
    batch, max_len = 4, 90
    q, kc, vc, lens, table, stride = make_paged(gen, batch, heads, kv_heads, dim, block_size, max_len, 64 * 16 // block_size + 400)
    lens[0] = 0  # an empty sequence stays zero
    scale = 1.0 / math.sqrt(dim)
    kw = dict(batch=batch, heads=heads, kv_heads=kv_heads, head_dim=dim, block_size=block_size,
              block_table_batch_stride=stride, scale=scale)
    out = oracle.paged_kv_decode_attention_f32(q, kc, vc, lens, table, **kw)
    literal = oracle.paged_kv_decode_attention_f32(q, kc, vc, lens, table, literal=True, **kw)
    threaded = oracle.paged_kv_decode_attention_f32(q, kc, vc, lens, table, threads=4, **kw)
    assert np.array_equal(out, literal) and np.array_equal(out, threaded)
    assert not out[0].any()
    group = heads // kv_heads
    for b in range(batch):
        for h in range(heads):
            k = gather_dense(kc, table[b], lens[b], block_size, h // group)
            v = gather_dense(vc, table[b], lens[b], block_size, h // group)
            want, _ = dense_reference_f64(q[b, h][None], k, v, scale, np.ones((1, lens[b]), bool))
            assert np.abs(out[b, h] - want[0]).max() < 2e-6


def test_single_key_and_uniform_scores_closed_forms():
    gen = rng(20)
    dim = 16
    q = gen.normal(size=(1, 2, dim)).astype(np.float32)
    kc = gen.normal(size=(4, 4, 1, dim)).astype(np.float32)
    vc = gen.normal(size=(4, 4, 1, dim)).astype(np.float32)
    kw = dict(batch=1, heads=2, kv_heads=1, head_dim=dim, block_size=4, block_table_batch_stride=4, scale=0.3)
    one = oracle.paged_kv_decode_attention_f32(q, kc, vc, [1], [2, 0, 1, 3], **kw)
    assert np.array_equal(one[0, 0], vc[2, 0, 0]) and np.array_equal(one[0, 1], vc[2, 0, 0])
    # zero query: every score equal -> the mean of the values
    flat = oracle.paged_kv_decode_attention_f32(np.zeros_like(q), kc, vc, [11], [2, 0, 1, 3], **kw)
    rows = np.concatenate([vc[2, :, 0], vc[0, :, 0], vc[1, :3, 0]])
    assert np.abs(flat[0, 0] - rows.astype(np.float64).mean(axis=0)).max() < 1e-6
    # constant values: the weights sum to one
    ones = oracle.paged_kv_decode_attention_f32(q, kc, np.ones_like(vc), [13], [2, 0, 1, 3], **kw)
    assert np.abs(ones - 1.0).max() < 1e-6


def test_paged_equals_dense_and_block_permutation_is_invisible():
    # singe/tests/nn/cross_attention.rs:120-198 invariant; here bit for bit, since the arithmetic is shared.
    gen = rng(30)
    batch, heads, kv_heads, dim, block_size, max_len = 3, 4, 2, 32, 8, 40
    q, kc, vc, lens, table, stride = make_paged(gen, batch, heads, kv_heads, dim, block_size, max_len, 32, min_len=1)
    scale = 0.17
    kw = dict(batch=batch, heads=heads, kv_heads=kv_heads, head_dim=dim, block_size=block_size,
              block_table_batch_stride=stride, scale=scale)
    out = oracle.paged_kv_decode_attention_f32(q, kc, vc, lens, table, **kw)
    for b in range(batch):
        k = np.stack([gather_dense(kc, table[b], lens[b], block_size, g) for g in range(kv_heads)])[None]
        v = np.stack([gather_dense(vc, table[b], lens[b], block_size, g) for g in range(kv_heads)])[None]
        dense = oracle.scaled_dot_product_attention_f32(q[b][None, :, None, :], k, v, scale=scale)
        assert np.array_equal(dense[0, :, 0], out[b])
        bshd, _ = oracle.fmha_prefill_lse_f32(q[b][None, None], k.transpose(0, 2, 1, 3), v.transpose(0, 2, 1, 3),
                                              batch=1, query_len=1, key_len=int(lens[b]), heads=heads,
                                              kv_heads=kv_heads, head_dim=dim, scale=scale, causal=False)
        assert np.array_equal(bshd[0, 0], out[b])
    perm = gen.permutation(32)
    inverse = np.argsort(perm)
    moved = oracle.paged_kv_decode_attention_f32(q, kc[perm], vc[perm], lens, inverse[table].astype(np.uint32), **kw)
    assert np.array_equal(moved, out)
    # the FlashInfer form over the same pages gives the same rows (decode = one query per sequence)
    n = [(int(l) + block_size - 1) // block_size for l in lens]
    page_offsets = np.concatenate([[0], np.cumsum(n)])
    pages = np.concatenate([table[b, : n[b]] for b in range(batch)])
    last = [int(l) - (n[b] - 1) * block_size for b, l in enumerate(lens)]
    st, csr, lse2 = oracle.paged_attention_f32(q, kc, vc, np.arange(batch + 1), page_offsets, pages, last,
                                               scale=scale, causal=True)
    assert st == 0 and np.abs(csr - out).max() < 1e-6


@pytest.mark.parametrize("causal,window,softcap", [(False, None, None), (True, None, None), (True, 16, 30.0)])
@pytest.mark.parametrize("heads,kv_heads,dim,page_size", [(8, 2, 64, 1), (8, 1, 128, 16), (4, 4, 64, 7)])
def test_paged_attention_bottom_right_causal_matches_float64(heads, kv_heads, dim, page_size, causal, window, softcap):
    # shapes and options of kernel_plan/source/tests.rs:830-889; rule position = keys - queries + q
    # (normalization/attention.rs:482-488)
    sequences = [(1, 150), (70, 70), (20, 90), (3, 0)]
    query_offsets, page_offsets, last, needed = [0], [0], [], 0
    for queries, keys in sequences:
        query_offsets.append(query_offsets[-1] + queries)
        pages = (keys + page_size - 1) // page_size
        needed += pages
        page_offsets.append(needed)
        last.append(0 if keys == 0 else keys - (pages - 1) * page_size)
    page_count = needed + 3
    table = [(p * 7 + 2) % page_count for p in range(needed)]
    tokens = query_offsets[-1]

    def values(shape, seed):
        count = int(np.prod(shape))
        idx = np.arange(count, dtype=np.int64)
        return (((idx * 37 + seed * 11) % 41).astype(np.float32) / 20.0 - 1.0).reshape(shape)

    q = values((tokens, heads, dim), 1)
    kc = values((page_count, page_size, kv_heads, dim), 2)
    vc = values((page_count, page_size, kv_heads, dim), 3)
    st, out, lse2 = oracle.paged_attention_f32(q, kc, vc, query_offsets, page_offsets, table, last,
                                               causal=causal, window=window, softcap=softcap, threads=4)
    assert st == 0
    scale = 1.0 / math.sqrt(dim)
    group = heads // kv_heads
    kflat = kc.reshape(-1, kv_heads, dim)
    vflat = vc.reshape(-1, kv_heads, dim)
    for s, (queries, keys) in enumerate(sequences):
        slot = np.array([table[page_offsets[s] + key // page_size] * page_size + key % page_size
                         for key in range(keys)], dtype=np.int64)
        position = np.maximum(keys + np.arange(queries) - queries, 0)[:, None]
        key_index = np.arange(keys)[None, :]
        visible = np.ones((queries, keys), bool)
        if causal:
            visible &= key_index <= position
        if window is not None:
            visible &= key_index + window > position
        for h in range(heads):
            rows = q[query_offsets[s]: query_offsets[s + 1], h]
            k = kflat[slot, h // group] if keys else np.zeros((0, dim), np.float32)
            v = vflat[slot, h // group] if keys else np.zeros((0, dim), np.float32)
            if softcap is None:
                want, want_lse = dense_reference_f64(rows, k, v, scale, visible)
            else:
                s64 = np.tanh((rows.astype(np.float64) @ k.astype(np.float64).T) * scale / softcap) * softcap
                s64 = np.where(visible, s64, -np.inf)
                m = s64.max(axis=1, keepdims=True) if keys else np.zeros((queries, 1))
                p = np.exp(s64 - m)
                total = p.sum(axis=1, keepdims=True)
                with np.errstate(divide="ignore", invalid="ignore"):
                    want = np.where(total > 0, (p @ v.astype(np.float64)) / total, 0.0)
                    want_lse = m[:, 0] + np.log(total[:, 0])
            got = out[query_offsets[s]: query_offsets[s + 1], h]
            got_lse = lse2[query_offsets[s]: query_offsets[s + 1], h]
            assert np.abs(got - want).max() < 5e-6
            if keys == 0:
                assert np.all(np.isneginf(got_lse)) and not got.any()
            else:
                assert np.abs(got_lse - want_lse / math.log(2.0)).max() < 1e-5


def test_dense_causal_matches_torch_sdpa_and_both_dense_oracles_agree():
    # The workload shape of the f32 correctness anchor, shortened: [1, 8, L, 64], scale 1/8, causal.
    gen = rng(40)
    batch, heads, length, dim = 1, 8, 96, 64
    q, k, v = (gen.normal(size=(batch, heads, length, dim)).astype(np.float32) for _ in range(3))
    a = oracle.softcapped_window_attention_f32(q, k, v, batch=batch, query_len=length, key_len=length, heads=heads,
                                               kv_heads=heads, head_dim=dim, scale=0.125, causal=True, threads=4)
    b = oracle.scaled_dot_product_attention_f32(q, k, v, scale=0.125, causal=True, threads=4)
    assert np.array_equal(a, b)
    t = torch.nn.functional.scaled_dot_product_attention(
        torch.from_numpy(q).double(), torch.from_numpy(k).double(), torch.from_numpy(v).double(),
        is_causal=True, scale=0.125).float().numpy()
    assert np.abs(a - t).max() < 2e-6
    # BSHD prefill over the same data, with LSE
    c, lse = oracle.fmha_prefill_lse_f32(q.transpose(0, 2, 1, 3), k.transpose(0, 2, 1, 3), v.transpose(0, 2, 1, 3),
                                         batch=batch, query_len=length, key_len=length, heads=heads,
                                         kv_heads=heads, head_dim=dim, scale=0.125, causal=True, threads=4)
    assert np.array_equal(c.transpose(0, 2, 1, 3), a)
    s = np.einsum("bhqd,bhkd->bhqk", q.astype(np.float64), k.astype(np.float64)) * 0.125
    s = np.where(np.tril(np.ones((length, length), bool)), s, -np.inf)
    want_lse = np.log(np.exp(s - s.max(-1, keepdims=True)).sum(-1)) + s.max(-1)
    assert np.abs(lse - want_lse).max() < 1e-5


def test_sdpa_mask_sinks_key_lengths_against_float64():
    gen = rng(41)
    batch, heads, kv_heads, lq, lk, dim = 2, 4, 2, 5, 9, 16
    q = gen.normal(size=(batch, heads, lq, dim)).astype(np.float32)
    k = gen.normal(size=(batch, kv_heads, lk, dim)).astype(np.float32)
    v = gen.normal(size=(batch, kv_heads, lk, dim)).astype(np.float32)
    mask = gen.normal(size=(1, 1, lq, lk)).astype(np.float32)
    mask[0, 0, 2, 3] = -np.inf
    sinks = gen.normal(size=(heads,)).astype(np.float32)
    lengths = np.array([9, 4], dtype=np.int32)
    got = oracle.scaled_dot_product_attention_f32(q, k, v, scale=0.25, mask=mask, sinks=sinks, key_lengths=lengths)
    for b in range(batch):
        for h in range(heads):
            s = (q[b, h].astype(np.float64) @ k[b, h // 2].astype(np.float64).T) * 0.25 + mask[0, 0]
            s[:, lengths[b]:] = -np.inf
            m = np.maximum(s.max(axis=1), sinks[h])[:, None]
            p = np.exp(s - m)
            total = p.sum(axis=1, keepdims=True) + np.exp(sinks[h] - m)
            want = (p @ v[b, h // 2].astype(np.float64)) / total
            assert np.abs(got[b, h] - want).max() < 2e-6


def test_top_left_causal_prefill_and_empty_row_lse():
    # singe-kernel's paged prefill hides key > query with no prefix offset (cpu/attention.rs:1282) and
    # writes -1e20 for a row that sees nothing (:1304).
    gen = rng(50)
    heads, kv_heads, dim, block_size = 4, 2, 16, 4
    lens_q, lens_kv = [3, 2], [6, 0]
    offsets = [0, 3]
    q = gen.normal(size=(5, heads, dim)).astype(np.float32)
    kc = gen.normal(size=(8, block_size, kv_heads, dim)).astype(np.float32)
    vc = gen.normal(size=(8, block_size, kv_heads, dim)).astype(np.float32)
    table = np.array([[5, 2], [1, 7]], dtype=np.uint32)
    out, lse = oracle.paged_kv_prefill_attention_f32(q, kc, vc, lens_q, lens_kv, offsets, table, batch=2,
                                                     total_query_tokens=5, heads=heads, kv_heads=kv_heads,
                                                     head_dim=dim, block_size=block_size,
                                                     block_table_batch_stride=2, causal=True, scale=0.25)
    assert np.all(lse[3:] == np.float32(-1.0e20)) and not out[3:].any()
    for h in range(heads):
        k = gather_dense(kc, table[0], 6, block_size, h // 2)
        v = gather_dense(vc, table[0], 6, block_size, h // 2)
        visible = np.arange(6)[None, :] <= np.arange(3)[:, None]
        want, want_lse = dense_reference_f64(q[:3, h], k, v, 0.25, visible)
        assert np.abs(out[:3, h] - want).max() < 2e-6 and np.abs(lse[:3, h] - want_lse).max() < 1e-5


def test_splitk_reduce_recovers_the_unsplit_row():
    gen = rng(60)
    batch, heads, dim, keys, splits = 2, 3, 8, 40, 4
    q = gen.normal(size=(batch, heads, dim))
    k = gen.normal(size=(batch, heads, keys, dim))
    v = gen.normal(size=(batch, heads, keys, dim))
    attn = np.zeros((batch, heads, splits, dim))
    lse = np.zeros((batch, heads, splits))
    full = np.zeros((batch, heads, dim))
    for b in range(batch):
        for h in range(heads):
            want, _ = dense_reference_f64(q[b, h][None], k[b, h], v[b, h], 0.3, np.ones((1, keys), bool))
            full[b, h] = want[0]
            for s in range(splits):
                part = slice(s * 10, (s + 1) * 10)
                o, l = dense_reference_f64(q[b, h][None], k[b, h, part], v[b, h, part], 0.3, np.ones((1, 10), bool))
                attn[b, h, s], lse[b, h, s] = o[0], l[0]
    got = oracle.splitk_reduce_f32(attn, lse, batch=batch, heads=heads, splits=splits, head_dim=dim)
    assert np.abs(got - full).max() < 2e-6


def test_fp8_cache_dequantises_to_bf16_values():
    gen = rng(70)
    codes = gen.integers(0, 256, size=(3, 4, 2, 8)).astype(np.uint8)
    codes[(codes & 0x7F) == 0x7F] = 0x7E
    scales = np.abs(gen.normal(size=(3, 2))).astype(np.float32) + 0.01
    got = oracle.dequantize_f8e4m3_cache(codes, scales)
    table = oracle.f8e4m3_table()
    want = torch.from_numpy(table[codes] * scales[:, None, :, None]).to(torch.bfloat16).float().numpy()
    assert np.array_equal(got, want)


# ---- rotation, cache append and the paging bridge ---------------------------------------------------

def test_rotary_embedding_closed_forms():
    """Angle 0 is the identity, a quarter turn maps (even, odd) to (-odd, even), rotation keeps each
    pair's length, and positions repeat with the sequence length (cpu/normalization/attention.rs:172-185)."""
    rng = np.random.default_rng(3)
    x = rng.standard_normal((2, 3, 5, 8)).astype(np.float32)
    pairs = 3  # the last pair of each row is not rotated
    zeros, ones = np.zeros((5, pairs), np.float32), np.ones((5, pairs), np.float32)
    assert np.array_equal(oracle.rotary_embedding_f32(x, ones, zeros), x)
    quarter = oracle.rotary_embedding_f32(x, zeros, ones)
    assert np.array_equal(quarter[..., 0:6:2], -x[..., 1:6:2]) and np.array_equal(quarter[..., 1:6:2], x[..., 0:6:2])
    assert np.array_equal(quarter[..., 6:], x[..., 6:])
    angle = rng.uniform(0, 6.28, (5, pairs)).astype(np.float32)
    turned = oracle.rotary_embedding_f32(x, np.cos(angle), np.sin(angle))
    lengths = lambda v: v[..., 0:6:2] ** 2 + v[..., 1:6:2] ** 2
    assert np.allclose(lengths(turned), lengths(x), rtol=1e-5)
    want = x[..., 0:6:2] * np.cos(angle) - x[..., 1:6:2] * np.sin(angle)  # position = row % sequence
    assert np.allclose(turned[..., 0:6:2], want, atol=1e-6)


def test_rotary_cache_write_closed_forms():
    """Half-split pairs, cells chosen by (page, slot), untouched cells kept, negative indices counted from the
    end, an index outside the cache reported and skipped (rotary_cache.rs:92-185, 367-400)."""
    rng = np.random.default_rng(5)
    tokens, heads, groups, dim, pages, slots = 4, 3, 2, 8, 3, 4
    q = rng.standard_normal((tokens, heads, dim)).astype(np.float32)
    k = rng.standard_normal((tokens, groups, dim)).astype(np.float32)
    v = rng.standard_normal((tokens, groups, dim)).astype(np.float32)
    kc = rng.standard_normal((pages, slots, groups, dim)).astype(np.float32)
    vc = rng.standard_normal((pages, slots, groups, dim)).astype(np.float32)
    angle = rng.uniform(0, 6.28, (tokens, dim // 2)).astype(np.float32)
    page_index, slot_index = [2, 0, -1, 1], [1, 3, -4, 2]
    status, q_out, kc_out, vc_out = oracle.rotary_cache_write_f32(q, k, v, np.cos(angle), np.sin(angle), page_index, slot_index, kc, vc)
    assert status == 0
    half = dim // 2
    want = np.concatenate([q[..., :half] * np.cos(angle)[:, None] - q[..., half:] * np.sin(angle)[:, None],
                           q[..., half:] * np.cos(angle)[:, None] + q[..., :half] * np.sin(angle)[:, None]], axis=-1)
    assert np.allclose(q_out, want, atol=1e-6)
    cells = [(2, 1), (0, 3), (2, 0), (1, 2)]  # -1 -> page 2, -4 -> slot 0
    touched = np.zeros((pages, slots), bool)
    for t, (p, s) in enumerate(cells):
        touched[p, s] = True
        assert np.array_equal(vc_out[p, s], v[t])
        assert np.allclose(np.linalg.norm(kc_out[p, s], axis=-1), np.linalg.norm(k[t], axis=-1), rtol=1e-5)
    assert np.array_equal(kc_out[~touched], kc[~touched]) and np.array_equal(vc_out[~touched], vc[~touched])
    # identity angles + RMS norm with a weight: x / rms(x) * w
    weight = rng.standard_normal(dim).astype(np.float32)
    ones, zeros = np.ones((tokens, half), np.float32), np.zeros((tokens, half), np.float32)
    _, q_norm, _, _ = oracle.rotary_cache_write_f32(q, k, v, ones, zeros, page_index, slot_index, kc, vc, query_norm=(1e-6, weight))
    rms = np.sqrt((q.astype(np.float64) ** 2).mean(-1, keepdims=True) + 1e-6)
    assert np.allclose(q_norm, q / rms * weight, atol=1e-5)
    # out of range: reported, that token's cells untouched, the others written
    status, _, kc_bad, _ = oracle.rotary_cache_write_f32(q, k, v, ones, zeros, [2, 3, -1, 1], slot_index, kc, vc)
    assert status == 1 and np.array_equal(kc_bad[0, 3], kc[0, 3]) and np.array_equal(kc_bad[2, 1], k[0])


def test_paging_indices_against_brute_force():
    """The FlashInfer index set of the reference's generator (conformance.py:1570-1582) and its shuffle
    recipe (kernel_plan/source/tests.rs:853-889) through the CSR -> table conversion."""
    status, packed, qlen, klen, table = oracle.paging_indices([0, 1, 6, 9], [0, 3, 5, 5], [4, 0, 6, 2, 5], [2, 3, 0], tokens=9,
                                                              page_size=4, cache_pages=7, width=4, row_elements=32)
    assert status == 0
    assert packed.tolist() == [0, 32, 192, 288] and qlen.tolist() == [1, 5, 3] and klen.tolist() == [10, 7, 0]
    assert table.tolist() == [[4, 0, 6, 0], [2, 5, 0, 0], [0, 0, 0, 0]]
    for page_size in (1, 16, 7):
        sequences = [(1, 150), (70, 70), (20, 90), (3, 0)]
        qo, po, last = [0], [0], []
        for queries, keys in sequences:
            qo.append(qo[-1] + queries)
            n = -(-keys // page_size)
            po.append(po[-1] + n)
            last.append(0 if keys == 0 else keys - (n - 1) * page_size)
        count = po[-1]
        pages = [(p * 7 + 2) % count for p in range(count)]
        width = max(b - a for a, b in zip(po, po[1:]))
        status, packed, qlen, klen, table = oracle.paging_indices(qo, po, pages, last, tokens=qo[-1], page_size=page_size,
                                                                  cache_pages=count, width=width, row_elements=1)
        assert status == 0 and klen.tolist() == [k for _, k in sequences] and qlen.tolist() == [q for q, _ in sequences]
        for s, (a, b) in enumerate(zip(po, po[1:])):
            assert table[s, :b - a].tolist() == pages[a:b] and not table[s, b - a:].any()
    # the reference's invalid tuples are refused here too
    assert oracle.paging_indices([0, 1, 3], [0, 2, 3], [1, 0, 3], [2, 1], tokens=3, page_size=4, cache_pages=3, width=2, row_elements=1)[0] == 1
    assert oracle.paging_indices([0, 2, 1], [0, 2, 3], [1, 0, 2], [2, 1], tokens=3, page_size=4, cache_pages=3, width=2, row_elements=1)[0] == 1


def test_paged_mla_attention_against_a_float64_restatement_and_closed_forms():
    """The latent-attention oracle has no numeric fixture in the reference: it is pinned by an independent numpy
    float64 restatement (a dropped positional term, a wrong slot or a wrong causal end fails it), by single-key rows
    (out == that latent row, lse == score / ln 2) and by the paging error contract."""
    gen = np.random.default_rng(5)
    tokens, heads, latent, positional, pages, slots = 7, 3, 24, 8, 9, 4
    q = gen.standard_normal((tokens, heads, latent)).astype(np.float32)
    qp = gen.standard_normal((tokens, heads, positional)).astype(np.float32)
    lc = gen.standard_normal((pages, slots, latent)).astype(np.float32)
    pc = gen.standard_normal((pages, slots, positional)).astype(np.float32)
    qo, po, table, last = [0, 3, 4, 7], [0, 3, 3, 7], [8, 0, 3, 5, 1, 2, 6], [2, 0, 1]
    for causal in (False, True):
        status, out, lse = oracle.paged_mla_attention(q, qp, lc, pc, qo, po, table, last, causal=causal, scale=None if causal else 0.3)
        assert status == 0
        scale = 1.0 / np.sqrt(latent + positional) if causal else 0.3
        for s in range(3):
            own = table[po[s]:po[s + 1]]
            keys = 0 if not own else (len(own) - 1) * slots + last[s]
            rows = np.concatenate([lc[p] for p in own])[:keys].astype(np.float64) if own else np.zeros((0, latent))
            tails = np.concatenate([pc[p] for p in own])[:keys].astype(np.float64) if own else np.zeros((0, positional))
            count = qo[s + 1] - qo[s]
            for t in range(qo[s], qo[s + 1]):
                position = max(keys + (t - qo[s]) - count, 0)
                end = min(keys, position + 1) if causal else keys
                for h in range(heads):
                    if end == 0:
                        assert not out[t, h].any() and np.isneginf(lse[t, h])
                        continue
                    scores = (rows[:end] @ q[t, h].astype(np.float64) + tails[:end] @ qp[t, h].astype(np.float64)) * scale
                    weights = np.exp(scores - scores.max())
                    assert np.allclose(out[t, h], (weights / weights.sum()) @ rows[:end], atol=2e-6)
                    assert abs(lse[t, h] - (scores.max() + np.log(weights.sum())) / np.log(2.0)) < 1e-5
    # A single key: the output is its latent row, the LSE its score in base two.
    status, out, lse = oracle.paged_mla_attention(q[:1], qp[:1], lc, pc, [0, 1], [0, 1], [4], [1], scale=0.5)
    assert status == 0 and np.array_equal(out[0, 0], lc[4, 0])
    score = (np.dot(q[0, 0].astype(np.float64), lc[4, 0]) + np.dot(qp[0, 0].astype(np.float64), pc[4, 0])) * 0.5
    assert abs(lse[0, 0] - score / np.log(2.0)) < 1e-5
    # The paging error contract is the op's (spec/neural/attention.rs:372-406).
    assert oracle.paged_mla_attention(q[:1], qp[:1], lc, pc, [0, 1], [0, 1], [pages], [1])[0] == 1
    assert oracle.paged_mla_attention(q[:1], qp[:1], lc, pc, [0, 2], [0, 1], [0], [1])[0] == 1


@pytest.mark.parametrize("causal", [True, False])
def test_prefill_literal_loop_equals_the_hoisted_one_bit_for_bit(causal):
    """The benchmark's single-thread CPU line keeps the reference's loop shape (cpu/attention.rs:1776-1830: the weight
    re-evaluated per output dimension); it must give the bits of the restatement every parity test uses, on the rows it
    is asked for, and leave the others alone."""
    rng = np.random.default_rng(17)
    batch, query_len, key_len, heads, kv_heads, dim = 2, 9, 13, 4, 2, 8
    q = rng.standard_normal((batch, query_len, heads, dim)).astype(np.float32)
    k = rng.standard_normal((batch, key_len, kv_heads, dim)).astype(np.float32)
    v = rng.standard_normal((batch, key_len, kv_heads, dim)).astype(np.float32)
    kw = dict(batch=batch, query_len=query_len, key_len=key_len, heads=heads, kv_heads=kv_heads, head_dim=dim, scale=0.3, causal=causal)
    want, want_lse = oracle.fmha_prefill_lse_f32(q, k, v, **kw)
    got, got_lse = oracle.fmha_prefill_lse_f32_literal(q, k, v, **kw)
    assert np.array_equal(got, want) and np.array_equal(got_lse, want_lse)
    part, part_lse = oracle.fmha_prefill_lse_f32_literal(q, k, v, row_first=3, row_count=4, **kw)
    assert np.array_equal(part[:, 3:7], want[:, 3:7]) and np.array_equal(part_lse[:, :, 3:7], want_lse[:, :, 3:7])
    assert not part[:, :3].any() and not part[:, 7:].any()
