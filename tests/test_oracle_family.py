"""Pins of the oracle's restatements of the rest of the singe-kernel dense family (ragged packed prefill, windowed decode
with a log-sum-exp, prefill with sink logits, sliding-window attention over block-table keys): each against an independent
float64 restatement written from the definition, against closed forms, and, where two reference functions must agree on a
special case, against the oracle function that is already pinned, bit for bit."""
import numpy as np
import pytest

import oracle


def softmax_rows(scores, values, extra=None):
    """float64: weights of `scores` (optionally with one more logit `extra` that weighs nothing) times `values`."""
    scores = np.asarray(scores, dtype=np.float64)
    if scores.size == 0:
        return None, None
    largest = max(scores.max(), -np.inf if extra is None else extra)
    weights = np.exp(scores - largest)
    denom = weights.sum() + (0.0 if extra is None else np.exp(extra - largest))
    return (weights[:, None] * np.asarray(values, dtype=np.float64)).sum(axis=0) / denom, largest + np.log(denom)


def test_ragged_prefill_against_float64_and_per_sequence_prefill():
    rng = np.random.default_rng(1)
    heads, kv_heads, dim = 4, 2, 8
    lens_q, lens_kv, offsets = [3, 0, 5, 2], [3, 4, 9, 0], [0, 3, 7, 16]   # sequence 3 has queries and no keys
    tokens, kv_tokens = 18, 18
    q = rng.standard_normal((tokens, heads, dim)).astype(np.float32)
    k = rng.standard_normal((kv_tokens, kv_heads, dim)).astype(np.float32)
    v = rng.standard_normal((kv_tokens, kv_heads, dim)).astype(np.float32)
    for causal in (False, True):
        out, lse = oracle.ragged_kv_prefill_attention_f32(q, k, v, lens_q, lens_kv, offsets, causal=causal, scale=0.3)
        want, want_lse = np.zeros_like(out, dtype=np.float64), np.zeros_like(lse, dtype=np.float64)
        for b in range(4):
            for qi in range(lens_q[b]):
                for h in range(heads):
                    keys = [j for j in range(lens_kv[b]) if not (causal and j > qi)]
                    t = offsets[b] + qi
                    if not keys:
                        want_lse[t, h] = -1e20
                        continue
                    rows = [offsets[b] + j for j in keys]
                    scores = [0.3 * float(q[t, h].astype(np.float64) @ k[r, h // 2].astype(np.float64)) for r in rows]
                    want[t, h], want_lse[t, h] = softmax_rows(scores, v[rows, h // 2])
        empty = want_lse == -1e20
        assert np.abs(out - want).max() < 2e-6 and np.abs(lse - want_lse)[~empty].max() < 2e-6
        assert (lse[empty] == np.float32(-1e20)).all()
        assert (out[3:7] == 0).all() and (lse[3:7] == 0).all()  # tokens 3..6 belong to no sequence: zeros
        assert (out[16:18] == 0).all() and (lse[16:18] == np.float32(-1e20)).all()
        # Sequence 2 alone is a dense prefill of 5 queries over 9 keys: the pinned dense restatement gives the same bits.
        dense, dense_lse = oracle.fmha_prefill_lse_f32(q[7:12][None], k[7:16][None], v[7:16][None], batch=1, query_len=5, key_len=9,
                                                       heads=heads, kv_heads=kv_heads, head_dim=dim, scale=0.3, causal=causal)
        assert np.array_equal(dense[0], out[7:12]) and np.array_equal(dense_lse[0].T, lse[7:12])


def test_windowed_decode_is_the_last_row_of_windowed_attention():
    rng = np.random.default_rng(2)
    batch, heads, kv_heads, key_len, dim = 2, 4, 2, 37, 16
    q = rng.standard_normal((batch, heads, dim)).astype(np.float32)
    k = rng.standard_normal((batch, kv_heads, key_len, dim)).astype(np.float32)
    v = rng.standard_normal((batch, kv_heads, key_len, dim)).astype(np.float32)
    for window, cap in ((0, None), (5, None), (1, 3.0), (40, 0.7)):
        out, lse = oracle.softcapped_window_decode_lse_f32(q, k, v, scale=0.25, window_size=window, soft_cap=cap)
        for b in range(batch):
            for h in range(heads):
                keys = [j for j in range(key_len) if not (window > 0 and j + window < key_len - 1)]
                scores = np.array([0.25 * float(q[b, h].astype(np.float64) @ k[b, h // 2, j].astype(np.float64)) for j in keys])
                if cap is not None:
                    scores = np.tanh(scores / cap) * cap
                want, want_lse = softmax_rows(scores, v[b, h // 2, keys])
                assert np.abs(out[b, h] - want).max() < 2e-6 and abs(lse[b, h] - want_lse) < 2e-6
        # The same rows as the last query of the causal windowed prefill (cpu/attention.rs:1835-1925), bit for bit.
        queries = np.zeros((batch, heads, key_len, dim), dtype=np.float32)
        queries[:, :, -1] = q
        dense = oracle.softcapped_window_attention_f32(queries, k, v, batch=batch, query_len=key_len, key_len=key_len, heads=heads,
                                                       kv_heads=kv_heads, head_dim=dim, scale=0.25, causal=True, window_size=window,
                                                       soft_cap=cap)
        assert np.array_equal(dense[:, :, -1], out)
    single, single_lse = oracle.softcapped_window_decode_lse_f32(q, k[:, :, :1], v[:, :, :1], scale=0.25)
    assert np.array_equal(single, np.repeat(v[:, :, 0], 2, axis=1))  # one key: the output is its value


def test_sink_prefill_against_float64_and_the_sink_that_weighs_nothing():
    rng = np.random.default_rng(3)
    batch, query_len, key_len, heads, kv_heads, dim = 2, 6, 11, 4, 2, 8
    q = rng.standard_normal((batch, query_len, heads, dim)).astype(np.float32)
    k = rng.standard_normal((batch, key_len, kv_heads, dim)).astype(np.float32)
    v = rng.standard_normal((batch, key_len, kv_heads, dim)).astype(np.float32)
    sinks = rng.standard_normal(heads).astype(np.float32)
    for start_q, window, causal in ((0, 0, True), (5, 0, True), (5, 3, True), (2, 4, False), (0, 1, True), (9, 2, True)):
        out = oracle.attention_sink_prefill_f32(q, k, v, sinks, start_q=start_q, window=window, scale=0.4, causal=causal)
        for b in range(batch):
            for qi in range(query_len):
                position = start_q + qi
                start = 0 if window == 0 else max(position - (window - 1), 0)
                keys = [j for j in range(key_len) if not (causal and j > position) and not (window != 0 and j < start)]
                for h in range(heads):
                    scores = [0.4 * float(q[b, qi, h].astype(np.float64) @ k[b, j, h // 2].astype(np.float64)) for j in keys]
                    if keys:
                        want, _ = softmax_rows(scores, v[b, keys, h // 2], extra=float(sinks[h]))
                    else:
                        want = np.zeros(dim)
                    assert np.abs(out[b, qi, h] - want).max() < 2e-6, (start_q, window, causal, b, qi, h)
    # A sink of -inf weighs nothing in the denominator either: the plain causal prefill, bit for bit.
    none = np.full(heads, -np.inf, dtype=np.float32)
    plain, _ = oracle.fmha_prefill_lse_f32(q, k, v, batch=batch, query_len=query_len, key_len=key_len, heads=heads, kv_heads=kv_heads,
                                           head_dim=dim, scale=0.4, causal=True)
    assert np.array_equal(oracle.attention_sink_prefill_f32(q, k, v, none, scale=0.4, causal=True), plain)
    # A huge sink takes all the weight: outputs go to zero.
    huge = np.full(heads, 1e4, dtype=np.float32)
    assert np.abs(oracle.attention_sink_prefill_f32(q, k, v, huge, scale=0.4, causal=True)).max() == 0.0


def test_paged_sliding_window_is_the_dense_one_through_any_table():
    rng = np.random.default_rng(4)
    batch, query_len, key_len, heads, kv_heads, dim, block = 2, 5, 13, 4, 2, 8, 4
    blocks_per = (key_len + block - 1) // block
    physical = 11
    q = rng.standard_normal((batch, query_len, heads, dim)).astype(np.float32)
    k = rng.standard_normal((batch, key_len, kv_heads, dim)).astype(np.float32)
    v = rng.standard_normal((batch, key_len, kv_heads, dim)).astype(np.float32)
    table = rng.permutation(physical)[: batch * blocks_per].reshape(batch, blocks_per).astype(np.uint32)
    key_cache = rng.standard_normal((physical, block, kv_heads, dim)).astype(np.float32)
    value_cache = rng.standard_normal((physical, block, kv_heads, dim)).astype(np.float32)
    for b in range(batch):
        for j in range(key_len):
            key_cache[table[b, j // block], j % block] = k[b, j]
            value_cache[table[b, j // block], j % block] = v[b, j]
    for query_start, key_start, window, output_scale in ((8, 0, 4, 1.0), (8, 0, 100, 0.5), (3, 6, 2, 1.0), (0, 20, 3, 1.0)):
        dense = oracle.sliding_window_attention_f32(q, k, v, batch=batch, query_len=query_len, key_len=key_len, heads=heads,
                                                    kv_heads=kv_heads, head_dim=dim, query_start=query_start, key_start=key_start,
                                                    window=window, scale=0.35, output_scale=output_scale).reshape(q.shape)
        paged = oracle.sliding_window_attention_paged_kv_f32(q, key_cache, value_cache, table, key_len=key_len, query_start=query_start,
                                                             key_start=key_start, window=window, scale=0.35, output_scale=output_scale)
        assert np.array_equal(dense, paged)
    assert (oracle.sliding_window_attention_paged_kv_f32(q, key_cache, value_cache, table, key_len=key_len, query_start=0, key_start=20,
                                                         window=3, scale=0.35) == 0).all()  # every key lies after every query
    # A block id outside the cache hides its keys: the same as a dense call whose keys of that block are pushed out of
    # reach (scores of -inf cannot be asked of the dense form, so the check is against float64).
    broken = table.copy()
    broken[0, 1] = physical + 3
    got = oracle.sliding_window_attention_paged_kv_f32(q, key_cache, value_cache, broken, key_len=key_len, query_start=12, key_start=0,
                                                       window=100, scale=0.35)
    for qi in range(query_len):
        for h in range(heads):
            keys = [j for j in range(key_len) if j <= 12 + qi and j // block != 1]
            scores = [0.35 * float(q[0, qi, h].astype(np.float64) @ k[0, j, h // 2].astype(np.float64)) for j in keys]
            want, _ = softmax_rows(scores, v[0, keys, h // 2])
            assert np.abs(got[0, qi, h] - want).max() < 2e-6
