#!/usr/bin/env python3
"""Writes tests/golden/sdpa_fixtures.npz: small attention problems with the answers of a library routine,
torch.nn.functional.scaled_dot_product_attention on the CPU in float32 (and torch.logsumexp for the
log-sum-exps), so the CPU oracle is checked against an implementation that shares no code with it.

Nothing of the reference is imported or run.  Re-run only to add cases: the committed .npz is what the tests read
(numpy.load without pickling).  Arrays are named <case>/<tensor>.
"""
import os

import numpy as np
import torch
import torch.nn.functional as F

HERE = os.path.dirname(os.path.abspath(__file__))


def case(store, name, *, batch, heads, kv_heads, query_len, key_len, dim, scale, causal=None, mask=False, seed=0):
    """causal: None, "top_left" (key > query hidden) or "bottom_right" (key > key_len - query_len + query hidden)."""
    gen = torch.Generator().manual_seed(seed)
    q = torch.randn((batch, heads, query_len, dim), generator=gen)
    k = torch.randn((batch, kv_heads, key_len, dim), generator=gen)
    v = torch.randn((batch, kv_heads, key_len, dim), generator=gen)
    bias = torch.zeros((query_len, key_len))
    rows, cols = torch.arange(query_len)[:, None], torch.arange(key_len)[None, :]
    if causal == "top_left":
        bias = bias.masked_fill(cols > rows, float("-inf"))
    elif causal == "bottom_right":
        bias = bias.masked_fill(cols > rows + (key_len - query_len), float("-inf"))
    extra = None
    if mask:
        extra = torch.randn((batch, heads, query_len, key_len), generator=gen)
    total = bias[None, None] + (extra if extra is not None else 0.0)
    out = F.scaled_dot_product_attention(q, k, v, attn_mask=total.expand(batch, heads, query_len, key_len), scale=scale,
                                         enable_gqa=heads != kv_heads)
    group = heads // kv_heads
    scores = torch.einsum("bhqd,bhkd->bhqk", q, k.repeat_interleave(group, dim=1)) * scale + total
    store[f"{name}/query"] = q.numpy()
    store[f"{name}/key"] = k.numpy()
    store[f"{name}/value"] = v.numpy()
    store[f"{name}/out"] = out.numpy()
    store[f"{name}/lse"] = torch.logsumexp(scores, dim=-1).numpy()  # natural log
    store[f"{name}/scale"] = np.float32(scale)
    if extra is not None:
        store[f"{name}/mask"] = extra.numpy()


def main():
    store = {}
    case(store, "anchor_causal", batch=1, heads=4, kv_heads=4, query_len=48, key_len=48, dim=32, scale=0.125, causal="top_left", seed=1)
    case(store, "gqa_full", batch=2, heads=6, kv_heads=2, query_len=24, key_len=40, dim=16, scale=0.25, seed=2)
    case(store, "gqa_causal_square", batch=1, heads=8, kv_heads=2, query_len=33, key_len=33, dim=32, scale=32 ** -0.5, causal="top_left", seed=3)
    case(store, "chunk_bottom_right", batch=1, heads=4, kv_heads=2, query_len=9, key_len=50, dim=32, scale=32 ** -0.5, causal="bottom_right", seed=4)
    case(store, "prefix_top_left", batch=1, heads=4, kv_heads=1, query_len=20, key_len=37, dim=16, scale=0.3, causal="top_left", seed=5)
    case(store, "masked", batch=1, heads=3, kv_heads=3, query_len=12, key_len=17, dim=8, scale=0.5, mask=True, seed=6)
    case(store, "decode", batch=3, heads=8, kv_heads=2, query_len=1, key_len=45, dim=32, scale=0.125, seed=7)
    np.savez_compressed(os.path.join(HERE, "sdpa_fixtures.npz"), **store)
    print("wrote", len(store), "arrays")


if __name__ == "__main__":
    main()
