"""GPU parity of the f32 forms of the two block-table ops (paged_kv_decode_attention_f32,
paged_kv_prefill_attention_f32) against the oracle's restatement of the reference's CPU functions
(singe-kernel/src/cpu/attention.rs:1172-1341), through the C ABI.  Tolerance 1e-4 absolute."""
import numpy as np
import pytest
import torch

import oracle
from singe_amd import error
from singe_amd.kernel import attention as A

pytestmark = pytest.mark.gpu
TOLERANCE = 1e-4


def caches(gen, blocks, block_size, kv_heads, dim):
    shape = (blocks, block_size, kv_heads, dim)
    return gen.normal(size=shape).astype(np.float32), gen.normal(size=shape).astype(np.float32)


def table_for(gen, lengths, block_size, blocks, stride):
    order = gen.permutation(blocks)
    table = np.zeros((len(lengths), stride), dtype=np.uint32)
    at = 0
    for b, length in enumerate(lengths):
        need = -(-int(length) // block_size)
        table[b, :need] = order[at:at + need]
        at += need
    return table


@pytest.mark.parametrize("dim", [4, 16, 64, 128, 256])
@pytest.mark.parametrize("heads,kv_heads,block_size", [(8, 2, 16), (4, 4, 7), (12, 2, 1)])
def test_decode_matches_oracle(dim, heads, kv_heads, block_size):
    gen = np.random.default_rng(dim * 31 + heads)
    lengths = np.array([1, 150, 70, 0, 333], dtype=np.int32)  # an empty sequence gives zeros
    batch, blocks = len(lengths), 700 if block_size == 1 else 120
    stride = -(-int(lengths.max()) // block_size) + 2
    kc, vc = caches(gen, blocks, block_size, kv_heads, dim)
    table = table_for(gen, lengths, block_size, blocks, stride)
    q = gen.normal(size=(batch, heads, dim)).astype(np.float32)
    scale = dim ** -0.5
    want = oracle.paged_kv_decode_attention_f32(q, kc, vc, lengths, table, batch=batch, heads=heads, kv_heads=kv_heads,
                                                head_dim=dim, block_size=block_size, block_table_batch_stride=stride, scale=scale)
    config = A.PagedKvDecodeAttentionConfig(batch, heads, kv_heads, dim, block_size, blocks, stride, scale)
    out = torch.full((batch, heads, dim), 7.0, device="cuda")
    A.paged_kv_decode_attention_f32(None, out, *(torch.from_numpy(x).cuda() for x in (q, kc, vc, lengths, table.view(np.int32))), config)
    got = out.cpu().numpy()
    assert np.abs(got - want).max() < TOLERANCE
    assert not got[3].any()


def test_decode_long_sequences_and_wild_table_entries():
    gen = np.random.default_rng(11)
    batch, heads, kv_heads, dim, block_size, blocks = 3, 16, 4, 128, 16, 600
    lengths = np.array([4096, 513, 2222], dtype=np.int32)
    stride = 300
    kc, vc = caches(gen, blocks, block_size, kv_heads, dim)
    table = table_for(gen, lengths, block_size, blocks, stride)
    table[1, 40:] = 0xFFFFFFFF  # past the sequence: never read
    q = gen.normal(size=(batch, heads, dim)).astype(np.float32)
    want = oracle.paged_kv_decode_attention_f32(q, kc, vc, lengths, np.where(table == 0xFFFFFFFF, 0, table), batch=batch, heads=heads,
                                                kv_heads=kv_heads, head_dim=dim, block_size=block_size,
                                                block_table_batch_stride=stride, scale=0.1, threads=8)
    config = A.PagedKvDecodeAttentionConfig(batch, heads, kv_heads, dim, block_size, blocks, stride, 0.1)
    out = torch.empty((batch, heads, dim), device="cuda")
    A.paged_kv_decode_attention_f32(None, out, *(torch.from_numpy(x).cuda() for x in (q, kc, vc, lengths, table.view(np.int32))), config)
    assert np.abs(out.cpu().numpy() - want).max() < TOLERANCE


def test_decode_validation_and_workspace():
    gen = np.random.default_rng(12)
    batch, heads, kv_heads, dim, block_size, blocks, stride = 2, 4, 2, 64, 16, 8, 4
    kc, vc = caches(gen, blocks, block_size, kv_heads, dim)
    config = A.PagedKvDecodeAttentionConfig(batch, heads, kv_heads, dim, block_size, blocks, stride, 0.1)
    q = torch.zeros((batch, heads, dim), device="cuda")
    out = torch.zeros_like(q)
    lens = torch.tensor([5, 9], dtype=torch.int32, device="cuda")
    table = torch.zeros((batch, stride), dtype=torch.int32, device="cuda")
    tk, tv = torch.from_numpy(kc).cuda(), torch.from_numpy(vc).cuda()
    with pytest.raises(error.LengthTooShort) as info:
        A.paged_kv_decode_attention_f32(None, out, q, tk[:-1], tv, lens, table, config)
    assert info.value.name == "key_cache"
    with pytest.raises(error.LengthTooShort) as info:
        A.paged_kv_decode_attention_f32(None, out, q, tk, tv, lens, table, config, workspace=torch.empty(64, dtype=torch.uint8, device="cuda"))
    assert info.value.name == "workspace"
    odd = A.PagedKvDecodeAttentionConfig(batch, heads, kv_heads, 48, block_size, blocks, stride, 0.1)
    with pytest.raises(error.UnsupportedWidth):
        A.paged_kv_decode_attention_f32(None, torch.zeros((batch, heads, 48), device="cuda"), torch.zeros((batch, heads, 48), device="cuda"),
                                        torch.zeros((blocks, block_size, kv_heads, 48), device="cuda"),
                                        torch.zeros((blocks, block_size, kv_heads, 48), device="cuda"), lens, table, odd)
    with pytest.raises(error.InvalidLength):
        A.paged_kv_decode_attention_f32(None, out, q, tk, tv, lens, table,
                                        A.PagedKvDecodeAttentionConfig(batch, heads, 3, dim, block_size, blocks, stride, 0.1))


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("dim,heads,kv_heads,block_size", [(64, 8, 2, 16), (128, 4, 4, 7), (16, 6, 1, 1), (256, 10, 2, 32)])
def test_prefill_matches_oracle(causal, dim, heads, kv_heads, block_size):
    gen = np.random.default_rng(dim + heads + int(causal))
    # sequences in the reference's test shape: (queries, keys) with more keys than queries, fewer, none
    lens_q = np.array([1, 70, 20, 3], dtype=np.int32)
    lens_kv = np.array([150, 70, 9, 0], dtype=np.int32)
    offsets = np.array([0, 1, 73, 95], dtype=np.int32)  # tokens 71, 72 and 93, 94 belong to no sequence
    tokens, batch, blocks = 100, 4, 300
    stride = -(-int(lens_kv.max()) // block_size) + 1
    kc, vc = caches(gen, blocks, block_size, kv_heads, dim)
    table = table_for(gen, lens_kv, block_size, blocks, stride)
    q = gen.normal(size=(tokens, heads, dim)).astype(np.float32)
    scale = dim ** -0.5
    want, want_lse = oracle.paged_kv_prefill_attention_f32(
        q, kc, vc, lens_q, lens_kv, offsets, table, batch=batch, total_query_tokens=tokens, heads=heads, kv_heads=kv_heads,
        head_dim=dim, block_size=block_size, block_table_batch_stride=stride, causal=causal, scale=scale)
    config = A.PagedKvPrefillAttentionConfig(batch, tokens, heads, kv_heads, dim, block_size, blocks, stride, causal, scale)
    out = torch.full((tokens, heads, dim), 7.0, device="cuda")
    lse = torch.full((tokens, heads), 7.0, device="cuda")
    A.paged_kv_prefill_attention_f32(None, out, lse, *(torch.from_numpy(x).cuda() for x in (q, kc, vc, lens_q, lens_kv, offsets, table.view(np.int32))), config)
    got, got_lse = out.cpu().numpy(), lse.cpu().numpy()
    assert np.abs(got - want).max() < TOLERANCE
    empty = want_lse == np.float32(-1.0e20)
    assert empty[95:98].all() and np.array_equal(got_lse[empty], want_lse[empty])
    assert np.abs(got_lse[~empty] - want_lse[~empty]).max() < TOLERANCE
    # tokens of no sequence: zeros and an LSE of zero, as the CPU form's zero-filled outputs hold
    for token in (71, 72, 93, 94, 98, 99):
        assert not got[token].any() and not got_lse[token].any() and not want[token].any() and not want_lse[token].any()


def test_prefill_validation():
    config = A.PagedKvPrefillAttentionConfig(2, 10, 4, 2, 64, 16, 8, 4, True, 0.1)
    f = lambda *shape: torch.zeros(shape, device="cuda")
    i = lambda n: torch.zeros(n, dtype=torch.int32, device="cuda")
    args = [f(10, 4, 64), f(10, 4), f(10, 4, 64), f(8, 16, 2, 64), f(8, 16, 2, 64), i(2), i(2), i(2), torch.zeros((2, 4), dtype=torch.int32, device="cuda")]
    A.paged_kv_prefill_attention_f32(None, *args, config)
    short = list(args); short[1] = f(10, 3)
    with pytest.raises(error.LengthTooShort) as info:
        A.paged_kv_prefill_attention_f32(None, *short, config)
    assert info.value.name == "lse"
    short = list(args); short[7] = i(1)
    with pytest.raises(error.LengthTooShort) as info:
        A.paged_kv_prefill_attention_f32(None, *short, config)
    assert info.value.name == "actual_seq_offsets"
