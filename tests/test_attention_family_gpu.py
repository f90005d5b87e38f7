"""The rest of the singe-kernel dense family on the GPU, through the C ABI, against the CPU oracle on the same seeded inputs:
softcapped_window_attention_{bf16,f16}, attention_sink_prefill_{f32,bf16,f16}, fmha_decode_lse_*, softcapped_window_decode_lse_*,
ragged_kv_prefill_attention_* and the sliding-window attention over dense, packed and block-table keys.  f32 within 1e-4,
bf16 within max-abs 2e-2 / mean-abs 2e-3, f16 within 5e-3 / 5e-4 (outputs; log-sum-exps within 1e-4 / 2e-2 / 5e-3)."""
import numpy as np
import pytest
import torch

import oracle
from singe_amd import error
from singe_amd.kernel import attention as A

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16, torch.float16]
BOUND = {torch.float32: (1e-4, 1e-4), torch.bfloat16: (2e-2, 2e-3), torch.float16: (5e-3, 5e-4)}


def close(got, want, dtype, what=""):
    got, want = got.float().cpu().numpy(), np.asarray(want, dtype=np.float32)
    assert np.isfinite(got).all(), what
    gap = np.abs(got - want)
    worst, mean = BOUND[dtype]
    assert gap.max(initial=0.0) <= worst and (gap.size == 0 or gap.mean() <= mean), (what, gap.max(), gap.mean())


def normal(shape, dtype, seed):
    generator = torch.Generator().manual_seed(seed)
    return torch.randn(shape, generator=generator).to(dtype).cuda()


def host(tensor):
    return tensor.float().cpu().numpy()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("head_dim,causal,window,cap", [
    (128, True, 0, 5.0), (128, True, 40, None), (128, True, 33, 2.5), (128, False, 17, None), (64, False, 50, 4.0),
    (128, False, 0, None), (40, True, 9, 3.0), (256, False, 6, None)])
def test_softcapped_window_attention_16_bit(dtype, head_dim, causal, window, cap):
    batch, heads, kv_heads, query_len, key_len = 2, 4, 2, 150, 150
    q = normal((batch, heads, query_len, head_dim), dtype, 1)
    k = normal((batch, kv_heads, key_len, head_dim), dtype, 2)
    v = normal((batch, kv_heads, key_len, head_dim), dtype, 3)
    out = torch.full_like(q, float("nan"))
    scale = head_dim ** -0.5
    config = A.SoftcappedWindowAttentionConfig(A.bhsd_config(batch, heads, kv_heads, query_len, key_len, head_dim, scale, causal), window, cap)
    run = A.softcapped_window_attention_bf16 if dtype == torch.bfloat16 else A.softcapped_window_attention_f16
    run(None, out, q, k, v, config)
    torch.cuda.synchronize()
    want = oracle.softcapped_window_attention_f32(host(q), host(k), host(v), batch=batch, query_len=query_len, key_len=key_len, heads=heads,
                                                  kv_heads=kv_heads, head_dim=head_dim, scale=scale, causal=causal, window_size=window,
                                                  soft_cap=cap, threads=8)
    close(out, want, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("head_dim,query_len,key_len,start_q,window,causal", [
    (64, 40, 40, 0, 0, True), (128, 130, 130, 0, 0, True), (128, 70, 200, 130, 0, True), (128, 70, 200, 130, 25, True),
    (32, 9, 50, 3, 4, False), (128, 160, 160, 0, 30, True), (96, 5, 5, 0, 1, True), (128, 3, 64, 200, 16, True)])
def test_attention_sink_prefill(dtype, head_dim, query_len, key_len, start_q, window, causal):
    batch, heads, kv_heads = 2, 4, 2
    q = normal((batch, query_len, heads, head_dim), dtype, 4)
    k = normal((batch, key_len, kv_heads, head_dim), dtype, 5)
    v = normal((batch, key_len, kv_heads, head_dim), dtype, 6)
    sinks = (normal((heads,), torch.float32, 7) * 3).to(dtype)
    out = torch.full_like(q, float("nan"))
    scale = head_dim ** -0.5
    config = A.AttentionSinkPrefillConfig.contiguous(batch, query_len, key_len, heads, kv_heads, head_dim, start_q, window, scale, causal)
    {torch.float32: A.attention_sink_prefill_f32, torch.bfloat16: A.attention_sink_prefill_bf16,
     torch.float16: A.attention_sink_prefill_f16}[dtype](None, out, q, k, v, sinks, config)
    torch.cuda.synchronize()
    want = oracle.attention_sink_prefill_f32(host(q), host(k), host(v), host(sinks), start_q=start_q, window=window, scale=scale, causal=causal)
    close(out, want, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("head_dim,key_len,heads,kv_heads", [(128, 300, 8, 2), (64, 1, 4, 4), (80, 77, 6, 3), (256, 40, 2, 1)])
def test_fmha_decode_lse(dtype, head_dim, key_len, heads, kv_heads):
    batch = 3
    q = normal((batch, heads, head_dim), dtype, 8)
    k = normal((batch, key_len, kv_heads, head_dim), dtype, 9)
    v = normal((batch, key_len, kv_heads, head_dim), dtype, 10)
    out = torch.full_like(q, float("nan"))
    lse = torch.full((batch, heads), float("nan"), device="cuda")
    scale = head_dim ** -0.5
    config = A.FmhaDecodeConfig.contiguous(batch, key_len, heads, kv_heads, head_dim, scale)
    {torch.float32: A.fmha_decode_lse_f32, torch.bfloat16: A.fmha_decode_lse_bf16, torch.float16: A.fmha_decode_lse_f16}[dtype](
        None, out, lse, q, k, v, config)
    torch.cuda.synchronize()
    want, want_lse = oracle.fmha_prefill_lse_f32(host(q)[:, None], host(k), host(v), batch=batch, query_len=1, key_len=key_len, heads=heads,
                                                 kv_heads=kv_heads, head_dim=head_dim, scale=scale, causal=False)
    close(out, want[:, 0], dtype)
    assert np.abs(lse.cpu().numpy() - want_lse[:, :, 0]).max() <= {torch.float32: 1e-4, torch.bfloat16: 2e-2, torch.float16: 5e-3}[dtype]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("head_dim,key_len,window,cap", [(128, 500, 0, None), (128, 500, 64, None), (64, 90, 1, 2.0), (128, 33, 200, 0.5),
                                                          (48, 129, 128, 6.0)])
def test_softcapped_window_decode_lse(dtype, head_dim, key_len, window, cap):
    batch, heads, kv_heads = 2, 8, 2
    q = normal((batch, heads, head_dim), dtype, 11)
    k = normal((batch, kv_heads, key_len, head_dim), dtype, 12)
    v = normal((batch, kv_heads, key_len, head_dim), dtype, 13)
    out = torch.full_like(q, float("nan"))
    lse = torch.full((batch, heads), float("nan"), device="cuda")
    scale = head_dim ** -0.5
    config = A.SoftcappedWindowDecodeConfig.bnsd_contiguous(batch, key_len, heads, kv_heads, head_dim, scale, window, cap)
    {torch.float32: A.softcapped_window_decode_lse_f32, torch.bfloat16: A.softcapped_window_decode_lse_bf16,
     torch.float16: A.softcapped_window_decode_lse_f16}[dtype](None, out, lse, q, k, v, config)
    torch.cuda.synchronize()
    want, want_lse = oracle.softcapped_window_decode_lse_f32(host(q), host(k), host(v), scale=scale, window_size=window, soft_cap=cap)
    close(out, want, dtype)
    assert np.abs(lse.cpu().numpy() - want_lse).max() <= {torch.float32: 1e-4, torch.bfloat16: 2e-2, torch.float16: 5e-3}[dtype]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("head_dim,heads,kv_heads", [(128, 4, 2), (64, 6, 6), (24, 2, 1)])
def test_ragged_kv_prefill(dtype, causal, head_dim, heads, kv_heads):
    lens_q = [5, 0, 130, 3, 70, 2]
    lens_kv = [5, 9, 200, 0, 70, 1]
    offsets = [0, 5, 14, 214, 217, 287]   # sequence 3 has queries and no keys; tokens 289 .. 291 belong to no sequence
    tokens, kv_tokens = 292, 289
    q = normal((tokens, heads, head_dim), dtype, 14)
    k = normal((kv_tokens, kv_heads, head_dim), dtype, 15)
    v = normal((kv_tokens, kv_heads, head_dim), dtype, 16)
    out = torch.full_like(q, 7.0)
    lse = torch.full((tokens, heads), 7.0, device="cuda")
    scale = head_dim ** -0.5
    config = A.RaggedKvPrefillAttentionConfig.contiguous(len(lens_q), tokens, kv_tokens, heads, kv_heads, head_dim, causal, scale)
    index = lambda values: torch.tensor(values, dtype=torch.int32, device="cuda")
    {torch.float32: A.ragged_kv_prefill_attention_f32, torch.bfloat16: A.ragged_kv_prefill_attention_bf16,
     torch.float16: A.ragged_kv_prefill_attention_f16}[dtype](None, out, lse, q, k, v, index(lens_q), index(lens_kv), index(offsets), config)
    torch.cuda.synchronize()
    want, want_lse = oracle.ragged_kv_prefill_attention_f32(host(q), host(k), host(v), lens_q, lens_kv, offsets, causal=causal, scale=scale)
    owned = np.zeros(tokens, dtype=bool)
    for offset, count in zip(offsets, lens_q):
        owned[offset:offset + count] = True
    close(out[torch.from_numpy(owned).cuda()], want[owned], dtype)
    got_lse = lse.cpu().numpy()
    empty = want_lse == np.float32(-1e20)
    assert (got_lse[empty & owned[:, None]] == np.float32(-1e20)).all()
    live = owned[:, None] & ~empty
    assert np.abs(got_lse[live] - want_lse[live]).max() <= {torch.float32: 1e-4, torch.bfloat16: 2e-2, torch.float16: 5e-3}[dtype]
    assert (out[~torch.from_numpy(owned).cuda()].float() == 7.0).all() and (got_lse[~owned] == 7.0).all()  # left alone


@pytest.mark.parametrize("head_dim,query_len,key_len,query_start,key_start,window,output_scale", [
    (64, 20, 60, 40, 0, 8, 1.0), (128, 33, 33, 0, 0, 1, 1.0), (32, 7, 90, 100, 20, 500, 0.25), (16, 5, 12, 0, 30, 4, 1.0),
    (200, 9, 40, 31, 0, 16, 2.0)])
def test_sliding_window_attention_dense_packed_and_paged(head_dim, query_len, key_len, query_start, key_start, window, output_scale):
    batch, heads, kv_heads, block = 2, 4, 2, 8
    q = normal((batch, query_len, heads, head_dim), torch.float32, 17)
    k = normal((batch, key_len, kv_heads, head_dim), torch.float32, 18)
    v = normal((batch, key_len, kv_heads, head_dim), torch.float32, 19)
    scale = head_dim ** -0.5
    config = A.SlidingWindowAttentionConfig.contiguous(batch, query_len, key_len, heads, kv_heads, head_dim, query_start, key_start, window,
                                                       scale).with_output_scale(output_scale)
    want = oracle.sliding_window_attention_f32(host(q), host(k), host(v), batch=batch, query_len=query_len, key_len=key_len, heads=heads,
                                               kv_heads=kv_heads, head_dim=head_dim, query_start=query_start, key_start=key_start,
                                               window=window, scale=scale, output_scale=output_scale).reshape(q.shape)
    out = torch.full_like(q, float("nan"))
    A.sliding_window_attention_f32(None, out, q, k, v, config)
    torch.cuda.synchronize()
    close(out, want, torch.float32, "dense")

    packed = torch.cat([torch.zeros(5, device="cuda"), q.flatten(), k.flatten(), torch.zeros(3, device="cuda"), v.flatten()])
    out.fill_(float("nan"))
    A.sliding_window_attention_packed_qkv_f32(None, out, packed, A.PackedQkvAttentionConfig(config, 5, 5 + q.numel(), 8 + q.numel() + k.numel()))
    torch.cuda.synchronize()
    close(out, want, torch.float32, "packed")

    blocks_per = (key_len + block - 1) // block
    physical = batch * blocks_per + 3
    table = torch.from_numpy(np.random.default_rng(5).permutation(physical)[: batch * blocks_per].reshape(batch, blocks_per).astype(np.int32)).cuda()
    key_cache = torch.randn((physical, block, kv_heads, head_dim), device="cuda")
    value_cache = torch.randn((physical, block, kv_heads, head_dim), device="cuda")
    for b in range(batch):
        for j in range(key_len):
            key_cache[table[b, j // block], j % block] = k[b, j]
            value_cache[table[b, j // block], j % block] = v[b, j]
    kv_features = kv_heads * head_dim
    paged = A.PagedKvAttentionConfig(config, block, physical, blocks_per, block * kv_features, block * kv_features)
    out.fill_(float("nan"))
    A.sliding_window_attention_paged_kv_f32(None, out, q, key_cache, value_cache, table, paged)
    torch.cuda.synchronize()
    close(out, want, torch.float32, "paged")
    # A block id outside the cache hides its keys (the reference kernel's block_valid test).
    broken = table.clone()
    broken[0, 0] = physical + 9
    out.fill_(float("nan"))
    A.sliding_window_attention_paged_kv_f32(None, out, q, key_cache, value_cache, broken, paged)
    torch.cuda.synchronize()
    want_broken = oracle.sliding_window_attention_paged_kv_f32(host(q), host(key_cache), host(value_cache), broken.cpu().numpy().view(np.uint32),
                                                               key_len=key_len, query_start=query_start, key_start=key_start, window=window,
                                                               scale=scale, output_scale=output_scale)
    close(out, want_broken, torch.float32, "paged, one block outside the cache")


def test_family_validation_on_the_device():
    q = torch.zeros((1, 4, 2, 64), device="cuda")
    config = A.SlidingWindowAttentionConfig.contiguous(1, 4, 4, 2, 2, 64, 0, 0, 0, 0.1)   # window 0
    with pytest.raises(error.InvalidLength):
        A.sliding_window_attention_f32(None, q, q, q, q, config)
    good = A.SlidingWindowAttentionConfig.contiguous(1, 4, 4, 2, 2, 64, 0, 0, 2, 0.1)
    with pytest.raises(error.LengthTooShort) as caught:
        A.sliding_window_attention_f32(None, q, q, q[:, :3].contiguous(), q, good)
    assert caught.value.name == "key"
    capped = A.SoftcappedWindowDecodeConfig.bnsd_contiguous(1, 4, 2, 2, 64, 0.1, 2, -1.0)   # a cap must be positive
    lse = torch.zeros((1, 2), device="cuda")
    with pytest.raises(error.InvalidLength):
        A.softcapped_window_decode_lse_f32(None, q[:, 0].contiguous(), lse, q[:, 0].contiguous(), q, q, capped)
