"""Dense f32 attention on the GPU against the CPU oracle, through the C ABI.  f32 tolerance: 1e-4."""
import numpy as np
import pytest
import torch

import oracle
from singe_amd.kernel import attention as A

pytestmark = pytest.mark.gpu

TOL = 1e-4


def test_dense_causal_f32_anchor():
    # batch 1, 8 heads, head_dim 64, seq 512, f32 N(0, 1), scale 1/8, causal, [B, H, L, D] order
    batch, heads, length, dim = 1, 8, 512, 64
    gen = torch.Generator(device="cuda")
    gen.manual_seed(0x51A6E + 1)
    q, k, v = (torch.randn((batch, heads, length, dim), generator=gen, device="cuda") for _ in range(3))
    out = torch.full_like(q, float("nan"))
    config = A.bhsd_config(batch, heads, heads, length, length, dim, 0.125, True)
    A.softcapped_window_attention_f32(None, out, q, k, v, A.SoftcappedWindowAttentionConfig(config))
    torch.cuda.synchronize()
    want = oracle.softcapped_window_attention_f32(q.cpu().numpy(), k.cpu().numpy(), v.cpu().numpy(), batch=batch,
                                                  query_len=length, key_len=length, heads=heads, kv_heads=heads,
                                                  head_dim=dim, scale=0.125, causal=True, threads=8)
    other = oracle.scaled_dot_product_attention_f32(q.cpu().numpy(), k.cpu().numpy(), v.cpu().numpy(), scale=0.125,
                                                    causal=True, threads=8)
    assert np.array_equal(want, other)  # the two CPU surfaces agree bit for bit on this shape
    gap = np.abs(out.cpu().numpy() - want)
    assert gap.max() <= TOL, gap.max()
    out2 = torch.empty_like(q)
    A.fmha_prefill_f32(None, out2, q, k, v, config)
    torch.cuda.synchronize()
    assert torch.equal(out, out2)


@pytest.mark.parametrize("dim", [4, 16, 33, 64, 96, 128, 200])
@pytest.mark.parametrize("causal", [False, True])
def test_prefill_f32_bshd_with_lse(dim, causal):
    batch, lq, lk, heads, kv_heads = 2, 37, 130, 4, 2
    gen = torch.Generator(device="cuda")
    gen.manual_seed(dim)
    q = torch.randn((batch, lq, heads, dim), generator=gen, device="cuda")
    k = torch.randn((batch, lk, kv_heads, dim), generator=gen, device="cuda")
    v = torch.randn((batch, lk, kv_heads, dim), generator=gen, device="cuda")
    out = torch.full_like(q, float("nan"))
    lse = torch.full((batch, heads, lq), float("nan"), device="cuda")
    scale = float(dim) ** -0.5
    A.fmha_prefill_lse_f32(None, out, lse, q, k, v, A.FmhaPrefillConfig.contiguous(batch, lq, lk, heads, kv_heads, dim, scale, causal))
    torch.cuda.synchronize()
    want, want_lse = oracle.fmha_prefill_lse_f32(q.cpu().numpy(), k.cpu().numpy(), v.cpu().numpy(), batch=batch,
                                                 query_len=lq, key_len=lk, heads=heads, kv_heads=kv_heads,
                                                 head_dim=dim, scale=scale, causal=causal, threads=4)
    assert np.abs(out.cpu().numpy() - want).max() <= TOL
    assert np.abs(lse.cpu().numpy() - want_lse).max() <= TOL


@pytest.mark.parametrize("window,cap", [(0, 30.0), (5, None), (16, 2.5)])
def test_softcapped_window_f32(window, cap):
    batch, heads, kv_heads, lq, lk, dim = 1, 4, 2, 70, 70, 32
    gen = torch.Generator(device="cuda")
    gen.manual_seed(7)
    q = torch.randn((batch, heads, lq, dim), generator=gen, device="cuda")
    k = torch.randn((batch, kv_heads, lk, dim), generator=gen, device="cuda")
    v = torch.randn((batch, kv_heads, lk, dim), generator=gen, device="cuda")
    out = torch.full_like(q, float("nan"))
    config = A.bhsd_config(batch, heads, kv_heads, lq, lk, dim, 0.3, True)
    A.softcapped_window_attention_f32(None, out, q, k, v, A.SoftcappedWindowAttentionConfig(config, window, cap))
    torch.cuda.synchronize()
    want = oracle.softcapped_window_attention_f32(q.cpu().numpy(), k.cpu().numpy(), v.cpu().numpy(), batch=batch,
                                                  query_len=lq, key_len=lk, heads=heads, kv_heads=kv_heads, head_dim=dim,
                                                  scale=0.3, causal=True, window_size=window, soft_cap=cap)
    assert np.abs(out.cpu().numpy() - want).max() <= TOL


@pytest.mark.parametrize("cap", [0.0, -2.5, float("inf"), float("nan")])
def test_softcapped_window_f32_refuses_a_cap_that_is_not_positive_and_finite(cap):
    # validate_softcapped_window_attention_config: a cap must be finite and above zero, and is looked at before the window
    from singe_amd import error
    batch, heads, lq, dim = 1, 2, 8, 32
    q = torch.zeros((batch, heads, lq, dim), device="cuda")
    out = torch.zeros_like(q)
    config = A.bhsd_config(batch, heads, heads, lq, lq, dim, 0.3, True)
    with pytest.raises(error.InvalidLength):
        A.softcapped_window_attention_f32(None, out, q, q, q, A.SoftcappedWindowAttentionConfig(config, 2 ** 40, cap))
