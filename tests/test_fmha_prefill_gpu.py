"""Dense flash-attention prefill on the GPU against the CPU oracle (fmha_prefill_lse_f32 restated),
through the C ABI.  bf16 outputs: max-abs 2e-2, mean-abs 2e-3; natural-log LSE within 2e-3."""
import numpy as np
import pytest
import torch

import oracle
from singe_amd import error
from singe_amd.kernel import attention as A

pytestmark = pytest.mark.gpu

MAX_ABS, MEAN_ABS, LSE_ABS = 2e-2, 2e-3, 2e-3


def make(batch, query_len, key_len, heads, kv_heads, seed, dim=128):
    gen = torch.Generator(device="cuda")
    gen.manual_seed(seed)
    q = torch.randn((batch, query_len, heads, dim), generator=gen, device="cuda").to(torch.bfloat16)
    k = torch.randn((batch, key_len, kv_heads, dim), generator=gen, device="cuda").to(torch.bfloat16)
    v = torch.randn((batch, key_len, kv_heads, dim), generator=gen, device="cuda").to(torch.bfloat16)
    return q, k, v


def run(q, k, v, causal, scale=None, with_lse=True):
    batch, query_len, heads, dim = q.shape
    key_len, kv_heads = k.shape[1], k.shape[2]
    scale = float(1.0 / np.sqrt(np.float32(dim))) if scale is None else scale
    config = A.FmhaPrefillConfig.contiguous(batch, query_len, key_len, heads, kv_heads, dim, scale, causal)
    out = torch.full_like(q, float("nan"))
    lse = torch.full((batch, heads, query_len), float("nan"), device="cuda", dtype=torch.float32)
    if with_lse:
        A.fmha_prefill_lse_bf16(None, out, lse, q, k, v, config)
    else:
        A.fmha_prefill_bf16(None, out, q, k, v, config)
    torch.cuda.synchronize()
    want, want_lse = oracle.fmha_prefill_lse_f32(
        q.float().cpu().numpy(), k.float().cpu().numpy(), v.float().cpu().numpy(), batch=batch, query_len=query_len,
        key_len=key_len, heads=heads, kv_heads=kv_heads, head_dim=dim, scale=scale, causal=causal, threads=8)
    return out.float().cpu().numpy(), lse.cpu().numpy(), want, want_lse


def check(got, lse, want, want_lse, label, with_lse=True):
    assert np.isfinite(got).all(), f"{label}: non-finite output"
    gap = np.abs(got - want)
    assert gap.max() <= MAX_ABS, f"{label}: max-abs {gap.max()}"
    assert gap.mean() <= MEAN_ABS, f"{label}: mean-abs {gap.mean()}"
    if with_lse:
        assert np.abs(lse - want_lse).max() <= LSE_ABS, f"{label}: lse {np.abs(lse - want_lse).max()}"


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("batch,query_len,key_len,heads,kv_heads", [
    (1, 128, 128, 1, 1), (2, 256, 256, 4, 2), (1, 64, 64, 2, 2), (1, 100, 100, 3, 1), (1, 1, 1, 1, 1),
    (1, 33, 97, 2, 1), (1, 300, 129, 2, 2), (1, 512, 512, 8, 8), (1, 640, 1000, 4, 1),
])
def test_prefill_matches_oracle(batch, query_len, key_len, heads, kv_heads, causal):
    q, k, v = make(batch, query_len, key_len, heads, kv_heads, seed=query_len * 7 + key_len)
    got, lse, want, want_lse = run(q, k, v, causal)
    check(got, lse, want, want_lse, f"{batch}x{query_len}x{key_len} h{heads}/{kv_heads} causal={causal}")


def test_prefill_without_lse_and_explicit_scale():
    q, k, v = make(1, 200, 200, 2, 1, seed=5)
    got, lse, want, want_lse = run(q, k, v, True, scale=0.05, with_lse=False)
    check(got, lse, want, want_lse, "no lse", with_lse=False)


def test_prefill_headline_slice_matches_oracle():
    # One batch item and four heads of the headline shape (seq 4096, head_dim 128, causal): the full
    # [4, 4096, 32, 128] problem is covered by the structural test below.
    q, k, v = make(1, 4096, 4096, 4, 4, seed=99)
    got, lse, want, want_lse = run(q, k, v, True)
    check(got, lse, want, want_lse, "seq 4096")


def test_prefill_full_size_properties():
    # Full headline size, checked through facts that do not need the oracle: with V = 1 every output
    # is 1; with all keys equal the output is the mean of the visible values (a running mean under the
    # causal mask); and rows are independent of batch/head neighbours (same data -> same rows).
    batch, seq, heads, dim = 4, 4096, 32, 128
    gen = torch.Generator(device="cuda")
    gen.manual_seed(3)
    q = torch.randn((batch, seq, heads, dim), generator=gen, device="cuda").to(torch.bfloat16)
    k = torch.randn((1, seq, 1, dim), generator=gen, device="cuda").to(torch.bfloat16).expand(batch, seq, heads, dim).contiguous()
    v = torch.ones((batch, seq, heads, dim), device="cuda", dtype=torch.bfloat16)
    config = A.FmhaPrefillConfig.contiguous(batch, seq, seq, heads, heads, dim, float(dim ** -0.5), True)
    out = torch.empty_like(q)
    A.fmha_prefill_bf16(None, out, q, k, v, config)
    torch.cuda.synchronize()
    assert (out.float() - 1.0).abs().max().item() <= 2 ** -7
    # zero queries: uniform weights over the visible keys -> running mean of V along the sequence
    v2 = torch.randn((1, seq, 1, dim), generator=gen, device="cuda").to(torch.bfloat16).expand(batch, seq, heads, dim).contiguous()
    A.fmha_prefill_bf16(None, out, torch.zeros_like(q), k, v2, config)
    torch.cuda.synchronize()
    mean = torch.cumsum(v2[0, :, 0].double(), dim=0) / torch.arange(1, seq + 1, device="cuda").double()[:, None]
    assert (out.double() - mean[None, :, None, :]).abs().max().item() <= 2e-2
    assert torch.equal(out[0, :, 0], out[3, :, 31])


def test_prefill_validation_errors():
    q, k, v = make(1, 64, 64, 2, 1, seed=1)
    out = torch.empty_like(q)
    good = A.FmhaPrefillConfig.contiguous(1, 64, 64, 2, 1, 128, 0.1, True)
    from dataclasses import replace
    with pytest.raises(error.InvalidLength):
        A.fmha_prefill_bf16(None, out, q, k, v, replace(good, kv_heads=0))
    with pytest.raises(error.InvalidLength):
        A.fmha_prefill_bf16(None, out, q, k, v, replace(good, scale=float("inf")))
    with pytest.raises(error.LengthTooShort):
        A.fmha_prefill_bf16(None, out, q, k[:, :63].contiguous(), v, good)
    wide = lambda heads: torch.zeros((1, 64, heads, 320), device="cuda", dtype=torch.bfloat16)
    with pytest.raises(error.UnsupportedWidth):  # head dimensions past 256 have no kernel
        A.fmha_prefill_bf16(None, wide(4), wide(4), wide(2), wide(2), A.FmhaPrefillConfig.contiguous(1, 64, 64, 4, 2, 320, 0.1, True))


@pytest.mark.parametrize("magnitude,causal", [(8.0, True), (8.0, False), (30.0, True), (0.01, True)])
def test_scores_that_keep_outrunning_the_reference_point(magnitude, causal):
    # Scores grow steadily along the keys (by far more than the lag the running maximum is allowed), so every
    # block moves the softmax reference point and rescales the output; small magnitudes give a flat softmax.
    batch, seq, heads, kv_heads = 1, 700, 4, 2
    gen = torch.Generator(device="cuda")
    gen.manual_seed(int(magnitude * 100) + int(causal))
    q = (torch.randn((batch, seq, heads, 128), generator=gen, device="cuda") * magnitude).to(torch.bfloat16)
    k = (torch.randn((batch, seq, kv_heads, 128), generator=gen, device="cuda") * magnitude).to(torch.bfloat16)
    v = torch.randn((batch, seq, kv_heads, 128), generator=gen, device="cuda").to(torch.bfloat16)
    k[:, :, :, 0] += torch.linspace(0, 40 * magnitude, seq, device="cuda").to(torch.bfloat16)[None, :, None]
    q[:, :, :, 0] = magnitude
    scale = float(1.0 / np.sqrt(np.float32(128)))
    config = A.FmhaPrefillConfig.contiguous(batch, seq, seq, heads, kv_heads, 128, scale, causal)
    out = torch.full_like(q, float("nan"))
    lse = torch.full((batch, heads, seq), float("nan"), device="cuda", dtype=torch.float32)
    A.fmha_prefill_lse_bf16(None, out, lse, q, k, v, config)
    want, want_lse = oracle.fmha_prefill_lse_f32(q.float().cpu().numpy(), k.float().cpu().numpy(), v.float().cpu().numpy(), batch=batch,
                                                 query_len=seq, key_len=seq, heads=heads, kv_heads=kv_heads, head_dim=128,
                                                 scale=scale, causal=causal, threads=8)
    got = out.float().cpu().numpy()
    assert np.isfinite(got).all()
    gap = np.abs(got - want)
    assert gap.max() <= 2e-2 and gap.mean() <= 2e-3, (gap.max(), gap.mean())
    assert (np.abs(lse.cpu().numpy() - want_lse) / np.maximum(1.0, np.abs(want_lse))).max() <= 1e-5


@pytest.fixture
def two_tiles_a_wave():
    """Sends every dense call that has the form to the kernel that gives a wave two 32-row tiles."""
    from singe_amd import _native
    _native.lib().singe_hip_set_dense_prefill_rows_per_wave(64)
    yield
    _native.lib().singe_hip_set_dense_prefill_rows_per_wave(0)


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("batch,query_len,key_len,heads,kv_heads", [
    (1, 256, 256, 1, 1), (2, 512, 512, 4, 2), (1, 64, 64, 2, 2), (1, 100, 128, 3, 1), (1, 1, 64, 1, 1),
    (1, 300, 192, 2, 2), (1, 1024, 1024, 8, 8), (1, 640, 1024, 4, 1), (1, 1024, 320, 2, 1), (3, 768, 768, 2, 1),
    # key counts that leave a last tile of 1, 63, 33, 32 and 31 keys, fewer keys than a tile, and rows past the last key
    (1, 257, 257, 2, 1), (1, 1000, 1000, 2, 2), (2, 300, 191, 2, 1), (1, 97, 97, 1, 1), (1, 512, 160, 2, 2), (1, 350, 607, 3, 3),
    (1, 40, 33, 1, 1), (1, 700, 63, 2, 1), (1, 64, 1, 1, 1),
])
def test_two_tiles_a_wave_matches_oracle(two_tiles_a_wave, batch, query_len, key_len, heads, kv_heads, causal):
    q, k, v = make(batch, query_len, key_len, heads, kv_heads, seed=query_len * 11 + key_len)
    got, lse, want, want_lse = run(q, k, v, causal)
    check(got, lse, want, want_lse, f"two tiles: {batch}x{query_len}x{key_len} h{heads}/{kv_heads} causal={causal}")


@pytest.mark.parametrize("rows_per_wave", [64, 32])
@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("key_len", [1, 63, 65, 250, 1000])
def test_rows_behind_the_last_key_are_not_read(rows_per_wave, causal, key_len):
    # keys and values are the front of buffers whose rows behind the last key hold NaN: a last tile that is not whole
    # must re-read its last key there (a NaN value under a zero weight would still be a NaN)
    from singe_amd import _native
    q, k_all, v_all = make(1, 384, key_len + 96, 2, 1, seed=key_len + 5)
    k_all[:, key_len:] = float("nan")
    v_all[:, key_len:] = float("nan")
    _native.lib().singe_hip_set_dense_prefill_rows_per_wave(rows_per_wave)
    try:
        got, lse, want, want_lse = run(q, k_all[:, :key_len], v_all[:, :key_len], causal)
    finally:
        _native.lib().singe_hip_set_dense_prefill_rows_per_wave(0)
    check(got, lse, want, want_lse, f"NaN behind key {key_len}, causal={causal}, {rows_per_wave} rows a wave")


def test_two_tiles_a_wave_negative_scale_and_no_lse(two_tiles_a_wave):
    q, k, v = make(1, 512, 512, 2, 1, seed=8)
    got, lse, want, want_lse = run(q, k, v, True, scale=-0.07, with_lse=False)
    check(got, lse, want, want_lse, "two tiles, negative scale", with_lse=False)


def test_two_tiles_a_wave_headline_slice_and_default_choice():
    # The headline shape fills the chip with 256-row tiles, so the default choice is this kernel: a slice of it against the
    # oracle, and the whole of it equal to the 32-row kernel's answer within the rounding of the output.
    from singe_amd import _native
    q, k, v = make(1, 4096, 4096, 4, 4, seed=99)
    _native.lib().singe_hip_set_dense_prefill_rows_per_wave(64)
    try:
        got, lse, want, want_lse = run(q, k, v, True)
    finally:
        _native.lib().singe_hip_set_dense_prefill_rows_per_wave(0)
    check(got, lse, want, want_lse, "two tiles, seq 4096")
    batch, seq, heads, dim = 4, 4096, 32, 128
    q, k, v = make(batch, seq, seq, heads, heads, seed=4)
    config = A.FmhaPrefillConfig.contiguous(batch, seq, seq, heads, heads, dim, float(dim ** -0.5), True)
    chosen, narrow = torch.empty_like(q), torch.empty_like(q)
    lse_chosen = torch.empty((batch, heads, seq), device="cuda", dtype=torch.float32)
    lse_narrow = torch.empty_like(lse_chosen)
    A.fmha_prefill_lse_bf16(None, chosen, lse_chosen, q, k, v, config)
    _native.lib().singe_hip_set_dense_prefill_rows_per_wave(32)
    try:
        A.fmha_prefill_lse_bf16(None, narrow, lse_narrow, q, k, v, config)
    finally:
        _native.lib().singe_hip_set_dense_prefill_rows_per_wave(0)
    torch.cuda.synchronize()
    assert (chosen.float() - narrow.float()).abs().max().item() <= 2 ** -6
    assert (lse_chosen - lse_narrow).abs().max().item() <= 1e-4


@pytest.mark.parametrize("causal", [True, False])
def test_two_tiles_a_wave_f16(two_tiles_a_wave, causal):
    q, k, v = (t.to(torch.float16) for t in make(2, 600, 576, 4, 2, seed=13))
    scale = float(1.0 / np.sqrt(np.float32(128)))
    config = A.FmhaPrefillConfig.contiguous(2, 600, 576, 4, 2, 128, scale, causal)
    out = torch.full_like(q, float("nan"))
    lse = torch.full((2, 4, 600), float("nan"), device="cuda")
    A.fmha_prefill_lse_f16(None, out, lse, q, k, v, config)
    torch.cuda.synchronize()
    want, want_lse = oracle.fmha_prefill_lse_f32(q.float().cpu().numpy(), k.float().cpu().numpy(), v.float().cpu().numpy(), batch=2,
                                                 query_len=600, key_len=576, heads=4, kv_heads=2, head_dim=128, scale=scale,
                                                 causal=causal, threads=8)
    gap = np.abs(out.float().cpu().numpy() - want)
    # (f16 carries three more bits than bf16)
    assert gap.max() <= MAX_ABS / 6 and gap.mean() <= MEAN_ABS / 6, (gap.max(), gap.mean())
    assert np.abs(lse.cpu().numpy() - want_lse).max() <= LSE_ABS


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("batch,query_len,key_len,heads,kv_heads", [
    (1, 256, 256, 1, 1), (2, 512, 512, 4, 2), (1, 100, 128, 3, 1), (1, 1024, 1024, 8, 8), (1, 640, 1024, 4, 1), (1, 1024, 320, 2, 1),
    (1, 257, 257, 2, 1), (1, 1000, 1000, 2, 2), (2, 300, 191, 2, 1), (1, 350, 607, 3, 3), (1, 40, 33, 1, 1), (1, 64, 1, 1, 1),
])
@pytest.mark.parametrize("dim", [16, 32, 48, 64, 80, 96, 112])
def test_two_tiles_a_wave_other_head_dims(two_tiles_a_wave, batch, query_len, key_len, heads, kv_heads, causal, dim):
    # the other builds of the two-tile kernel: whole key tiles and last tiles that are not
    q, k, v = make(batch, query_len, key_len, heads, kv_heads, seed=query_len * 13 + key_len, dim=dim)
    from singe_amd import _native
    import ctypes
    config = A.FmhaPrefillConfig.contiguous(batch, query_len, key_len, heads, kv_heads, dim, 0.125, causal)
    assert _native.lib().singe_hip_dense_prefill_rows_per_wave(ctypes.byref(config._c())) == 64
    got, lse, want, want_lse = run(q, k, v, causal)
    check(got, lse, want, want_lse, f"two tiles, head_dim {dim}: {batch}x{query_len}x{key_len} h{heads}/{kv_heads} causal={causal}")


@pytest.mark.parametrize("dim", [16, 32, 48, 64, 80, 96, 112])
@pytest.mark.parametrize("causal", [True, False])
def test_two_tiles_a_wave_other_head_dims_f16_and_nan_behind_the_last_key(two_tiles_a_wave, causal, dim):
    q, k_all, v_all = (t.to(torch.float16) for t in make(1, 600, 1000 + 96, 4, 2, seed=17, dim=dim))
    k_all[:, 1000:] = float("nan")
    v_all[:, 1000:] = float("nan")
    k, v = k_all[:, :1000], v_all[:, :1000]
    config = A.FmhaPrefillConfig.contiguous(1, 600, 1000, 4, 2, dim, 0.125, causal)
    out = torch.full_like(q, float("nan"))
    lse = torch.full((1, 4, 600), float("nan"), device="cuda")
    A.fmha_prefill_lse_f16(None, out, lse, q, k, v, config)
    torch.cuda.synchronize()
    want, want_lse = oracle.fmha_prefill_lse_f32(q.float().cpu().numpy(), k.float().cpu().numpy(), v.float().cpu().numpy(), batch=1,
                                                 query_len=600, key_len=1000, heads=4, kv_heads=2, head_dim=dim, scale=0.125,
                                                 causal=causal, threads=8)
    gap = np.abs(out.float().cpu().numpy() - want)
    assert gap.max() <= MAX_ABS / 6 and gap.mean() <= MEAN_ABS / 6, (gap.max(), gap.mean())
    assert np.abs(lse.cpu().numpy() - want_lse).max() <= LSE_ABS


@pytest.mark.parametrize("dim", [128, 64, 96, 80, 48, 16])
@pytest.mark.parametrize("causal", [True, False])
def test_two_tiles_a_wave_head_major_layout(two_tiles_a_wave, causal, dim):
    # tensors stored [batch, heads, len, dim] (strides of their own for every operand), a key count that leaves a last
    # tile of 21 keys
    batch, heads, kv_heads, query_len, key_len = 2, 4, 2, 530, 725
    gen = torch.Generator(device="cuda")
    gen.manual_seed(dim + causal)
    q = torch.randn((batch, heads, query_len, dim), generator=gen, device="cuda").to(torch.bfloat16)
    k = torch.randn((batch, kv_heads, key_len, dim), generator=gen, device="cuda").to(torch.bfloat16)
    v = torch.randn((batch, kv_heads, key_len, dim), generator=gen, device="cuda").to(torch.bfloat16)
    scale = float(dim) ** -0.5
    config = A.bhsd_config(batch, heads, kv_heads, query_len, key_len, dim, scale, causal)
    out = torch.full_like(q, float("nan"))
    lse = torch.full((batch, heads, query_len), float("nan"), device="cuda", dtype=torch.float32)
    A.fmha_prefill_lse_bf16(None, out, lse, q, k, v, config)
    torch.cuda.synchronize()
    rows = lambda tensor: tensor.float().permute(0, 2, 1, 3).contiguous().cpu().numpy()
    want, want_lse = oracle.fmha_prefill_lse_f32(rows(q), rows(k), rows(v), batch=batch, query_len=query_len, key_len=key_len,
                                                 heads=heads, kv_heads=kv_heads, head_dim=dim, scale=scale, causal=causal, threads=8)
    check(rows(out), lse.cpu().numpy(), want, want_lse, f"two tiles, head-major layout, head_dim {dim}, causal={causal}")
