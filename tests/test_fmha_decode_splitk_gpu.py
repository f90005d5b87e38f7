"""GPU parity of the dense f32 split-KV decode (fmha_decode_splitk_f32, fmha_decode_splitk_reduce_f32) against the
oracle's restatement of the reference kernel, through the C ABI.  Tolerance 1e-4 absolute (f32)."""
import numpy as np
import pytest
import torch

import oracle
from singe_amd import error
from singe_amd.kernel import attention as A

pytestmark = pytest.mark.gpu
TOLERANCE = 1e-4


def make(seed, batch, keys, heads, kv_heads, dim):
    gen = np.random.default_rng(seed)
    q = gen.normal(size=(batch, heads, dim)).astype(np.float32)
    k = gen.normal(size=(batch, keys, kv_heads, dim)).astype(np.float32)
    v = gen.normal(size=(batch, keys, kv_heads, dim)).astype(np.float32)
    return q, k, v


def cuda(*arrays):
    return [torch.from_numpy(a).cuda() for a in arrays]


@pytest.mark.parametrize("dim", [4, 8, 16, 32, 64, 128, 256])
@pytest.mark.parametrize("heads,kv_heads", [(4, 4), (8, 2), (6, 1)])
def test_split_kernel_matches_oracle(dim, heads, kv_heads):
    batch, keys = 2, 77
    q, k, v = make(dim + heads, batch, keys, heads, kv_heads, dim)
    tq, tk, tv = cuda(q, k, v)
    for splits, per in ((1, 77), (4, 20), (5, 20), (77, 1), (3, 7)):
        config = A.FmhaDecodeSplitKConfig.contiguous(batch, keys, heads, kv_heads, splits, per, dim, dim ** -0.5)
        out = torch.full((batch, heads, splits, dim), 7.0, device="cuda")
        lse = torch.full((batch, heads, splits), 7.0, device="cuda")
        A.fmha_decode_splitk_f32(None, out, lse, tq, tk, tv, config)
        want, want_lse = oracle.fmha_decode_splitk_f32(q, k, v, splits=splits, kv_len_per_split=per, scale=dim ** -0.5)
        torch.cuda.synchronize()
        assert np.abs(out.cpu().numpy() - want).max() < TOLERANCE, (splits, per)
        got_lse = lse.cpu().numpy()
        empty = want_lse == np.float32(-1.0e20)
        assert np.array_equal(got_lse[empty], want_lse[empty])  # -1e20 exactly, and zeros beside it
        assert not out.cpu().numpy()[empty].any()
        assert np.abs(got_lse[~empty] - want_lse[~empty]).max() < TOLERANCE, (splits, per)


def test_split_kernel_with_strides_and_unaligned_rows():
    # key / value rows padded to 67 elements (rows off the 16-byte grid), outputs with gaps between splits
    batch, keys, heads, kv_heads, dim, splits, per = 2, 41, 4, 2, 64, 3, 14
    q, k, v = make(9, batch, keys, heads, kv_heads, dim)
    pad = 67
    kp = np.zeros((batch, keys, kv_heads, pad), np.float32); kp[..., :dim] = k
    vp = np.zeros((batch, keys, kv_heads, pad), np.float32); vp[..., :dim] = v
    tq, tk, tv = cuda(q, kp, vp)
    config = A.FmhaDecodeSplitKConfig(batch, keys, heads, kv_heads, splits, per, dim,
                                      heads * dim, keys * kv_heads * pad, keys * kv_heads * pad, heads * splits * 80,
                                      dim, kv_heads * pad, kv_heads * pad, splits * 80, 80, pad, pad, heads * 8, 8, 0.125)
    out = torch.zeros((batch, heads, splits, 80), device="cuda")
    lse = torch.zeros((batch, heads, 8), device="cuda")
    A.fmha_decode_splitk_f32(None, out, lse, tq, tk, tv, config)
    want, want_lse = oracle.fmha_decode_splitk_f32(q, k, v, splits=splits, kv_len_per_split=per, scale=0.125)
    assert np.abs(out.cpu().numpy()[..., :dim] - want).max() < TOLERANCE
    assert not out.cpu().numpy()[..., dim:].any()
    assert np.abs(lse.cpu().numpy()[..., :splits] - want_lse).max() < TOLERANCE


@pytest.mark.parametrize("batch,keys,heads,kv_heads,dim,max_splits", [(2, 300, 8, 2, 64, 16), (1, 1000, 4, 4, 32, 64),
                                                                       (3, 9, 6, 3, 16, 32), (1, 4096, 32, 8, 128, 8)])
def test_split_then_reduce_matches_unsplit_decode(batch, keys, heads, kv_heads, dim, max_splits):
    q, k, v = make(keys, batch, keys, heads, kv_heads, dim)
    tq, tk, tv = cuda(q, k, v)
    scale = dim ** -0.5
    whole, _ = oracle.fmha_decode_splitk_f32(q, k, v, splits=1, kv_len_per_split=keys, scale=scale)
    config = A.FmhaDecodeSplitKReduceConfig.contiguous(batch, keys, heads, kv_heads, dim, max_splits, scale)
    effective = min(max_splits, keys)
    attn_scratch = torch.empty(batch * heads * effective * dim, device="cuda")
    lse_scratch = torch.empty(batch * heads * effective, device="cuda")
    for choice in [config] + [config.explicit_tuning(t) for t in A.attention_splitk_candidates(config)]:
        out = torch.full((batch, heads, dim), 7.0, device="cuda")
        A.fmha_decode_splitk_reduce_f32(None, out, attn_scratch, lse_scratch, tq, tk, tv, choice)
        assert np.abs(out.cpu().numpy() - whole[:, :, 0]).max() < TOLERANCE, choice.tuning
        # and against the oracle's own split + reduce for the same split count
        splits = effective if choice.tuning.kind == A.TuningChoice.DEFAULT else choice.tuning.value.splits
        per = -(-keys // splits)
        attn, lse = oracle.fmha_decode_splitk_f32(q, k, v, splits=splits, kv_len_per_split=per, scale=scale)
        want = oracle.splitk_reduce_f32(attn, lse, batch=batch, heads=heads, splits=splits, head_dim=dim)
        assert np.abs(out.cpu().numpy() - want).max() < TOLERANCE


def test_tuning_choices():
    batch, keys, heads, kv_heads, dim, max_splits = 2, 512, 8, 2, 64, 16
    q, k, v = make(3, batch, keys, heads, kv_heads, dim)
    tq, tk, tv = cuda(q, k, v)
    whole, _ = oracle.fmha_decode_splitk_f32(q, k, v, splits=1, kv_len_per_split=keys, scale=0.125)
    config = A.FmhaDecodeSplitKReduceConfig.contiguous(batch, keys, heads, kv_heads, dim, max_splits, 0.125)
    attn_scratch = torch.empty(batch * heads * max_splits * dim, device="cuda")
    lse_scratch = torch.empty(batch * heads * max_splits, device="cuda")
    out = torch.zeros((batch, heads, dim), device="cuda")
    A.clear_tune_cache()
    assert A.cached_fmha_decode_splitk_reduce_tuning(config) is None
    with pytest.raises(error.TuneCacheMiss):
        A.fmha_decode_splitk_reduce_f32(None, out, attn_scratch, lse_scratch, tq, tk, tv, config.cached_tuning())
    A.fmha_decode_splitk_reduce_f32(None, out, attn_scratch, lse_scratch, tq, tk, tv, config.tune(A.TuneOptions(1, 3, 100)))
    assert np.abs(out.cpu().numpy() - whole[:, :, 0]).max() < TOLERANCE
    best = A.cached_fmha_decode_splitk_reduce_tuning(config)
    assert best in A.attention_splitk_candidates(config)
    out.zero_()
    A.fmha_decode_splitk_reduce_f32(None, out, attn_scratch, lse_scratch, tq, tk, tv, config.cached_tuning())
    assert np.abs(out.cpu().numpy() - whole[:, :, 0]).max() < TOLERANCE
    # max_candidates limits the ladder from its low end (autotune.rs:632-635): only 1 and 2 are timed
    again = A.tune_fmha_decode_splitk_reduce_f32(None, out, attn_scratch, lse_scratch, tq, tk, tv, config, A.TuneOptions(0, 0, 2))
    assert again.splits in (1, 2) and A.cached_fmha_decode_splitk_reduce_tuning(config) == again
    with pytest.raises(error.NoTuneCandidates):
        A.fmha_decode_splitk_reduce_f32(None, out, attn_scratch, lse_scratch, tq, tk, tv, config.retune(A.TuneOptions(1, 1, 0)))
    # a different problem has its own entry
    other = A.FmhaDecodeSplitKReduceConfig.contiguous(batch, keys, heads, kv_heads, dim, 8, 0.125)
    assert A.cached_fmha_decode_splitk_reduce_tuning(other) is None
    A.clear_tune_cache()
    assert A.cached_fmha_decode_splitk_reduce_tuning(config) is None


def test_tuning_is_refused_during_stream_capture():
    batch, keys, heads, kv_heads, dim, max_splits = 1, 256, 4, 2, 64, 8
    q, k, v = make(4, batch, keys, heads, kv_heads, dim)
    tq, tk, tv = cuda(q, k, v)
    whole, _ = oracle.fmha_decode_splitk_f32(q, k, v, splits=1, kv_len_per_split=keys, scale=0.125)
    config = A.FmhaDecodeSplitKReduceConfig.contiguous(batch, keys, heads, kv_heads, dim, max_splits, 0.125)
    attn_scratch = torch.empty(batch * heads * max_splits * dim, device="cuda")
    lse_scratch = torch.empty(batch * heads * max_splits, device="cuda")
    out = torch.zeros((batch, heads, dim), device="cuda")
    A.clear_tune_cache()
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    failures = []
    with torch.cuda.stream(stream):
        graph.capture_begin()
        try:
            for choice in (config.tune(A.TuneOptions()), config.retune(A.TuneOptions()), config.cached_tuning()):
                try:
                    A.fmha_decode_splitk_reduce_f32(stream, out, attn_scratch, lse_scratch, tq, tk, tv, choice)
                    failures.append("accepted")
                except error.AutotuneDuringCapture:
                    pass
            # the default and an explicit choice only enqueue, so they may be captured
            A.fmha_decode_splitk_reduce_f32(stream, out, attn_scratch, lse_scratch, tq, tk, tv, config)
        finally:
            graph.capture_end()
    assert not failures
    for _ in range(3):
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert np.abs(out.cpu().numpy() - whole[:, :, 0]).max() < TOLERANCE
