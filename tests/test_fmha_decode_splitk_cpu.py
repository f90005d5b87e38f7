"""No-GPU checks of the dense split-KV decode convention: the reference's own unit tests of its config types
(singe-kernel/src/cuda/attention/tests.rs:111-194) reproduced through the C ABI, and the oracle's restatement of
the split kernel pinned by an independent float64 computation, closed forms and the split / reduce identity."""
import ctypes

import numpy as np
import pytest

import oracle
from singe_amd import _native, error
from singe_amd.kernel import attention as A

FAKE = 0x1000


def reduce_status(config, out=64, attn=256, lse=32, query=64, key=160, value=160):
    c = config._c()
    return _native.lib().singe_hip_fmha_decode_splitk_reduce_f32(
        None, FAKE, out, FAKE, attn, FAKE, lse, FAKE, query, FAKE, key, FAKE, value, ctypes.byref(c))


def test_config_builders_preserve_tuning_choice():
    # tests.rs:111-129
    config = A.FmhaDecodeSplitKReduceConfig.contiguous(2, 5, 4, 2, 8, 4, 0.5)
    tuning = A.AttentionSplitKTuning.create(2)
    assert config.tuning == A.TuningChoice.Default()
    assert config.explicit_tuning(tuning).tuning == A.TuningChoice.Explicit(tuning)
    assert config.cached_tuning().tuning == A.TuningChoice.Cached()
    assert config.tune(A.TuneOptions()).tuning.kind == A.TuningChoice.TUNE
    assert config.retune(A.TuneOptions()).tuning.kind == A.TuningChoice.RETUNE
    assert A.TuneOptions() == A.TuneOptions(1, 5, 2**64 - 1)  # autotune.rs:63-71


def test_candidates_include_power_ladder_and_max():
    # tests.rs:131-147
    config = A.FmhaDecodeSplitKReduceConfig.contiguous(2, 17, 4, 2, 8, 6, 0.5)
    assert [t.splits for t in A.attention_splitk_candidates(config)] == [1, 2, 4, 6]
    config = A.FmhaDecodeSplitKReduceConfig.contiguous(2, 17, 4, 2, 8, 4, 0.5)
    assert [t.splits for t in A.attention_splitk_candidates(config)] == [1, 2, 4]
    # key_len caps the ladder (mod.rs:2365), the full ladder ends at 64
    config = A.FmhaDecodeSplitKReduceConfig.contiguous(2, 3, 4, 2, 8, 8, 0.5)
    assert [t.splits for t in A.attention_splitk_candidates(config)] == [1, 2, 3]
    config = A.FmhaDecodeSplitKReduceConfig.contiguous(1, 4096, 4, 2, 8, 100, 0.5)
    assert [t.splits for t in A.attention_splitk_candidates(config)] == [1, 2, 4, 8, 16, 32, 64, 100]


def test_validation_accepts_exact_lengths():
    # tests.rs:149-153: lengths pass; the launch then fails for want of a device or succeeds, never a length error
    config = A.FmhaDecodeSplitKReduceConfig.contiguous(2, 5, 4, 2, 8, 4, 0.5)
    assert reduce_status(config) not in (1, 2, 3, 4)


def test_validation_caps_scratch_at_key_len():
    # tests.rs:155-159: max_splits 8 over 3 keys needs scratch for 3 splits only
    config = A.FmhaDecodeSplitKReduceConfig.contiguous(2, 3, 4, 2, 8, 8, 0.5)
    assert reduce_status(config, 64, 192, 24, 64, 96, 96) not in (1, 2, 3, 4)
    assert reduce_status(config, 64, 191, 24, 64, 96, 96) == 2


def test_validation_rejects_short_scratch():
    # tests.rs:161-179
    config = A.FmhaDecodeSplitKReduceConfig.contiguous(2, 5, 4, 2, 8, 4, 0.5)
    assert reduce_status(config, attn=255) == 2
    detail = _native.ErrorDetail()
    _native.lib().singe_hip_last_error(ctypes.byref(detail))
    assert (detail.name, detail.minimum, detail.actual) == (b"attn_scratch", 256, 255)
    assert reduce_status(config, lse=31) == 2
    # the other buffers, in the reference's order: query, key, value, out (mod.rs:2290-2305)
    assert reduce_status(config, query=63) == 2 and reduce_status(config, key=159) == 2
    assert reduce_status(config, value=159) == 2 and reduce_status(config, out=63) == 2
    _native.lib().singe_hip_last_error(ctypes.byref(detail))
    assert detail.name == b"out"
    assert reduce_status(config, query=63, out=63) == 2
    _native.lib().singe_hip_last_error(ctypes.byref(detail))
    assert detail.name == b"query"


def test_tuning_rejects_too_many_splits():
    # tests.rs:181-194: zero, more than max_splits, more than key_len
    config = A.FmhaDecodeSplitKReduceConfig.contiguous(2, 5, 4, 2, 8, 4, 0.5)
    assert reduce_status(config.explicit_tuning(A.AttentionSplitKTuning(0))) == 1
    assert reduce_status(config.explicit_tuning(A.AttentionSplitKTuning(5))) == 1
    wide = A.FmhaDecodeSplitKReduceConfig.contiguous(2, 3, 4, 2, 8, 8, 0.5)
    assert reduce_status(wide.explicit_tuning(A.AttentionSplitKTuning(4)), 64, 192, 24, 64, 96, 96) == 1


def test_config_validation():
    # validate_fmha_decode_splitk_reduce_config (mod.rs:2554-2560) and validate_fmha_decode_config (:3530-3555)
    with pytest.raises(error.InvalidLength):
        A.FmhaDecodeSplitKReduceConfig.contiguous(2, 5, 4, 2, 8, 0, 0.5)
    with pytest.raises(error.InvalidLength):
        A.FmhaDecodeSplitKReduceConfig.contiguous(2, 5, 4, 3, 8, 4, 0.5)
    with pytest.raises(error.InvalidLength):
        A.FmhaDecodeSplitKReduceConfig.contiguous(2, 0, 4, 2, 8, 4, 0.5)
    with pytest.raises(error.InvalidLength):
        A.FmhaDecodeSplitKReduceConfig.contiguous(2, 5, 4, 2, 8, 4, float("inf"))
    good = A.FmhaDecodeSplitKReduceConfig.contiguous(2, 5, 4, 2, 8, 4, 0.5)
    bad = A.FmhaDecodeSplitKReduceConfig(good.decode, 0)
    assert reduce_status(bad) == 1
    # an unknown tuning kind is an argument error; Cached without a device is a runtime or cache-miss answer, never a launch
    odd = A.FmhaDecodeSplitKReduceConfig(good.decode, 4, A.TuningChoice(9))
    assert reduce_status(odd) == 9


def split_status(config, out, lse, query, key, value, pointers=FAKE):
    c = config._c()
    return _native.lib().singe_hip_fmha_decode_splitk_f32(None, pointers, out, pointers, lse, pointers, query, pointers, key,
                                                          pointers, value, ctypes.byref(c))


def test_split_config_validation_and_lengths():
    # FmhaDecodeSplitKConfig::contiguous (mod.rs:2662-2697) and validate_lengths (:2699-2760)
    config = A.FmhaDecodeSplitKConfig.contiguous(2, 5, 4, 2, 4, 2, 8, 0.5)
    assert (config.output_batch_stride, config.output_head_stride, config.output_split_stride) == (128, 32, 8)
    assert (config.lse_batch_stride, config.lse_head_stride) == (16, 4)
    assert split_status(config, 256, 32, 64, 160, 160) not in (1, 2, 3, 4)
    assert split_status(config, 255, 32, 64, 160, 160) == 2
    assert split_status(config, 256, 31, 64, 160, 160) == 2
    assert split_status(config, 256, 32, 63, 160, 160) == 2
    assert split_status(config, 256, 32, 64, 159, 160) == 2
    assert split_status(config, 256, 32, 64, 160, 159) == 2
    import dataclasses
    for field in ("splits", "kv_len_per_split", "output_split_stride", "lse_head_stride", "head_dim"):
        assert split_status(dataclasses.replace(config, **{field: 0}), 256, 32, 64, 160, 160) == 1, field
    assert split_status(dataclasses.replace(config, kv_heads=3), 256, 32, 64, 160, 160) == 1
    # a width outside the kernel set (cutile/attention/splitk.rs:124-139 returns UnsupportedParameter there)
    odd = A.FmhaDecodeSplitKConfig.contiguous(2, 5, 4, 2, 4, 2, 12, 0.5)
    assert split_status(odd, 4 * 96, 32, 96, 240, 240) == 5
    assert split_status(config, 256, 32, 64, 160, 160, pointers=None) == 6


def float64_split(q, k, v, splits, per, scale):
    batch, heads, dim = q.shape
    _, keys, kv_heads, _ = k.shape
    out = np.zeros((batch, heads, splits, dim))
    lse = np.full((batch, heads, splits), np.float64(np.float32(-1.0e20)))
    for b in range(batch):
        for h in range(heads):
            g = h // (heads // kv_heads)
            for s in range(splits):
                lo, hi = min(s * per, keys), min(s * per + per, keys)
                if lo == hi:
                    continue
                scores = k[b, lo:hi, g].astype(np.float64) @ q[b, h].astype(np.float64) * scale
                weights = np.exp(scores - scores.max())
                out[b, h, s] = weights @ v[b, lo:hi, g].astype(np.float64) / weights.sum()
                lse[b, h, s] = scores.max() + np.log(weights.sum())
    return out, lse


def test_oracle_split_kernel_against_float64_and_closed_forms():
    gen = np.random.default_rng(5)
    batch, keys, heads, kv_heads, dim = 2, 37, 6, 2, 16
    q = gen.normal(size=(batch, heads, dim)).astype(np.float32)
    k = gen.normal(size=(batch, keys, kv_heads, dim)).astype(np.float32)
    v = gen.normal(size=(batch, keys, kv_heads, dim)).astype(np.float32)
    for splits, per in ((1, 37), (4, 10), (5, 10), (37, 1), (3, 5)):
        out, lse = oracle.fmha_decode_splitk_f32(q, k, v, splits=splits, kv_len_per_split=per, scale=0.25)
        want, want_lse = float64_split(q, k, v, splits, per, 0.25)
        assert np.abs(out - want).max() < 2e-6 and np.abs(lse - want_lse).max() < 2e-6, (splits, per)
    # a split past the keys: zeros and -1e20 exactly
    out, lse = oracle.fmha_decode_splitk_f32(q, k, v, splits=5, kv_len_per_split=10, scale=0.25)
    assert not out[:, :, 4].any() and np.all(lse[:, :, 4] == np.float32(-1.0e20))
    # one key per split: the value itself and the score
    out, lse = oracle.fmha_decode_splitk_f32(q, k, v, splits=37, kv_len_per_split=1, scale=0.25)
    for h in range(heads):
        assert np.array_equal(out[:, h], v[:, :, h // 3])
    # grouped heads read their kv head: heads 0-2 share keys 0, heads 3-5 keys 1
    same = np.repeat(q[:, :1], heads, axis=1)
    out, _ = oracle.fmha_decode_splitk_f32(same, k, v, splits=2, kv_len_per_split=19, scale=0.25)
    assert np.array_equal(out[:, 0], out[:, 2]) and np.array_equal(out[:, 3], out[:, 5]) and not np.array_equal(out[:, 0], out[:, 3])


def test_oracle_split_then_reduce_is_the_unsplit_decode():
    gen = np.random.default_rng(6)
    batch, keys, heads, kv_heads, dim = 2, 50, 4, 2, 8
    q = gen.normal(size=(batch, heads, dim)).astype(np.float32)
    k = gen.normal(size=(batch, keys, kv_heads, dim)).astype(np.float32)
    v = gen.normal(size=(batch, keys, kv_heads, dim)).astype(np.float32)
    whole, _ = float64_split(q, k, v, 1, keys, 0.3)
    for splits in (1, 2, 7, 50):
        per = -(-keys // splits)
        attn, lse = oracle.fmha_decode_splitk_f32(q, k, v, splits=splits, kv_len_per_split=per, scale=0.3)
        got = oracle.splitk_reduce_f32(attn, lse, batch=batch, heads=heads, splits=splits, head_dim=dim)
        assert np.abs(got - whole[:, :, 0]).max() < 2e-6, splits
