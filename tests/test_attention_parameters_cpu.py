"""AttentionParameters, its candidates and parameter_key (singe/src/backend/cuda/kernel_plan/source/parameters.rs:21-57,
221-230; attention.rs:113-175), through the C ABI without a device: the default, what is taken and what is refused as
a stale record, and the key strings, written out here by hand from the reference's format strings."""
import ctypes

import numpy as np
import pytest

from singe_amd import _native, error, neural


def test_default_and_candidates():
    default = neural.default_attention_parameters()
    # warps 4, key_tile 64, stages 1 and no launch bound as in the reference's default (parameters.rs:34-44); the
    # threshold is this device's own (twice its compute units; 256 units are assumed when no device is visible)
    assert (default.warps, default.key_tile, default.stages, default.min_blocks) == (4, 64, 1, None)
    assert default.split_below_blocks > 0 and default.split_below_blocks % 2 == 0
    candidates = neural.attention_candidates()
    assert candidates[0] == default and len(candidates) == len(set(candidates)) > 1
    # the thresholds the reference tries are among them (attention.rs:122), and the staged and bounded variants
    for below in (64, 0, 256):
        assert neural.AttentionParameters(split_below_blocks=below) in candidates
    assert any(c.stages == 2 for c in candidates) and any(c.min_blocks == 2 for c in candidates)


def test_every_candidate_is_taken_and_anything_else_is_a_stale_record():
    try:
        for candidate in neural.attention_candidates():
            neural.set_attention_parameters(candidate)
            assert neural.attention_parameters() == candidate
        for stale in (neural.AttentionParameters(warps=8, split_below_blocks=64), neural.AttentionParameters(key_tile=128),
                      neural.AttentionParameters(stages=3), neural.AttentionParameters(split_below_blocks=77),
                      neural.AttentionParameters(min_blocks=4)):
            with pytest.raises(error.StaleRecord):
                neural.set_attention_parameters(stale)
    finally:
        neural.set_attention_parameters(None)
    assert neural.attention_parameters() == neural.default_attention_parameters()


def _paged_key(problem, data_type):
    need = _native.lib().singe_hip_paged_attention_parameter_key(ctypes.byref(problem), data_type, None, 0)
    buffer = ctypes.create_string_buffer(need + 1)
    assert _native.lib().singe_hip_paged_attention_parameter_key(ctypes.byref(problem), data_type, buffer, need + 1) == need
    return buffer.value.decode()


POLICY = "NumericalPolicy { precision: Full, determinism: Allow }"


def test_paged_attention_parameter_key_of_the_references_own_test_operands():
    # parameter_tests.rs:244-276: query [5, 4, 16] bf16, caches [4, 32, 2, 16], indices [3], [3], [4], [2] (i32), causal
    problem = _native.PagedAttentionProblemC(5, 4, 2, 16, 32, 2, 4, 4, 0, 1, 0, 0, 0, 0.0, 0.0, 0)
    attributes = ("ScaledDotProductAttentionAttributes { scale: None, causal: true, window: None, softcap: None, masked: false, "
                  "sinks: false, key_lengths: false }")
    assert _paged_key(problem, _native.DATA_TYPE_BF16) == (
        f"kernel|paged_attention|{POLICY}|{attributes} Bf16[5, 4, 16][64, 16, 1]+0 Bf16[4, 32, 2, 16][1024, 32, 16, 1]+0 "
        "Bf16[4, 32, 2, 16][1024, 32, 16, 1]+0 I32[3][1]+0 I32[3][1]+0 I32[4][1]+0 I32[2][1]+0")
    # an axis of one element addresses with stride 0 (layout/mod.rs:32-40): kv_heads 1, one sequence
    problem = _native.PagedAttentionProblemC(3, 1, 1, 128, 32, 1, 4, 1, 1, 0, 1, 1, 1, 0.25, 30.0, 16)
    attributes = ("ScaledDotProductAttentionAttributes { scale: Some(0.25), causal: false, window: Some(16), softcap: Some(30.0), "
                  "masked: false, sinks: false, key_lengths: false }")
    assert _paged_key(problem, _native.DATA_TYPE_F16) == (
        f"kernel|paged_attention|{POLICY}|{attributes} F16[3, 1, 128][128, 0, 1]+0 F16[4, 32, 1, 128][4096, 128, 0, 1]+0 "
        "F16[4, 32, 1, 128][4096, 128, 0, 1]+0 I64[2][1]+0 I64[2][1]+0 I64[1][0]+0 I64[1][0]+0")
    # a short buffer is filled as far as it goes and the needed length still comes back
    short = ctypes.create_string_buffer(10)
    assert _native.lib().singe_hip_paged_attention_parameter_key(ctypes.byref(problem), 2, short, 10) > 10
    assert short.value == b"kernel|pa"


def test_dense_attention_parameter_key():
    problem = _native.AttentionProblemC(1, 4, 2, 8, 96, 16, 16, (ctypes.c_int64 * 4)(0, 0, 96, 1), _native.DATA_TYPE_F16, 1, 0, 0, 0,
                                        0.0, 0.0, 0)
    def key(masked, sinks, lengths):
        need = _native.lib().singe_hip_attention_parameter_key(ctypes.byref(problem), masked, sinks, lengths, None, 0)
        buffer = ctypes.create_string_buffer(need + 1)
        _native.lib().singe_hip_attention_parameter_key(ctypes.byref(problem), masked, sinks, lengths, buffer, need + 1)
        return buffer.value.decode()
    head = f"kernel|attention|{POLICY}|ScaledDotProductAttentionAttributes {{ scale: None, causal: true, window: None, softcap: None, "
    operands = " F16[1, 4, 8, 16][0, 128, 16, 1]+0 F16[1, 2, 96, 16][0, 1536, 16, 1]+0 F16[1, 2, 96, 16][0, 1536, 16, 1]+0"
    assert key(0, 0, 0) == head + "masked: false, sinks: false, key_lengths: false }" + operands
    # a mask over [query, key] broadcast to [1, 1, 8, 96], sinks [4], key lengths [1] i32 (attention.rs:241-247)
    assert key(1, 1, 1) == (head + "masked: true, sinks: true, key_lengths: true }" + operands +
                            " F16[1, 1, 8, 96][0, 0, 96, 1]+0 F16[4][1]+0 I32[1][0]+0")


@pytest.mark.parametrize("value", [0.25, 30.0, 128 ** -0.5, 1.0, 0.1, 1e-7, 123456.789, 3e20, -0.05, 1e16, 0.00001])
def test_scales_are_spelled_as_the_shortest_digits_that_read_back(value):
    problem = _native.PagedAttentionProblemC(1, 1, 1, 16, 16, 1, 1, 1, 0, 0, 1, 0, 0, value, 0.0, 0)
    text = _paged_key(problem, 0)
    spelled = text.split("scale: Some(")[1].split(")")[0]
    assert np.float32(float(spelled)) == np.float32(value)                    # reads back to the same f32
    digits = spelled.replace("-", "").replace(".", "").split("e")[0].strip("0")
    shortest = np.format_float_scientific(np.float32(value), unique=True, trim="-").split("e")[0].replace("-", "").replace(".", "")
    assert len(digits) <= max(len(shortest), 1)                               # and with no digit to spare
    assert ("." in spelled) or ("e" in spelled)                               # Debug always shows a fraction or an exponent
