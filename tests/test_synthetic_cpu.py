"""The library's seeded input streams (csrc/synthetic_inputs.cpp), which bench.py draws its tensors from: the words are
held to splitmix64's published first outputs, the normal values to a restatement of the recipe with Python's own math
(the same libm in double), and the things a caller of another language relies on are checked: any range of a tensor can
be made alone and by any number of threads, streams of different tensors differ, the first two moments are N(0, 1)'s."""
import math

import numpy as np
import torch

from singe_amd import _native, synthetic

MASK = (1 << 64) - 1


def _word(seed, index):
    z = (seed + (index + 1) * 0x9E3779B97F4A7C15) & MASK
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & MASK
    return z ^ (z >> 31)


def _normal(seed, first, count, threads=1):
    out = np.empty(count, dtype=np.float32)
    _native.lib().singe_hip_synthetic_normal_f32(seed, first, out.ctypes.data, count, threads)
    return out


def test_words_are_splitmix64():
    # the first outputs of splitmix64 seeded with zero, as its author's reference code prints them
    published = [0xE220A8397B1DCDAF, 0x6E789E6AA1B965F4, 0x06C45D188009454F, 0xF88BB8A8724C81EC]
    lib = _native.lib()
    assert [lib.singe_hip_synthetic_word(0, i) for i in range(4)] == published
    for seed in (1, 0x51A6E, MASK):
        for index in (0, 1, 12345, (1 << 40) + 3):
            assert lib.singe_hip_synthetic_word(seed, index) == _word(seed, index)


def test_seed_of_a_tensor_is_the_base_seed_xor_fnv1a_of_its_name():
    def fnv(name):
        value = 0xCBF29CE484222325
        for byte in name.encode():
            value = ((value ^ byte) * 0x100000001B3) & MASK
        return value

    lib = _native.lib()
    assert fnv("") == 0xCBF29CE484222325 and fnv("a") == 0xAF63DC4C8601EC8C  # FNV-1a's published test vectors
    for name in ("", "a", "paged_decode.key_cache"):
        assert lib.singe_hip_synthetic_seed(0x51A6E, name.encode()) == 0x51A6E ^ fnv(name)


def test_normal_values_follow_the_stated_recipe():
    seed = 0x51A6E ^ 77
    got = _normal(seed, 0, 4000)
    for i in range(2000):
        word = _word(seed, i)
        u1 = ((word >> 40) + 1) / 2.0 ** 24
        u2 = ((word >> 16) & 0xFFFFFF) / 2.0 ** 24
        radius = math.sqrt(-2.0 * math.log(u1))
        assert got[2 * i] == np.float32(radius * math.cos(2.0 * math.pi * u2))
        assert got[2 * i + 1] == np.float32(radius * math.sin(2.0 * math.pi * u2))


def test_any_range_by_any_number_of_threads():
    seed = 99
    whole = _normal(seed, 0, 300_001)
    for first, count, threads in ((0, 300_001, 7), (1, 299_999, 16), (777, 100_001, 3), (12_345, 5, 8), (299_999, 2, 4)):
        assert np.array_equal(_normal(seed, first, count, threads), whole[first:first + count]), (first, count, threads)


def test_moments_and_independence_of_streams():
    a, b = _normal(1, 0, 1 << 21, 8), _normal(2, 0, 1 << 21, 8)
    for values in (a, b):
        assert abs(float(values.mean())) < 3e-3 and abs(float(values.std()) - 1.0) < 3e-3
        assert np.isfinite(values).all() and np.abs(values).max() < 5.8  # sqrt(-2 ln 2^-24) = 5.77
    assert abs(float(np.mean(a * b))) < 3e-3
    assert abs(float(np.mean(a[::2] * a[1::2]))) < 3e-3  # the two values of a word


def test_integers_and_permutation():
    lib = _native.lib()
    out = np.empty(10_000, dtype=np.int64)
    lib.singe_hip_synthetic_integers(5, 0, 512, 4096 - 512 + 1, out.ctypes.data, out.size)
    assert out.min() >= 512 and out.max() <= 4096 and len(np.unique(out)) > 3000
    assert out[3] == 512 + (((_word(5, 3) >> 32) * (4096 - 512 + 1)) >> 32)
    count = 4099
    perm = np.empty(count, dtype=np.int64)
    lib.singe_hip_synthetic_permutation(6, perm.ctypes.data, count)
    want = list(range(count))
    for k in range(count - 1):
        i = count - 1 - k
        j = ((_word(6, k) >> 32) * (i + 1)) >> 32
        want[i], want[j] = want[j], want[i]
    assert perm.tolist() == want and sorted(want) == list(range(count))


def test_portable_workloads_do_not_depend_on_how_they_are_cut():
    kwargs = dict(batch=3, heads=8, kv_heads=2, physical_blocks=96, min_len=100, max_len=300, device="cpu", portable=True)
    one = synthetic.paged_decode_fp8_workload(chunk_blocks=96, **kwargs)
    other = synthetic.paged_decode_fp8_workload(chunk_blocks=7, **kwargs)
    assert torch.equal(one.key_cache, other.key_cache) and torch.equal(one.value_scales, other.value_scales)
    assert np.array_equal(one.seq_lens, other.seq_lens) and np.array_equal(one.block_table, other.block_table)
    # the benchmark's headline lengths: 32 draws from [512, 4096]
    lens = synthetic._PortableSource(synthetic.BASE_SEED, "cpu", "paged_decode").integers("seq_lens", 512, 4096, 32)
    assert int(lens.sum()) == 74_560
