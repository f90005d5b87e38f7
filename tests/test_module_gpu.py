"""The code object on a device: every kernel the library names resolves from the part it is said to live in."""
import ctypes

import pytest
import torch

from singe_amd import _native

pytestmark = pytest.mark.gpu


def test_every_kernel_resolves_on_the_device():
    torch.cuda.set_device(0)
    lib = _native.lib()
    listed = 0
    while lib.singe_hip_kernel(listed, None, None) == 0:
        listed += 1
    found = ctypes.c_int32(0)
    _native.check(lib.singe_hip_prepare(ctypes.byref(found)), "prepare")
    assert found.value == listed >= 113
    # torch's own launches still find a clean error state afterwards
    assert float((torch.ones(8, device="cuda") * 2).sum().item()) == 16.0
