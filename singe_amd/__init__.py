"""MI355X-native attention hot path behind the reference's op API.

``singe_amd.kernel.attention`` mirrors ``singe_kernel::cuda::attention`` (config structs and launch
functions); the kernels are hand-written gfx950 HIP in ``csrc/``, built into a code object that
``libsinge_hip_attention.so`` loads and launches through the C ABI of ``include/singe_hip_attention.h``.
"""
from . import error  # noqa: F401

__all__ = ["error"]
