"""Kernels whose loops cannot afford memory behind a register: a spilled register's reload waits on the counter that
the direct-to-LDS tile loads run on and drains them, and an accumulator array indexed by a variable anywhere in the
kernel lives in scratch memory for all of it (a loop that may end early is not unrolled).  This test compiles those
sources for gfx950 with the compiler's resource remarks and checks that the kernels named here use no scratch memory."""
import os
import re
import subprocess
import tempfile
from concurrent.futures import ThreadPoolExecutor

import pytest

from singe_amd import build

CSRC = os.path.join(os.path.dirname(build.__file__), "csrc")
# source, flags, kernels (regular expressions) that must not touch scratch memory
BUILDS = [
    ("latent_attention_mfma.hip", [], [r"singe_paged_mla_attention_(bf16|f16)_(l512_p64|any)"]),
    ("fmha_prefill_pair.hip", [], [r"singe_fmha_prefill_pair_.*"]),
    ("paged_attention_pair.hip", [], [r"singe_(rotary_)?paged_attention_pair_.*"]),
    ("paged_decode.hip", [], [r"singe_paged_decode_(bf16|f16)_d128_g1_b16", r"singe_paged_decode_f8kv_wide(_relaxed)?_d128_b16",
                              r"singe_paged_decode_(bf16|f16)_wide_d128_b16"]),
]


def remarks_of(name, flags):
    source = os.path.join(CSRC, name)
    with tempfile.TemporaryDirectory() as scratch:
        command = [build.hipcc()] + build.HIPCC_FLAGS + flags + ["-Rpass-analysis=kernel-resource-usage", "-I", os.path.dirname(source),
                                                                  source, "-o", os.path.join(scratch, "out.hsaco")]
        return subprocess.run(command, check=True, capture_output=True, text=True).stderr


@pytest.fixture(scope="module")
def remarks():
    with ThreadPoolExecutor(max_workers=min(4, os.cpu_count() or 1)) as pool:
        texts = list(pool.map(lambda item: remarks_of(item[0], item[1]), BUILDS))
    return {name: text for (name, _, _), text in zip(BUILDS, texts)}


@pytest.mark.parametrize("name,flags,patterns", BUILDS, ids=[item[0] for item in BUILDS])
def test_no_scratch_memory_in_the_kernels_that_cannot_afford_it(remarks, name, flags, patterns):
    scratch = {}
    kernel = None
    for line in remarks[name].splitlines():
        found = re.search(r"Function Name: (\S+)", line)
        if found:
            kernel = found.group(1)
        found = re.search(r"ScratchSize \[bytes/lane\]: (\d+)", line)
        if found and kernel is not None:
            scratch[kernel] = int(found.group(1))
    for pattern in patterns:
        named = {kernel: size for kernel, size in scratch.items() if re.fullmatch(pattern, kernel)}
        assert named, f"no kernel of {name} matches {pattern}"
        assert all(size == 0 for size in named.values()), {kernel: size for kernel, size in named.items() if size}
