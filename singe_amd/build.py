"""Builds the two native artefacts in-tree:

* ``singe_attention_gfx950.hsaco``: the gfx950 code object (hipcc --genco), and
* ``libsinge_hip_attention.so``: the C-ABI launcher (plain g++, no ROCm link dependency).

Run as ``python -m singe_amd.build``.  hipcc cross-compiles, so no GPU is needed.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
CODE_OBJECT = os.path.join(HERE, "singe_attention_gfx950.hsaco")
LIBRARY = os.path.join(HERE, "libsinge_hip_attention.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "--genco", "-O3", "-std=c++17",
    # packed fp32 VALU forms are kept off on this hardware pool
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]
HOST_SOURCES = ["hip_runtime_loader.cpp", "module.cpp", "paged_decode.cpp", "fmha_prefill.cpp", "paged_attention.cpp",
                "general_attention.cpp", "fmha_decode.cpp", "paged_rows_f32.cpp", "latent_attention.cpp", "cache_ops.cpp"]


def _run(cmd):
    print("+", " ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)


def hipcc() -> str:
    found = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(found):
        raise RuntimeError("hipcc not found")
    return found


def build_code_object(extra_flags=()) -> str:
    source = os.path.join(CSRC, "singe_attention_kernels.hip")
    _run([hipcc(), *HIPCC_FLAGS, *extra_flags, "-I", CSRC, source, "-o", CODE_OBJECT])
    return CODE_OBJECT


def build_library() -> str:
    sources = [os.path.join(CSRC, name) for name in HOST_SOURCES]
    _run(["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden", "-Wall", "-Wextra",
          "-I", os.path.join(ROOT, "include"), "-I", CSRC, *sources, "-o", LIBRARY, "-ldl", "-lpthread",
          "-Wl,--no-undefined"])
    return LIBRARY


def build() -> None:
    build_code_object()
    build_library()


if __name__ == "__main__":
    build()
    sys.exit(0)
