"""Builds the two native artefacts in-tree:

* ``singe_attention_gfx950.hsaco``: the gfx950 code object (hipcc --genco), and
* ``libsinge_hip_attention.so``: the C-ABI launcher (plain g++; it resolves the HIP runtime with dlopen, and
  links it only for the one hipcc-built unit that holds the fixed device scratch).

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
STATIC_SCRATCH_OBJECT = os.path.join(HERE, "csrc", "static_scratch.o")

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


def rocm_lib_dir() -> str:
    return os.path.join(os.path.dirname(os.path.dirname(os.path.realpath(hipcc()))), "lib")


def build_static_scratch() -> str:
    """The one host + device translation unit: the fixed device scratch of the entry points that allocate
    nothing, whose address the host takes with hipGetSymbolAddress (so it is registered with the runtime,
    not loaded as a module)."""
    source = os.path.join(CSRC, "static_scratch.hip")
    _run([hipcc(), "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
          "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
          "-I", os.path.join(ROOT, "include"), "-I", CSRC, "-c", source, "-o", STATIC_SCRATCH_OBJECT])
    return STATIC_SCRATCH_OBJECT


def build_library() -> str:
    sources = [os.path.join(CSRC, name) for name in HOST_SOURCES]
    lib_dir = rocm_lib_dir()
    _run(["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden", "-Wall", "-Wextra",
          "-I", os.path.join(ROOT, "include"), "-I", CSRC, *sources, build_static_scratch(), "-o", LIBRARY,
          "-L", lib_dir, "-lamdhip64", f"-Wl,-rpath,{lib_dir}", "-ldl", "-lpthread", "-Wl,--no-undefined"])
    return LIBRARY


def build() -> None:
    build_code_object()
    build_library()


if __name__ == "__main__":
    build()
    sys.exit(0)
