"""Builds the native artefacts in-tree:

* ``singe_attention_gfx950.<part>.hsaco``: the gfx950 code object, one part per kernel source (hipcc --genco), built
  side by side,
* ``singe_attention_gfx950.parts``: the same parts in one archive, the image ``singe_hip_load`` takes from a caller
  that embeds the kernels instead of shipping files, and
* ``libsinge_hip_attention.so``: the C-ABI launcher (plain g++; it resolves the HIP runtime with dlopen, and
  links it only for the one hipcc-built unit that holds the fixed device scratch).

Run as ``python -m singe_amd.build`` (everything) or ``python -m singe_amd.build --changed`` (only the parts whose
sources changed since they were last built).  hipcc cross-compiles, so no GPU is needed.
"""
from __future__ import annotations

import hashlib
import os
import re
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIBRARY = os.path.join(HERE, "libsinge_hip_attention.so")
STATIC_SCRATCH_OBJECT = os.path.join(HERE, "csrc", "static_scratch.o")

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "--genco", "-O3", "-std=c++17",
    # packed fp32 VALU forms are kept off on this hardware pool
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]
# (part name, source file, extra flags), in the order of kPartNames in csrc/module.cpp.
PARTS = [
    ("paged_decode", "paged_decode.hip", []),
    ("fmha_prefill", "fmha_prefill.hip", []),
    ("fmha_prefill_f32", "fmha_prefill_f32.hip", []),
    ("paged_attention", "paged_attention.hip", []),
    ("splitk_reduce", "splitk_reduce.hip", []),
    ("attention_rows_f32", "attention_rows_f32.hip", []),
    ("cache_ops", "cache_ops.hip", []),
    ("latent_attention", "latent_attention.hip", []),
    ("latent_attention_mfma", "latent_attention_mfma.hip", []),
    ("general_attention_f32", "general_attention.hip", ["-DSINGE_GENERAL_ELEMENT=0"]),
    ("general_attention_bf16", "general_attention.hip", ["-DSINGE_GENERAL_ELEMENT=1"]),
    ("general_attention_f16", "general_attention.hip", ["-DSINGE_GENERAL_ELEMENT=2"]),
    ("mfma_ceiling", "mfma_ceiling.hip", []),
    ("paged_decode_d64", "paged_decode.hip", ["-DSINGE_HEAD_DIM=64"]),
    ("fmha_prefill_d64", "fmha_prefill.hip", ["-DSINGE_HEAD_DIM=64"]),
    ("paged_attention_d64", "paged_attention.hip", ["-DSINGE_HEAD_DIM=64"]),
    ("general_attention_f64", "general_attention.hip", ["-DSINGE_GENERAL_ELEMENT=3"]),
    ("hbm_stream", "hbm_stream.hip", []),
    ("fmha_prefill_d32", "fmha_prefill.hip", ["-DSINGE_HEAD_DIM=32"]),
    ("paged_attention_d32", "paged_attention.hip", ["-DSINGE_HEAD_DIM=32"]),
    ("fmha_prefill_d96", "fmha_prefill.hip", ["-DSINGE_HEAD_DIM=96"]),
    ("paged_attention_d96", "paged_attention.hip", ["-DSINGE_HEAD_DIM=96"]),
    ("fmha_prefill_d16", "fmha_prefill.hip", ["-DSINGE_HEAD_DIM=16"]),
    ("paged_attention_d16", "paged_attention.hip", ["-DSINGE_HEAD_DIM=16"]),
    ("fmha_prefill_d48", "fmha_prefill.hip", ["-DSINGE_HEAD_DIM=48"]),
    ("paged_attention_d48", "paged_attention.hip", ["-DSINGE_HEAD_DIM=48"]),
    ("fmha_prefill_d80", "fmha_prefill.hip", ["-DSINGE_HEAD_DIM=80"]),
    ("paged_attention_d80", "paged_attention.hip", ["-DSINGE_HEAD_DIM=80"]),
    ("fmha_prefill_d112", "fmha_prefill.hip", ["-DSINGE_HEAD_DIM=112"]),
    ("paged_attention_d112", "paged_attention.hip", ["-DSINGE_HEAD_DIM=112"]),
    ("paged_decode_d32", "paged_decode.hip", ["-DSINGE_HEAD_DIM=32"]),
    ("paged_decode_d16", "paged_decode.hip", ["-DSINGE_HEAD_DIM=16"]),
    ("paged_decode_d48", "paged_decode.hip", ["-DSINGE_HEAD_DIM=48"]),
    ("paged_decode_d80", "paged_decode.hip", ["-DSINGE_HEAD_DIM=80"]),
    ("paged_decode_d96", "paged_decode.hip", ["-DSINGE_HEAD_DIM=96"]),
    ("paged_decode_d112", "paged_decode.hip", ["-DSINGE_HEAD_DIM=112"]),
    ("fmha_prefill_pair", "fmha_prefill_pair.hip", []),
    ("paged_attention_pair", "paged_attention_pair.hip", []),
    ("fmha_prefill_pair_d64", "fmha_prefill_pair.hip", ["-DSINGE_HEAD_DIM=64"]),
    ("paged_attention_pair_d64", "paged_attention_pair.hip", ["-DSINGE_HEAD_DIM=64"]),
    ("fmha_prefill_pair_d96", "fmha_prefill_pair.hip", ["-DSINGE_HEAD_DIM=96"]),
    ("paged_attention_pair_d96", "paged_attention_pair.hip", ["-DSINGE_HEAD_DIM=96"]),
    ("fmha_prefill_pair_d112", "fmha_prefill_pair.hip", ["-DSINGE_HEAD_DIM=112"]),
    ("paged_attention_pair_d112", "paged_attention_pair.hip", ["-DSINGE_HEAD_DIM=112"]),
    ("fmha_prefill_pair_d80", "fmha_prefill_pair.hip", ["-DSINGE_HEAD_DIM=80"]),
    ("paged_attention_pair_d80", "paged_attention_pair.hip", ["-DSINGE_HEAD_DIM=80"]),
    ("fmha_prefill_pair_d48", "fmha_prefill_pair.hip", ["-DSINGE_HEAD_DIM=48"]),
    ("paged_attention_pair_d48", "paged_attention_pair.hip", ["-DSINGE_HEAD_DIM=48"]),
    ("fmha_prefill_pair_d32", "fmha_prefill_pair.hip", ["-DSINGE_HEAD_DIM=32"]),
    ("paged_attention_pair_d32", "paged_attention_pair.hip", ["-DSINGE_HEAD_DIM=32"]),
    ("fmha_prefill_pair_d16", "fmha_prefill_pair.hip", ["-DSINGE_HEAD_DIM=16"]),
    ("paged_attention_pair_d16", "paged_attention_pair.hip", ["-DSINGE_HEAD_DIM=16"]),
]
HOST_SOURCES = ["hip_runtime_loader.cpp", "module.cpp", "paged_decode.cpp", "fmha_prefill.cpp", "paged_attention.cpp",
                "general_attention.cpp", "fmha_decode.cpp", "paged_rows_f32.cpp", "latent_attention.cpp", "cache_ops.cpp",
                "mfma_ceiling.cpp", "attention_parameters.cpp", "synthetic_inputs.cpp", "attention_family.cpp"]
JOBS = 8


def code_object(part: str) -> str:
    return os.path.join(HERE, f"singe_attention_gfx950.{part}.hsaco")


CODE_OBJECTS = [code_object(part) for part, _, _ in PARTS]


def _run(cmd):
    print("+", " ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)


def hipcc() -> str:
    found = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(found):
        raise RuntimeError("hipcc not found")
    return found


def _closure(source: str, seen=None) -> list:
    """The source and every header of this directory it includes, directly or not."""
    seen = seen if seen is not None else []
    path = os.path.join(CSRC, source)
    if path in seen or not os.path.exists(path):
        return seen
    seen.append(path)
    for name in re.findall(r'#include "([^"]+)"', open(path).read()):
        _closure(name, seen)
    return seen


def _fingerprint(source: str, flags) -> str:
    digest = hashlib.sha256(" ".join([*HIPCC_FLAGS, *flags]).encode())
    for path in sorted(_closure(source)):
        digest.update(open(path, "rb").read())
    return digest.hexdigest()


def build_part(part: str, source: str, flags, only_changed: bool = False) -> str:
    target, stamp = code_object(part), code_object(part) + ".stamp"
    fingerprint = _fingerprint(source, flags)
    if only_changed and os.path.exists(target) and os.path.exists(stamp) and open(stamp).read() == fingerprint:
        return target
    _run([hipcc(), *HIPCC_FLAGS, *flags, "-I", CSRC, os.path.join(CSRC, source), "-o", target])
    with open(stamp, "w") as handle:
        handle.write(fingerprint)
    return target


def build_code_object(only_changed: bool = False, parts=None) -> list:
    wanted = [entry for entry in PARTS if parts is None or entry[0] in parts]
    with ThreadPoolExecutor(max_workers=JOBS) as pool:
        return list(pool.map(lambda entry: build_part(*entry, only_changed=only_changed), wanted))


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


ARCHIVE = os.path.join(HERE, "singe_attention_gfx950.parts")
ARCHIVE_MAGIC = b"SINGE_HIP_PARTS\0"


def pack_archive(parts=None) -> bytes:
    """The parts' code objects as one image for ``singe_hip_load`` (what an embedding caller keeps with
    ``include_bytes!``): the magic, u32 version 1, u32 entries, then per entry the part's name in 48 bytes, u64 offset
    and u64 size, then the code objects, each at a multiple of 16 bytes.  Little-endian."""
    import struct

    names = [part for part, _, _ in PARTS if parts is None or part in parts]
    images = [open(code_object(part), "rb").read() for part in names]
    offset = 24 + 64 * len(names)
    table, body = b"", b""
    for name, image in zip(names, images):
        offset += -offset % 16
        table += struct.pack("<48sQQ", name.encode(), offset, len(image))
        offset += len(image)
    position = 24 + len(table)
    for image in images:
        body += b"\0" * (-(position + len(body)) % 16) + image
    return ARCHIVE_MAGIC + struct.pack("<II", 1, len(names)) + table + body


def write_archive() -> str:
    with open(ARCHIVE, "wb") as handle:
        handle.write(pack_archive())
    return ARCHIVE


def build(only_changed: bool = False) -> None:
    build_code_object(only_changed=only_changed)
    write_archive()
    build_library()


if __name__ == "__main__":
    build(only_changed="--changed" in sys.argv[1:])
    sys.exit(0)
