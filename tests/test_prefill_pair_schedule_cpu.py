"""The two-tile prefill kernels (dense and paged) write their score products as assembly (the compiler would give them
accumulation-register destinations), so the compiler does not know that those statements are matrix instructions and
keeps no distance between them and what reads their results: the distance is part of the kernel's hand-made schedule.
This test compiles the kernel to gfx950 assembly and checks, on what the compiler actually emitted (its register
allocator may add copies of its own), that no instruction touches the destination registers of such a product for at
least as many issue slots after it as the instruction's passes need (an 8-pass product: 11 wait states before a
vector instruction may read it), other than the next product of the same accumulation chain; and that no vector
instruction writes an operand of such a product in the two issue slots before it."""
import os
import re
import subprocess
import tempfile

import pytest

from singe_amd import build

CSRC = os.path.join(os.path.dirname(build.__file__), "csrc")
# (source, extra flags): every build of the two-tile kernels
BUILDS = [(source, [] if dim == 128 else [f"-DSINGE_HEAD_DIM={dim}"]) for dim in (128, 112, 96, 80, 64, 48, 32, 16)
          for source in ("fmha_prefill_pair.hip", "paged_attention_pair.hip")]
WAIT_STATES = 12


def registers(text, bank="v"):
    """Vector registers (v5, v[18:33]; bank "a": accumulation registers) an instruction's operand text names."""
    found = set()
    for first, last in re.findall(rf"\b{bank}\[(\d+):(\d+)\]", text):
        found.update(range(int(first), int(last) + 1))
    for single in re.findall(rf"\b{bank}(\d+)\b", text):
        found.add(int(single))
    return found


def instructions(assembly):
    """(text, inside an asm statement) for every instruction line, in program order."""
    inside = False
    for line in assembly.splitlines():
        stripped = line.strip()
        if stripped.startswith(";;#ASMSTART"):
            inside = True
            continue
        if stripped.startswith(";;#ASMEND"):
            inside = False
            continue
        if not stripped or stripped.startswith((";", ".", "//")) or stripped.endswith(":"):
            continue
        yield stripped.split(";")[0].strip(), inside


def assembly_of(name, flags):
    source = os.path.join(CSRC, name)
    with tempfile.TemporaryDirectory() as scratch:
        listing = os.path.join(scratch, "pair.s")
        command = [build.hipcc()] + [flag for flag in build.HIPCC_FLAGS if flag != "--genco"] + flags + [
            "--cuda-device-only", "-S", "-I", os.path.dirname(source), source, "-o", listing]
        subprocess.run(command, check=True, capture_output=True)
        return open(listing).read()


@pytest.fixture(scope="module")
def listings():
    """Every build's assembly, compiled side by side (a build takes a quarter of a minute)."""
    from concurrent.futures import ThreadPoolExecutor
    with ThreadPoolExecutor(max_workers=min(8, os.cpu_count() or 1)) as pool:
        texts = list(pool.map(lambda item: assembly_of(*item), BUILDS))
    return {(name, tuple(flags)): text for (name, flags), text in zip(BUILDS, texts)}


@pytest.mark.parametrize("name,flags", BUILDS, ids=lambda value: value if isinstance(value, str) else "".join(value) or "d128")
def test_nothing_touches_a_score_product_before_it_is_done(listings, name, flags):
    steps = int(flags[0].split("=")[1]) // 16 if flags else 8  # score products a chain
    program = list(instructions(listings[(name, tuple(flags))]))
    products = 0
    for at, (text, inside) in enumerate(program):
        if not (inside and text.startswith("v_mfma")):
            continue
        products += 1
        destination = registers(text.split(",")[0])
        assert len(destination) == 16, text
        # Operands written by a vector instruction just before (loads are waited for by a counter the compiler sets).
        sources = text.split(",", 1)[1]
        waited = 0
        for earlier, _ in reversed(program[max(0, at - 4):at]):
            nop = re.match(r"s_nop (\d+)", earlier)
            if nop:
                waited += int(nop.group(1)) + 1
                continue
            if waited >= 2:
                break
            if earlier.startswith("v_") and not earlier.startswith("v_mfma"):
                written = earlier.split(" ", 1)[1].split(",")[0]
                assert not (registers(written) & registers(sources)), f"{earlier!r} writes an operand of {text!r}"
                assert not (registers(written, "a") & registers(sources, "a")), f"{earlier!r} writes an operand of {text!r}"
            waited += 1
        waited = 0
        for later, later_inside in program[at + 1:]:
            if waited >= WAIT_STATES:
                break
            same_chain = later_inside and later.startswith("v_mfma") and registers(later.split(",")[0]) == destination
            if same_chain:
                break  # the chain's next product: the hardware forwards the accumulator
            assert not (registers(later) & destination), f"{later!r} follows {text!r} after {waited} wait states"
            nop = re.match(r"s_nop (\d+)", later)
            waited += int(nop.group(1)) + 1 if nop else 1
            if later.startswith("v_mfma"):
                waited += 7  # a matrix instruction holds the issue for its passes
    assert products >= 4 * 4 * steps  # four kernels at least, two blocks of two chains each
    # Q^T is loaded into accumulation registers by a statement the compiler does not know to be a load: nothing may
    # name those registers before the wait that follows the loads.
    loads = 0
    into_accumulation = ("global_load_dwordx4 a[", "ds_read_b128 a[")  # (the second: a Q^T worked out first and parked in LDS)
    for at, (text, inside) in enumerate(program):
        if not (inside and text.startswith(into_accumulation)):
            continue
        loads += 1
        loaded = registers(text.split(",")[0].split(" ", 1)[1], "a")
        for later, later_inside in program[at + 1:]:
            if later_inside and later.startswith("s_waitcnt vmcnt(0) lgkmcnt(0)"):
                break
            if later_inside and later.startswith(into_accumulation):
                continue
            assert not (registers(later, "a") & loaded), f"{later!r} names what {text!r} is still loading"
    assert loads >= 4 * 2 * steps


def test_the_block_texts_are_what_the_dealing_script_writes():
    # the .inc files beside the kernels are generated: a hand edit, or a change to the script that was not run, shows here
    import importlib.util
    spec = importlib.util.spec_from_file_location("prefill_pair_deal", os.path.join(CSRC, "prefill_pair_deal.py"))
    dealing = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(dealing)
    for dim, budget, load_slots in dealing.BLOCKS:
        body, used = dealing.deal(dim // 16, (dim + 31) // 32, budget, load_slots)
        text = dealing.HEADER.format(dim=dim, used=" ".join(f"{u:.0f}" for u in used)) + body
        assert open(os.path.join(CSRC, f"prefill_pair_block_d{dim}.inc")).read() == text, dim
