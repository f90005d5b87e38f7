"""No-GPU checks of the C-ABI library and the host layer: the library loads, exports every symbol the
header declares, and every validation that the reference performs before a launch returns the same
error without touching a device."""
import ctypes
import os
import re

import pytest

from singe_amd import _native, error
from singe_amd.kernel import attention as A

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "singe_hip_attention.h")).read()
    return sorted(set(re.findall(r"SINGE_HIP_API[^;(]*?\b(singe_hip_\w+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _native.lib()
    names = declared_symbols()
    assert len(names) >= 20
    for name in names:
        assert hasattr(lib, name), name


def test_code_object_is_built_and_every_part_names_its_kernels():
    images = {}
    for part, path in zip(_native.CODE_OBJECT_PARTS, _native.CODE_OBJECT_PATHS):
        assert os.path.exists(path), path
        images[part] = open(path, "rb").read()
    lib, names = _native.lib(), []
    name, part = ctypes.c_char_p(), ctypes.c_char_p()
    index = 0
    while lib.singe_hip_kernel(index, ctypes.byref(name), ctypes.byref(part)) == 0:
        assert name.value in images[part.value.decode()], (name.value, part.value)
        names.append(name.value)
        index += 1
    assert len(names) == len(set(names)) >= 113
    for kernel in (b"singe_paged_decode_bf16_d128_g1_b16", b"singe_paged_decode_f8kv_wide_d128_b16",
                   b"singe_paged_decode_combine_bf16", b"singe_fmha_prefill_bf16_d128_causal",
                   b"singe_fmha_prefill_f32_d64", b"singe_paged_attention_bf16_d128_i64", b"singe_paged_attention_bf16_d128_i32_p16",
                   b"singe_paged_kv_prefill_bf16_d128_p16", b"singe_rotary_paged_attention_bf16_d128_i64_p16"):
        assert kernel in names, kernel


def test_status_strings():
    lib = _native.lib()
    assert lib.singe_hip_status_string(0) == b"ok"
    assert lib.singe_hip_status_string(1) == b"invalid length"
    assert lib.singe_hip_status_string(2) == b"length too short"


GOOD = dict(batch=2, heads=8, kv_heads=2, head_dim=128, block_size=16, physical_blocks=8,
            block_table_batch_stride=4, scale=0.1)


def decode_status(config, lens=None, pointers=None):
    lens = lens or dict(out=2 * 8 * 128, query=2 * 8 * 128, key=8 * 16 * 2 * 128, value=8 * 16 * 2 * 128, seq=2, table=8)
    fake = 0x1000
    p = pointers or {}
    return _native.lib().singe_hip_paged_kv_decode_attention_bf16(
        None, p.get("out", fake), lens["out"], p.get("query", fake), lens["query"], p.get("key", fake), lens["key"],
        p.get("value", fake), lens["value"], p.get("seq", fake), lens["seq"], p.get("table", fake), lens["table"],
        p.get("workspace", fake), 1 << 30, ctypes.byref(config))


def test_decode_validation_order_and_codes():
    # validate_paged_kv_decode_attention_config, then validate_lengths (mod.rs:711-743, 2963-2985)
    for bad in (dict(batch=0), dict(heads=7), dict(scale=float("inf")), dict(physical_blocks=0)):
        with pytest.raises(error.InvalidLength):
            A.PagedKvDecodeAttentionConfig.contiguous(**{**GOOD, **bad})
        c = A.PagedKvDecodeAttentionConfig(**{**GOOD, **bad})._c()
        assert decode_status(c) == 1
    with pytest.raises(error.LengthExceedsI32):
        A.PagedKvDecodeAttentionConfig.contiguous(**{**GOOD, "batch": 2**31})
    assert decode_status(A.PagedKvDecodeAttentionConfig(**{**GOOD, "batch": 2**31})._c()) == 3
    c = A.PagedKvDecodeAttentionConfig.contiguous(**GOOD)._c()
    full = dict(out=2 * 8 * 128, query=2 * 8 * 128, key=8 * 16 * 2 * 128, value=8 * 16 * 2 * 128, seq=2, table=8)
    for name in full:
        status = decode_status(c, {**full, name: full[name] - 1})
        assert status == 2, name
        detail = _native.ErrorDetail()
        _native.lib().singe_hip_last_error(ctypes.byref(detail))
        assert detail.minimum == full[name] and detail.actual == full[name] - 1
    assert decode_status(c, pointers=dict(query=None)) == 6
    big = 1 << 30  # buffers long enough for any width: head dimensions past 256 have no kernel at all
    wide = dict(out=big, query=big, key=big, value=big, seq=2, table=8)
    assert decode_status(A.PagedKvDecodeAttentionConfig(**{**GOOD, "head_dim": 320})._c(), wide) == 5
    with pytest.raises(error.UnsupportedWidth):
        _native.check(5, "paged_kv_decode_attention_bf16")


def test_decode_workspace_query_needs_no_device():
    c = A.PagedKvDecodeAttentionConfig.contiguous(**GOOD)
    assert c.workspace_bytes() > 0
    assert _native.lib().singe_hip_paged_kv_decode_attention_workspace_bytes(None) == 0


def test_fmha_config_validation():
    good = A.FmhaPrefillConfig.contiguous(1, 64, 64, 4, 2, 128, 0.1, True)
    lib = _native.lib()
    assert lib.singe_hip_fmha_prefill_config_validate(ctypes.byref(good._c())) == 0
    from dataclasses import replace
    for bad in (replace(good, key_len=0), replace(good, kv_heads=3), replace(good, scale=float("nan")),
                replace(good, query_head_stride=0)):
        assert lib.singe_hip_fmha_prefill_config_validate(ctypes.byref(bad._c())) == 1
    # validate_lengths: a buffer shorter than the strides can reach
    fake = 0x1000
    need = 64 * 4 * 128
    status = lib.singe_hip_fmha_prefill_bf16(None, fake, need, fake, need - 1, fake, 64 * 2 * 128, fake, 64 * 2 * 128,
                                             ctypes.byref(good._c()))
    assert status == 2
    assert lib.singe_hip_fmha_prefill_bf16(None, fake, need, fake, need, None, 64 * 2 * 128, fake, 64 * 2 * 128,
                                           ctypes.byref(good._c())) == 6


def test_paged_attention_problem_validation():
    lib = _native.lib()
    fake = 0x1000
    def call(**changes):
        fields = dict(tokens=2, heads=2, kv_heads=2, head_dim=128, page_size=4, sequences=1, cache_pages=2, page_table=1,
                      index_type=1, causal=1, has_scale=0, has_window=0, has_softcap=0, scale=0.0, softcap=0.0, window=0)
        fields.update(changes)
        problem = _native.PagedAttentionProblemC(*fields.values())
        return lib.singe_hip_paged_attention_bf16(None, *([fake] * 10), ctypes.byref(problem))
    assert call(kv_heads=0) == 9
    assert call(heads=3) == 9
    assert call(page_size=0) == 9
    assert call(index_type=7) == 9
    assert call(head_dim=300) == 5  # beyond the general kernel's 256
    detail = _native.ErrorDetail()
    lib.singe_hip_last_error(ctypes.byref(detail))
    assert detail.minimum == 300  # the refused width
    assert call(tokens=0) == 0  # nothing to attend, nothing launched


def test_rotary_paged_attention_validation():
    lib = _native.lib()
    fake = 0x1000
    def call(rotation, cos=fake, **changes):
        fields = dict(tokens=2, heads=2, kv_heads=2, head_dim=128, page_size=4, sequences=1, cache_pages=2, page_table=1,
                      index_type=1, causal=1, has_scale=0, has_window=0, has_softcap=0, scale=0.0, softcap=0.0, window=0)
        fields.update(changes)
        problem = _native.PagedAttentionProblemC(*fields.values())
        return lib.singe_hip_rotary_paged_attention_bf16(None, *([fake] * 7), cos, fake, None, fake, None, None, ctypes.byref(problem),
                                                         None if rotation is None else ctypes.byref(rotation))
    good = _native.QueryRotationC(0, 1, 1e-5)
    assert call(None) == 6                                       # no rotation attributes
    assert call(_native.QueryRotationC(7, 0, 0.0)) == 9          # unknown table type
    assert call(good, head_dim=72) == 5                          # the fused form takes the multiples of 16 up to 128
    assert call(good, head_dim=144) == 5 and call(good, head_dim=8) == 5
    assert call(good, has_softcap=1, softcap=float("nan")) == 9  # a cap is taken; a cap that is no number is not
    assert call(good, cos=None) == 6
    assert call(good, tokens=0) == 0
    assert call(good, tokens=0, head_dim=80, has_softcap=1, softcap=5.0) == 0


def test_paged_attention_scratch_query_needs_no_device():
    lib = _native.lib()
    def wanted(**changes):
        fields = dict(tokens=32, heads=32, kv_heads=8, head_dim=128, page_size=16, sequences=32, cache_pages=100, page_table=100,
                      index_type=0, causal=1, has_scale=0, has_window=0, has_softcap=0, scale=0.0, softcap=0.0, window=0)
        fields.update(changes)
        return lib.singe_hip_paged_attention_scratch_bytes(ctypes.byref(_native.PagedAttentionProblemC(*fields.values())))
    lib.singe_hip_set_paged_attention_splits(4)
    try:
        assert wanted() == 4 * 32 * 32 * 129 * 4     # shares x rows x (128 values + a log-sum-exp) of f32
        assert wanted(head_dim=64) == 4 * 32 * 32 * 65 * 4   # the head_dim 64 build splits the same way
        assert wanted(head_dim=96) == 4 * 32 * 32 * 97 * 4   # so do the builds for the other multiples of 16
        assert wanted(head_dim=80) == 4 * 32 * 32 * 81 * 4
        assert wanted(head_dim=72) == 0               # the general kernel does not split
    finally:
        lib.singe_hip_set_paged_attention_splits(0)
    assert lib.singe_hip_paged_attention_scratch_bytes(None) == 0


def test_paged_mla_attention_validation():
    lib = _native.lib()
    fake = 0x1000
    def call(**changes):
        fields = dict(tokens=2, heads=2, latent_dim=32, position_dim=8, page_size=4, sequences=1, cache_pages=2, page_table=1,
                      data_type=1, index_type=0, causal=1, has_scale=0, scale=0.0)
        fields.update(changes)
        problem = _native.PagedMlaAttentionProblemC(*fields.values())
        return lib.singe_hip_paged_mla_attention(None, *([fake] * 9), None, None, ctypes.byref(problem))
    assert call(page_size=0) == 9 and call(latent_dim=0) == 9      # paged_mla_attention_problem's own refusals
    assert call(data_type=4) == 9 and call(index_type=3) == 9
    assert call(has_scale=1, scale=float("nan")) == 9
    assert call(latent_dim=576) == 5 and call(position_dim=160) == 5
    assert call(tokens=0) == 0


def test_paged_kv_prefill_config_validation_mirrors_reference_cases():
    """singe-kernel/src/cuda/attention/tests.rs:349-375."""
    lib = _native.lib()
    good = _native.PagedKvPrefillAttentionConfigC(2, 7, 4, 2, 8, 3, 5, 4, 1, 0.5)
    assert lib.singe_hip_paged_kv_prefill_attention_config_validate(ctypes.byref(good)) == 0
    bad_heads = _native.PagedKvPrefillAttentionConfigC(2, 7, 3, 2, 8, 3, 5, 4, 1, 0.5)
    assert lib.singe_hip_paged_kv_prefill_attention_config_validate(ctypes.byref(bad_heads)) == 1
    fake = 0x1000
    status = lib.singe_hip_paged_kv_prefill_attention_bf16(None, fake, 224, fake, 27, fake, 224, fake, 240, fake, 240, fake, 2,
                                                           fake, 2, fake, 2, fake, 8, ctypes.byref(good))
    assert status == 2
    detail = _native.ErrorDetail()
    lib.singe_hip_last_error(ctypes.byref(detail))
    assert detail.name == b"lse" and detail.minimum == 28 and detail.actual == 27


def test_dense_problem_and_splitk_validation():
    lib = _native.lib()
    fake = 0x1000
    def dense(**changes):
        fields = dict(batch=1, heads=4, kv_heads=2, query_len=3, key_len=5, head_dim=64, value_dim=64,
                      mask_strides=(ctypes.c_int64 * 4)(0, 0, 0, 0), data_type=0, causal=0, has_scale=0, has_window=0,
                      has_softcap=0, scale=0.0, softcap=0.0, window=0)
        fields.update(changes)
        problem = _native.AttentionProblemC(*fields.values())
        return lib.singe_hip_scaled_dot_product_attention(None, fake, fake, fake, None, None, None, fake, ctypes.byref(problem))
    assert dense(kv_heads=3) == 9
    assert dense(key_len=0) == 9
    assert dense(head_dim=0) == 9
    assert dense(data_type=5) == 9
    assert dense(head_dim=257) == 5
    assert dense(query_len=0) == 0  # an empty output, nothing launched
    assert dense(has_softcap=1, softcap=0.0) == 9
    config = _native.SplitKReduceConfigC(1, 2, 5, 8, 80, 40, 8, 10, 5, 16, 8)
    assert lib.singe_hip_splitk_reduce_f32(None, fake, 16, fake, 80, fake, 10, ctypes.byref(config)) != 2
    assert lib.singe_hip_splitk_reduce_f32(None, fake, 16, fake, 79, fake, 10, ctypes.byref(config)) == 2
    zero = _native.SplitKReduceConfigC(1, 2, 0, 8, 80, 40, 8, 10, 5, 16, 8)
    assert lib.singe_hip_splitk_reduce_f32(None, fake, 16, fake, 80, fake, 10, ctypes.byref(zero)) == 1


def test_f32_block_table_ops_validate_like_the_bf16_ones():
    lib = _native.lib()
    fake = 0x1000
    config = _native.PagedKvDecodeAttentionConfigC(**GOOD)
    lens = dict(out=2 * 8 * 128, query=2 * 8 * 128, key=8 * 16 * 2 * 128, value=8 * 16 * 2 * 128, seq=2, table=8)
    def decode(config=config, workspace=fake, workspace_bytes=1 << 30, **short):
        n = dict(lens, **short)
        return lib.singe_hip_paged_kv_decode_attention_f32(None, fake, n["out"], fake, n["query"], fake, n["key"], fake, n["value"],
                                                           fake, n["seq"], fake, n["table"], workspace, workspace_bytes, ctypes.byref(config))
    need = lib.singe_hip_paged_kv_decode_attention_f32_workspace_bytes(ctypes.byref(config))
    assert need == 2 * 8 * 64 * 129 * 4
    for name in ("out", "query", "key", "value", "seq", "table"):
        assert decode(**{name: lens[name] - 1}) == 2, name
    assert decode(workspace=None) == 6
    assert decode(workspace_bytes=need - 1) == 2
    assert decode(config=_native.PagedKvDecodeAttentionConfigC(**dict(GOOD, kv_heads=3))) == 1
    assert decode(config=_native.PagedKvDecodeAttentionConfigC(**dict(GOOD, head_dim=48)), out=1 << 20, query=1 << 20) == 5
    assert lib.singe_hip_paged_kv_decode_attention_f32_workspace_bytes(
        ctypes.byref(_native.PagedKvDecodeAttentionConfigC(**dict(GOOD, batch=0)))) == 0
    prefill = A.PagedKvPrefillAttentionConfig(2, 10, 4, 2, 64, 16, 8, 4, True, 0.1)._c()
    sizes = [10 * 4 * 64, 10 * 4, 10 * 4 * 64, 8 * 16 * 2 * 64, 8 * 16 * 2 * 64, 2, 2, 2, 8]
    def run(sizes, pointer=fake):
        flat = []
        for n in sizes:
            flat += [pointer, n]
        return lib.singe_hip_paged_kv_prefill_attention_f32(None, *flat, ctypes.byref(prefill))
    for index in range(9):
        short = list(sizes)
        short[index] -= 1
        assert run(short) == 2, index
    assert run(sizes, pointer=None) == 6


def test_parts_archive_is_checked_before_anything_changes():
    """singe_hip_load on an archive of parts: the build's own archive is taken; a wrong version, an entry count of
    zero, a part name the library does not know, a part listed twice and an entry that runs past the image are each
    refused with the status the header names, without a device."""
    import struct

    from singe_amd import build

    lib = _native.lib()
    magic = build.ARCHIVE_MAGIC
    entry = lambda name, offset, size: struct.pack("<48sQQ", name, offset, size)
    body = b"\x7fELF" + b"\0" * 60
    good = magic + struct.pack("<II", 1, 1) + entry(b"hbm_stream", 88, 64) + body
    try:
        assert lib.singe_hip_load(good, len(good)) == 0
        cases = {
            "version": (magic + struct.pack("<II", 2, 1) + entry(b"hbm_stream", 88, 64) + body, 9),
            "no entries": (magic + struct.pack("<II", 1, 0), 1),
            "entries past the image": (magic + struct.pack("<II", 1, 3) + entry(b"hbm_stream", 88, 64) + body, 1),
            "unknown part": (magic + struct.pack("<II", 1, 1) + entry(b"not_a_part", 88, 64) + body, 9),
            "part twice": (magic + struct.pack("<II", 1, 2) + entry(b"hbm_stream", 152, 64) + entry(b"hbm_stream", 152, 64) + body, 9),
            "runs past the end": (magic + struct.pack("<II", 1, 1) + entry(b"hbm_stream", 88, 65) + body, 2),
            "empty part": (magic + struct.pack("<II", 1, 1) + entry(b"hbm_stream", 88, 0) + body, 2),
            "header only": (magic + b"\x01", 1),
        }
        for name, (image, status) in cases.items():
            assert lib.singe_hip_load(image, len(image)) == status, name
        assert lib.singe_hip_load(None, 4) == 6 and lib.singe_hip_load(good, 0) == 1
        assert lib.singe_hip_load_part(b"hbm_stream", body, len(body)) == 0
        assert lib.singe_hip_load_part(b"hbm_strea", body, len(body)) == 9
        assert lib.singe_hip_load_part(b"hbm_stream_", body, len(body)) == 9
        assert lib.singe_hip_load_part(None, body, len(body)) == 6
    finally:
        lib.singe_hip_unload()


def test_build_archive_lists_every_part_at_aligned_offsets():
    import struct

    from singe_amd import build

    image = build.pack_archive()
    assert image[:16] == build.ARCHIVE_MAGIC
    version, entries = struct.unpack_from("<II", image, 16)
    assert version == 1 and entries == len(_native.CODE_OBJECT_PARTS)
    for index, (part, path) in enumerate(zip(_native.CODE_OBJECT_PARTS, _native.CODE_OBJECT_PATHS)):
        name, offset, size = struct.unpack_from("<48sQQ", image, 24 + 64 * index)
        assert name.rstrip(b"\0").decode() == part and offset % 16 == 0
        assert image[offset:offset + size] == open(path, "rb").read()


def test_fixed_scratch_limit_is_where_the_documents_say():
    """The entry point that allocates nothing refuses a config whose scratch exceeds the fixed array: at 32 query / 8 KV
    heads (and the 256 compute units the library assumes without a device) that is 759 sequences, not one more."""
    sized = lambda batch: A.PagedKvDecodeAttentionConfig.contiguous(batch, 32, 8, 128, 16, 16384, 256, 0.1).workspace_bytes()
    if not (0 < sized(1) < A.STATIC_SCRATCH_BYTES):
        pytest.skip("the library sees a device with another compute-unit count")
    text = open(os.path.join(ROOT, "include", "singe_hip_attention.h")).read()
    assert re.search(r"#define SINGE_HIP_STATIC_SCRATCH_BYTES \(16u << 20\)", text) and A.STATIC_SCRATCH_BYTES == 16 << 20
    assert sized(759) <= A.STATIC_SCRATCH_BYTES < sized(760)
    assert sized(32) < 5 << 20  # the headline decode shape uses under a third of it


def test_two_threads_hold_different_settings():
    """Per-thread options: each thread reads its own relaxed-numerics flag, decode workers and split threshold in the
    size queries it makes, whatever the other thread and the process-wide setters say meanwhile."""
    import threading

    lib = _native.lib()
    config = A.PagedKvDecodeAttentionConfig.contiguous(8, 32, 8, 128, 16, 1024, 64, 0.1)
    c = config._c()
    default_workers = int(lib.singe_hip_decode_workers(ctypes.byref(c)))
    default_bytes = config.workspace_bytes()
    barrier = threading.Barrier(2)
    seen, failures = {}, []

    def body(name, workers, relaxed, below):
        try:
            options = _native.ThreadOptionsC(relaxed, workers, 0, 0, 1, below)
            assert lib.singe_hip_set_thread_options(ctypes.byref(options)) == 0
            barrier.wait(timeout=10)
            if name == "a":  # a process-wide change made while both threads hold their own
                lib.singe_hip_set_decode_workers(48)
                lib.singe_hip_set_relaxed_numerics(1 - relaxed)
            barrier.wait(timeout=10)
            parameters = _native.AttentionParametersC()
            for _ in range(200):
                lib.singe_hip_attention_parameters(ctypes.byref(parameters))
                seen[name] = (int(lib.singe_hip_decode_workers(ctypes.byref(c))), config.workspace_bytes(),
                              int(lib.singe_hip_relaxed_numerics()), int(parameters.split_below_blocks))
                assert seen[name][0] == workers and seen[name][2] == relaxed and seen[name][3] == below
            barrier.wait(timeout=10)
            assert lib.singe_hip_set_thread_options(None) == 0
            cleared = _native.ThreadOptionsC()
            lib.singe_hip_thread_options(ctypes.byref(cleared))
            assert (cleared.relaxed_numerics, cleared.decode_workers, cleared.has_split_below_blocks) == (-1, 0, 0)
            assert int(lib.singe_hip_decode_workers(ctypes.byref(c))) == 48  # back on the process-wide value
        except Exception as problem:  # noqa: BLE001 - reported by the test's own thread
            failures.append((name, repr(problem)))
            barrier.abort()

    try:
        threads = [threading.Thread(target=body, args=("a", 64, 1, 7)), threading.Thread(target=body, args=("b", 512, 0, 300))]
        for thread in threads:
            thread.start()
        for thread in threads:
            thread.join(timeout=30)
        assert not failures, failures
        assert seen["a"][1] < seen["b"][1]  # more key ranges, more partial rows
        bad = _native.ThreadOptionsC(2, 0, 0, 0, 0, 0)
        assert lib.singe_hip_set_thread_options(ctypes.byref(bad)) == 9
        bad = _native.ThreadOptionsC(-1, 0, 65, 0, 0, 0)
        assert lib.singe_hip_set_thread_options(ctypes.byref(bad)) == 9
    finally:
        lib.singe_hip_set_decode_workers(0)
        lib.singe_hip_set_relaxed_numerics(0)
        lib.singe_hip_set_thread_options(None)
    assert int(lib.singe_hip_decode_workers(ctypes.byref(c))) == default_workers and config.workspace_bytes() == default_bytes


def test_dense_family_validation_order_needs_no_device():
    """The rest of the dense family checks config and lengths in the order of the reference's validate_lengths, before
    any pointer is read: statuses and the names they carry, on fake pointers."""
    lib = _native.lib()
    fake = 0x1000
    detail = _native.ErrorDetail()

    def named(status):
        lib.singe_hip_last_error(ctypes.byref(detail))
        return status, (detail.name or b"").decode()

    prefill = A.FmhaPrefillConfig.contiguous(2, 8, 8, 4, 2, 64, 0.1, True)
    full = 2 * 8 * 4 * 64
    sink = _native.AttentionSinkPrefillConfigC(prefill._c(), 3, 2)
    call = lambda lengths, config=sink: named(lib.singe_hip_attention_sink_prefill_f32(
        None, fake, lengths[0], fake, lengths[1], fake, lengths[2], fake, lengths[3], fake, lengths[4], ctypes.byref(config)))
    kv = 2 * 8 * 2 * 64
    assert call([full, full - 1, kv, kv, 4]) == (2, "query")          # query, key, value, out, then sinks (mod.rs:1843-1858)
    assert call([full - 1, full, kv - 1, kv, 4]) == (2, "key")
    assert call([full - 1, full, kv, kv, 4]) == (2, "out")
    assert call([full, full, kv, kv, 3]) == (2, "sinks")
    assert call([full, full, kv, kv, 4], _native.AttentionSinkPrefillConfigC(prefill._c(), 1 << 31, 2)) == (3, "start_q")
    assert named(lib.singe_hip_attention_sink_prefill_f32(None, fake, full, fake, full, fake, kv, fake, kv, None, 4, ctypes.byref(sink))) == (6, "sinks")

    decode = A.FmhaDecodeConfig.contiguous(2, 9, 4, 2, 64, 0.1)
    capped = _native.SoftcappedWindowDecodeConfigC(decode._c(), 4, 1, 0.0)   # a cap of zero is invalid
    rows, keys = 2 * 4 * 64, 2 * 9 * 2 * 64
    windowed = lambda config, lse_len=8: named(lib.singe_hip_softcapped_window_decode_lse_bf16(
        None, fake, rows, fake, lse_len, fake, rows, fake, keys, fake, keys, ctypes.byref(config)))
    assert windowed(capped) == (1, "soft_cap")
    assert windowed(_native.SoftcappedWindowDecodeConfigC(decode._c(), 1 << 31, 0, 0.0)) == (3, "window_size")
    assert windowed(_native.SoftcappedWindowDecodeConfigC(decode._c(), 4, 1, 2.0), lse_len=7) == (2, "lse")
    assert named(lib.singe_hip_fmha_decode_lse_f16(None, fake, rows, fake, 8, fake, rows, fake, keys - 1, fake, keys,
                                                   ctypes.byref(decode._c()))) == (2, "key")

    ragged = A.RaggedKvPrefillAttentionConfig.contiguous(3, 10, 12, 4, 2, 32, True, 0.2)._c()
    lengths = [10 * 4 * 32, 40, 10 * 4 * 32, 12 * 2 * 32, 12 * 2 * 32, 3, 3, 3]
    names = ["out", "lse", "query", "key", "value", "actual_seq_lens_q", "actual_seq_lens_kv", "actual_seq_offsets"]
    for position in reversed(range(8)):   # with every later length good, the first short one is the one reported
        short = list(lengths)
        for earlier in range(position, 8):
            short[earlier] = lengths[earlier] - (1 if earlier == position else 0)
        arguments = []
        for length in short:
            arguments += [fake, length]
        assert named(lib.singe_hip_ragged_kv_prefill_attention_f32(None, *arguments, ctypes.byref(ragged))) == (2, names[position])
    with pytest.raises(error.InvalidLength):
        A.RaggedKvPrefillAttentionConfig.contiguous(3, 10, 12, 4, 3, 32, True, 0.2)   # kv heads must divide heads

    sliding = A.SlidingWindowAttentionConfig.contiguous(2, 5, 13, 4, 2, 16, 8, 0, 4, 0.3)
    paged = _native.PagedKvAttentionConfigC(sliding._c(), 4, 11, 4, 4 * 2 * 16, 4 * 2 * 16)
    cache = 11 * 4 * 2 * 16
    through = lambda table_len, cache_len=cache, config=paged: named(lib.singe_hip_sliding_window_attention_paged_kv_f32(
        None, fake, 2 * 5 * 4 * 16, fake, 2 * 5 * 4 * 16, fake, cache_len, fake, cache, fake, table_len, ctypes.byref(config)))
    assert through(7) == (2, "block_table")       # (batch - 1) * stride + ceil(13 / 4) = 8 entries (mod.rs:2893-2900)
    assert through(8, cache - 1) == (2, "key_cache")
    assert through(8, cache, _native.PagedKvAttentionConfigC(sliding._c(), 0, 11, 4, 128, 128))[0] == 1
    packed = _native.PackedQkvAttentionConfigC(sliding._c(), 0, 10, 1 << 40)
    assert named(lib.singe_hip_sliding_window_attention_packed_qkv_f32(None, fake, 640, fake, 5000, ctypes.byref(packed))) == (2, "qkv")
