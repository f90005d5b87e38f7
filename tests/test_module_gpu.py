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


def _decode_through(lib, seed):
    """One small paged decode through `lib`'s C ABI; returns (status, output, oracle's output)."""
    import numpy as np

    import oracle
    from singe_amd import synthetic

    lens = [100, 1, 513, 0, 64, 300]
    work = synthetic.paged_decode_workload(batch=len(lens), heads=32, kv_heads=8, physical_blocks=256, seq_lens=lens, seed=seed)
    config = _native.PagedKvDecodeAttentionConfigC(work.batch, work.heads, work.kv_heads, work.head_dim, work.block_size,
                                                   work.physical_blocks, work.block_table_batch_stride, work.scale)
    out = torch.zeros((work.batch, work.heads, work.head_dim), device="cuda", dtype=torch.bfloat16)
    lengths = torch.from_numpy(work.seq_lens).cuda()
    table = torch.from_numpy(work.block_table.view(np.int32)).cuda()
    scratch = torch.empty(max(int(lib.singe_hip_paged_kv_decode_attention_workspace_bytes(ctypes.byref(config))), 256),
                          device="cuda", dtype=torch.uint8)
    status = lib.singe_hip_paged_kv_decode_attention_bf16(
        int(torch.cuda.current_stream().cuda_stream), out.data_ptr(), out.numel(), work.query.data_ptr(), work.query.numel(),
        work.key_cache.data_ptr(), work.key_cache.numel(), work.value_cache.data_ptr(), work.value_cache.numel(),
        lengths.data_ptr(), lengths.numel(), table.data_ptr(), table.numel(), scratch.data_ptr(), scratch.numel(),
        ctypes.byref(config))
    torch.cuda.synchronize()
    want = oracle.paged_kv_decode_attention_f32(
        work.query.float().cpu().numpy(), work.key_cache.float().cpu().numpy(), work.value_cache.float().cpu().numpy(),
        work.seq_lens, work.block_table, batch=work.batch, heads=work.heads, kv_heads=work.kv_heads, head_dim=work.head_dim,
        block_size=work.block_size, block_table_batch_stride=work.block_table_batch_stride, scale=work.scale, threads=4)
    return status, out.float().cpu().numpy(), want


def _prefill_through(lib, seed):
    """One small causal dense prefill (bf16, head_dim 128) through `lib`'s C ABI; (status, output, oracle's output)."""
    import numpy as np

    import oracle

    batch, seq, heads, dim = 1, 160, 2, 128
    generator = torch.Generator().manual_seed(seed)
    q, k, v = (torch.randn((batch, seq, heads, dim), generator=generator).to(torch.bfloat16).cuda() for _ in range(3))
    out = torch.zeros_like(q)
    strides = [seq * heads * dim] * 4 + [heads * dim] * 4 + [dim] * 4
    config = _native.FmhaPrefillConfigC(batch, seq, seq, heads, heads, dim, *strides, dim ** -0.5, 1)
    status = lib.singe_hip_fmha_prefill_bf16(int(torch.cuda.current_stream().cuda_stream), out.data_ptr(), out.numel(),
                                             q.data_ptr(), q.numel(), k.data_ptr(), k.numel(), v.data_ptr(), v.numel(),
                                             ctypes.byref(config))
    torch.cuda.synchronize()
    want, _ = oracle.fmha_prefill_lse_f32(q.float().cpu().numpy(), k.float().cpu().numpy(), v.float().cpu().numpy(),
                                          batch=batch, query_len=seq, key_len=seq, heads=heads, kv_heads=heads, head_dim=dim,
                                          scale=dim ** -0.5, causal=True, threads=4)
    return status, out.float().cpu().numpy(), np.asarray(want)


def _close(got, want):
    import numpy as np

    gap = np.abs(got - want)
    return bool(np.isfinite(got).all() and gap.max() <= 2e-2 and gap.mean() <= 2e-3)


def test_kernels_handed_over_as_bytes(tmp_path):
    """A copy of the library with no code object beside it: nothing launches until the kernels arrive as bytes, as an
    archive of parts (singe_hip_load), part by part (singe_hip_load_part) or from the archive's file; after an unload
    the copy is back to finding nothing, and the library next to its parts is untouched throughout."""
    import shutil

    from singe_amd import build

    torch.cuda.set_device(0)
    copy = _native.bind(shutil.copy(_native.LIBRARY_PATH, tmp_path / "libsinge_hip_attention.so"))
    status, _, _ = _decode_through(copy, 1)
    assert status == 7, status  # SINGE_HIP_KERNEL_NOT_PREPARED: no part next to the copy
    detail = _native.ErrorDetail()
    copy.singe_hip_last_error(ctypes.byref(detail))
    assert detail.name == b"paged_decode"

    archive = build.pack_archive()
    assert copy.singe_hip_load(archive, len(archive)) == 0
    for run in (_decode_through, _prefill_through):  # two different parts of the archive
        status, got, want = run(copy, 2)
        assert status == 0 and _close(got, want), run.__name__
    found = ctypes.c_int32(0)
    assert copy.singe_hip_prepare(ctypes.byref(found)) == 0 and found.value >= 113

    copy.singe_hip_unload()
    assert _decode_through(copy, 3)[0] == 7
    for part in ("paged_decode", "fmha_prefill"):
        image = open(build.code_object(part), "rb").read()
        assert copy.singe_hip_load_part(part.encode(), image, len(image)) == 0
    for run in (_decode_through, _prefill_through):
        status, got, want = run(copy, 4)
        assert status == 0 and _close(got, want), run.__name__
    assert copy.singe_hip_load_part(b"no_such_part", archive, 16) == 9  # SINGE_HIP_INVALID_ARGUMENT

    copy.singe_hip_unload()
    path = tmp_path / "kernels.parts"
    path.write_bytes(build.pack_archive(parts=("paged_decode",)))
    assert copy.singe_hip_load_file(str(path).encode()) == 0
    status, got, want = _decode_through(copy, 5)
    assert status == 0 and _close(got, want)
    assert _prefill_through(copy, 5)[0] == 7  # that archive holds the decode part only
    copy.singe_hip_unload()

    # the library next to its parts: an archive load, an unload, and the default lookup again
    lib = _native.lib()
    assert lib.singe_hip_load(archive, len(archive)) == 0
    status, got, want = _decode_through(lib, 6)
    assert status == 0 and _close(got, want)
    lib.singe_hip_unload()
    for run in (_decode_through, _prefill_through):
        status, got, want = run(lib, 7)
        assert status == 0 and _close(got, want), run.__name__
