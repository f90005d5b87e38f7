"""Paged decode over an fp8 e4m3 KV cache on the GPU against the CPU oracle run on the dequantised
cache (bf16_rne(f8e4m3_value(code) * scale), widened to f32), through the C ABI."""
import numpy as np
import pytest
import torch

import oracle
from singe_amd import synthetic
from singe_amd.kernel import attention as A

pytestmark = pytest.mark.gpu

MAX_ABS, MEAN_ABS = 2e-2, 2e-3


def run_gpu(work, relaxed=False, workers=0):
    A._native.lib().singe_hip_set_decode_workers(workers)
    A.set_relaxed_numerics(relaxed)
    try:
        config = A.PagedKvDecodeAttentionConfig.contiguous(work.batch, work.heads, work.kv_heads, work.head_dim,
                                                           work.block_size, work.physical_blocks,
                                                           work.block_table_batch_stride, work.scale)
        out = torch.full((work.batch, work.heads, work.head_dim), float("nan"), device="cuda", dtype=torch.bfloat16)
        A.paged_kv_decode_attention_f8e4m3kv_bf16(
            None, out, work.query, work.key_cache, work.value_cache, work.key_scales, work.value_scales,
            torch.from_numpy(work.seq_lens).cuda(), torch.from_numpy(work.block_table.view(np.int32)).cuda(), config)
        torch.cuda.synchronize()
    finally:
        A._native.lib().singe_hip_set_decode_workers(0)
        A.set_relaxed_numerics(False)
    return out.float().cpu().numpy()


def run_oracle(work):
    counts = (work.seq_lens.astype(np.int64) + work.block_size - 1) // work.block_size
    used = np.concatenate([work.block_table[b, :n] for b, n in enumerate(counts)] + [np.zeros(0, np.uint32)]).astype(np.int64)
    if len(used) == 0:
        used = np.zeros(1, dtype=np.int64)
    remap = np.zeros(work.physical_blocks, dtype=np.uint32)
    remap[used] = np.arange(len(used), dtype=np.uint32)
    table = np.zeros_like(work.block_table)
    for b, n in enumerate(counts):
        table[b, :n] = remap[work.block_table[b, :n]]
    index = torch.from_numpy(used).cuda()
    kc = oracle.dequantize_f8e4m3_cache(work.key_cache[index].cpu().numpy(), work.key_scales[index].cpu().numpy())
    vc = oracle.dequantize_f8e4m3_cache(work.value_cache[index].cpu().numpy(), work.value_scales[index].cpu().numpy())
    return oracle.paged_kv_decode_attention_f32(
        work.query.float().cpu().numpy(), kc, vc, work.seq_lens, table, batch=work.batch, heads=work.heads,
        kv_heads=work.kv_heads, head_dim=work.head_dim, block_size=work.block_size,
        block_table_batch_stride=work.block_table_batch_stride, scale=work.scale, threads=8)


def assert_close(got, want, label):
    assert np.isfinite(got).all(), f"{label}: non-finite output"
    gap = np.abs(got - want)
    assert gap.max() <= MAX_ABS, f"{label}: max-abs {gap.max()}"
    assert gap.mean() <= MEAN_ABS, f"{label}: mean-abs {gap.mean()}"


@pytest.mark.parametrize("relaxed", [False, True])
@pytest.mark.parametrize("heads,kv_heads,block_size", [(64, 8, 16), (8, 2, 16), (8, 1, 16), (6, 2, 32), (16, 1, 16),
                                                      (8, 2, 7), (8, 1, 1), (24, 2, 16), (40, 2, 16), (13, 1, 7)])
def test_fp8_decode_matches_oracle(heads, kv_heads, block_size, relaxed):
    lens = [0, 1, 15, 16, 17, 33, 100, 257, 900, 64, 31, 2048]
    blocks = sum((l + block_size - 1) // block_size for l in lens) + 5
    work = synthetic.paged_decode_fp8_workload(batch=len(lens), heads=heads, kv_heads=kv_heads, block_size=block_size,
                                               physical_blocks=blocks, seq_lens=lens, seed=50 + heads + block_size)
    got, want = run_gpu(work, relaxed), run_oracle(work)
    assert not got[0].any()
    assert_close(got, want, f"{heads}/{kv_heads} block {block_size} relaxed={relaxed}")


def test_fp8_decode_long_context_slice():
    # Four sequences of the long-context shape (context 32768, 64 query / 8 kv heads), small pool.
    work = synthetic.paged_decode_fp8_workload(batch=4, physical_blocks=4 * 2048 + 8)
    assert_close(run_gpu(work), run_oracle(work), "context 32768")


def test_fp8_codes_decode_to_the_reference_table():
    # One sequence per code: key b of sequence b dominates the softmax and every value element of that
    # key is code b with scale 1, so the output row is the widened code itself, bit for bit
    # (f8e4m3_value: singe-kernel/src/cpu/quantization.rs:265-280; the two NaN codes are left out).
    table = oracle.f8e4m3_table()
    codes = [c for c in range(256) if not np.isnan(table[c])]
    batch, kv_heads, dim, bs = len(codes), 1, 128, 16
    blocks = batch
    lens = np.full(batch, 16, dtype=np.int32)
    work = synthetic.paged_decode_fp8_workload(batch=batch, heads=4, kv_heads=kv_heads, physical_blocks=blocks,
                                               seq_lens=lens, seed=9)
    keys = torch.zeros((blocks, bs, kv_heads, dim), dtype=torch.uint8)
    values = torch.zeros((blocks, bs, kv_heads, dim), dtype=torch.uint8)
    for b, code in enumerate(codes):
        block = int(work.block_table[b, 0])
        keys[block, b % bs] = 0x48  # 8.0 in e4m3: score 8 * 128 * scale far above the zero rows
        values[block, b % bs] = code
    work.key_cache, work.value_cache = keys.cuda(), values.cuda()
    work.key_scales = torch.ones((blocks, kv_heads), device="cuda")
    work.value_scales = torch.ones((blocks, kv_heads), device="cuda")
    work.query = torch.ones((batch, 4, dim), device="cuda", dtype=torch.bfloat16)
    for relaxed in (False, True):
        got = run_gpu(work, relaxed)
        for b, code in enumerate(codes):
            assert np.array_equal(got[b, 0], np.full(dim, table[code], dtype=np.float32)), (hex(code), got[b, 0, :4])
