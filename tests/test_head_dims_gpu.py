"""Head dimensions other than 128 on the bf16 / f16 surfaces, against the CPU oracle through the C ABI.

The reference's own kernels take head_dim 4 to 64 for block-table decode
(singe-kernel/src/cuda/cutile/attention/paged.rs:799-810), 16 / 32 / 64 / 128 for the dense prefill's matrix path
(singe-kernel/src/cuda/attention/fmha.rs:752-755) and every multiple of 16 up to 128 for the tensor-core paged and dense
kernels (singe/src/backend/cuda/kernel_plan/source/paged_attention.rs:586-592); two of the three shapes of its own
paged test are head_dim 64 (kernel_plan/source/tests.rs:830-966).  Here every multiple of 16 up to 128 runs on a build
of the matrix-core dense, paged and decode kernels for that width, the other widths on the
one-wave-per-row kernels.  Tolerances as at head_dim 128: bf16 max-abs
2e-2 / mean-abs 2e-3, log-sum-exp 2e-3."""
import numpy as np
import pytest
import torch

import oracle
import test_fmha_prefill_gpu as dense
import test_paged_attention_gpu as paged
import test_paged_decode_gpu as decode
import test_paged_kv_prefill_gpu as table_prefill
from singe_amd import _native, neural, synthetic
from singe_amd.kernel import attention as A

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("options", paged.OPTIONS)
@pytest.mark.parametrize("heads,kv_heads,dim,page_size", [(8, 2, 64, 1), (4, 4, 64, 7), (8, 1, 64, 16), (64, 8, 64, 16), (6, 3, 64, 48),
                                                          (8, 2, 32, 1), (4, 4, 32, 7), (16, 2, 32, 16), (8, 2, 96, 1), (4, 4, 96, 7),
                                                          (16, 2, 96, 16), (6, 3, 96, 48), (8, 2, 16, 1), (8, 2, 16, 16), (4, 4, 48, 7),
                                                          (16, 2, 48, 16), (8, 2, 80, 16), (6, 3, 80, 5), (8, 2, 112, 16), (4, 1, 112, 3)])
def test_paged_attention_at_the_matrix_core_head_dims_matches_oracle(heads, kv_heads, dim, page_size, options):
    # the reference's recipe: decode, full prefill, chunked prefill, no keys (tests.rs:830-889), plus more queries than keys
    sequences = [(1, 150), (70, 70), (20, 90), (3, 0), (9, 4), (130, 300)]
    paged.run_case(sequences, heads, kv_heads, page_size, options, seed=heads + page_size, dim=dim)


@pytest.mark.parametrize("dim", [16, 32, 48, 80, 96, 112, 256])
@pytest.mark.parametrize("options", [neural.AttentionOptions(causal=True), neural.AttentionOptions(causal=True, window=16, softcap=30.0)])
def test_paged_attention_at_other_head_dims_matches_oracle(dim, options):
    paged.run_case([(1, 150), (70, 70), (20, 90), (3, 0)], 8, 2, 16, options, seed=dim, dim=dim)


@pytest.mark.parametrize("dim", [64, 32, 96, 16, 48, 80, 112])
@pytest.mark.parametrize("splits", [2, 7, 16])
def test_paged_attention_key_splits_at_other_head_dims(splits, dim):
    _native.lib().singe_hip_set_paged_attention_splits(splits)
    try:
        paged.run_case([(1, 1500), (1, 40), (5, 700), (2, 0), (1, 65), (130, 300)], 8, 2, 16, neural.AttentionOptions(causal=True),
                       seed=splits, dim=dim)
        paged.run_case([(1, 333), (3, 64)], 8, 1, 7, neural.AttentionOptions(), index_dtype=torch.int64, seed=splits + 1, dim=dim)
    finally:
        _native.lib().singe_hip_set_paged_attention_splits(0)


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("dim", [16, 32, 48, 64, 80, 96, 112, 72])
@pytest.mark.parametrize("batch,query_len,key_len,heads,kv_heads", [
    (1, 128, 128, 1, 1), (2, 256, 256, 4, 2), (1, 100, 100, 3, 1), (1, 1, 1, 1, 1), (1, 33, 97, 2, 1), (1, 300, 129, 2, 2),
    (1, 640, 1000, 4, 1),
])
def test_dense_prefill_at_the_references_other_head_dims(batch, query_len, key_len, heads, kv_heads, dim, causal):
    q, k, v = dense.make(batch, query_len, key_len, heads, kv_heads, seed=query_len * 7 + key_len + dim, dim=dim)
    got, lse, want, want_lse = dense.run(q, k, v, causal)
    dense.check(got, lse, want, want_lse, f"{batch}x{query_len}x{key_len} h{heads}/{kv_heads} d{dim} causal={causal}")


def test_dense_prefill_f16_at_head_dim_64():
    q, k, v = (t.to(torch.float16) for t in dense.make(2, 300, 300, 4, 2, seed=3, dim=64))
    config = A.FmhaPrefillConfig.contiguous(2, 300, 300, 4, 2, 64, 0.125, True)
    out = torch.full_like(q, float("nan"))
    lse = torch.full((2, 4, 300), float("nan"), device="cuda")
    A.fmha_prefill_lse_f16(None, out, lse, q, k, v, config)
    torch.cuda.synchronize()
    want, want_lse = oracle.fmha_prefill_lse_f32(q.float().cpu().numpy(), k.float().cpu().numpy(), v.float().cpu().numpy(), batch=2,
                                                 query_len=300, key_len=300, heads=4, kv_heads=2, head_dim=64, scale=0.125,
                                                 causal=True, threads=8)
    gap = np.abs(out.float().cpu().numpy() - want)
    assert gap.max() <= 2e-2 / 6 and gap.mean() <= 2e-3 / 6, (gap.max(), gap.mean())
    assert np.abs(lse.cpu().numpy() - want_lse).max() <= 2e-3


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("dim", [16, 32, 48, 64, 80, 96, 112, 40])
@pytest.mark.parametrize("causal", [True, False])
def test_block_table_prefill_at_other_head_dims(dim, causal, dtype):
    table_prefill.run_case([(130, 130), (1, 1), (33, 200), (64, 10)], 8, 2, 16, causal, seed=dim, dtype=dtype, dim=dim)
    table_prefill.run_case([(70, 70), (0, 12), (9, 0), (20, 90)], 4, 2, 7, causal, seed=dim + 1, gap_tokens=2, dtype=dtype, dim=dim)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("dim", [4, 8, 16, 32, 48, 64, 80, 96, 112])
@pytest.mark.parametrize("heads,kv_heads,block_size", [(8, 2, 16), (12, 4, 7), (8, 8, 1), (16, 1, 32)])
def test_block_table_decode_at_the_references_head_dims(dim, heads, kv_heads, block_size, dtype):
    lens = [0, 1, 15, 16, 17, 31, 32, 33, 100, 257, 300, 64]
    blocks = sum((n + block_size - 1) // block_size for n in lens) + 9
    work = synthetic.paged_decode_workload(batch=len(lens), heads=heads, kv_heads=kv_heads, head_dim=dim, block_size=block_size,
                                           physical_blocks=blocks, seq_lens=lens, seed=100 + heads * 31 + kv_heads + dim)
    # (bf16 values of N(0, 1) magnitude are f16 values too, so the same inputs and the same oracle serve both types)
    got, want = decode.run_gpu(work, dtype=dtype), decode.run_oracle(work)
    assert not got[0].any()  # an empty sequence keeps a zero row (cpu/attention.rs:1213-1215)
    decode.assert_close(got, want, f"d{dim} {heads}/{kv_heads} block {block_size}")


@pytest.mark.parametrize("dim", [64, 32, 16, 48, 112])
@pytest.mark.parametrize("workers", [0, 1, 3, 50, 4096])
def test_decode_splits_at_the_narrow_matrix_core_head_dims(workers, dim):
    lens = [200, 1, 333, 0, 97, 160, 31, 512]
    work = synthetic.paged_decode_workload(batch=len(lens), heads=8, kv_heads=2, head_dim=dim, physical_blocks=128, seq_lens=lens, seed=7)
    decode.assert_close(decode.run_gpu(work, workers), decode.run_oracle(work), f"d{dim} split {workers}")


@pytest.mark.parametrize("dim", [64, 32, 16, 80])
def test_decode_at_the_narrow_matrix_core_head_dims_full_size_matches_oracle(dim):
    # the second benchmark configuration at the reference's head dimensions
    work = synthetic.paged_decode_workload(head_dim=dim, fill="used")
    decode.assert_close(decode.run_gpu(work), decode.run_oracle(work), f"batch 32, ctx U[512, 4096], head_dim {dim}")
