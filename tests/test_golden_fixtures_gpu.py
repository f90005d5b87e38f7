"""The f32 HIP kernels, through the C ABI, on the library-routine fixtures of tests/golden/sdpa_fixtures.npz: the same
problems the oracle is pinned on (tests/test_golden_fixtures.py), so kernel and oracle are each held to an
implementation neither shares code with.  Tolerance 1e-4 absolute."""
import numpy as np
import pytest
import torch

from singe_amd import neural
from singe_amd.kernel import attention as A
from test_golden_fixtures import LN2, load, page

pytestmark = pytest.mark.gpu
TOLERANCE = 1e-4


def cuda(array, dtype=None):
    tensor = torch.from_numpy(np.ascontiguousarray(array)).cuda()
    return tensor if dtype is None else tensor.to(dtype)


@pytest.mark.parametrize("name,causal", [("anchor_causal", True), ("gqa_full", False), ("gqa_causal_square", True),
                                         ("prefix_top_left", True), ("decode", False)])
def test_dense_prefill_f32(name, causal):
    q, k, v, out, lse, scale, _ = load(name)
    batch, heads, query_len, dim = q.shape
    config = A.FmhaPrefillConfig.contiguous(batch, query_len, k.shape[2], heads, k.shape[1], dim, scale, causal)
    got = torch.empty((batch, query_len, heads, dim), device="cuda")
    got_lse = torch.empty((batch, heads, query_len), device="cuda")
    A.fmha_prefill_lse_f32(None, got, got_lse, cuda(q.transpose(0, 2, 1, 3)), cuda(k.transpose(0, 2, 1, 3)), cuda(v.transpose(0, 2, 1, 3)), config)
    assert np.abs(got.cpu().numpy().transpose(0, 2, 1, 3) - out).max() <= TOLERANCE
    assert np.abs(got_lse.cpu().numpy() - lse).max() <= TOLERANCE


@pytest.mark.parametrize("name,causal", [("anchor_causal", True), ("gqa_full", False), ("masked", False), ("decode", False)])
def test_dense_op_f32(name, causal):
    q, k, v, out, lse, scale, mask = load(name)
    options = neural.AttentionOptions(scale=scale, causal=causal)
    got = neural.attend(cuda(q), cuda(k), cuda(v), mask=None if mask is None else cuda(mask), options=options)
    assert np.abs(got.cpu().numpy() - out).max() <= TOLERANCE


@pytest.mark.parametrize("page_size", [1, 4, 16])
@pytest.mark.parametrize("name,causal", [("chunk_bottom_right", True), ("gqa_causal_square", True), ("gqa_full", False), ("decode", False)])
def test_paged_op_f32(name, causal, page_size):
    q, k, v, out, lse, scale, _ = load(name)
    batch, heads, query_len, dim = q.shape
    kc, vc, pages, page_offsets, last, _ = page(np.random.default_rng(page_size), k, v, page_size)
    rows = q.transpose(0, 2, 1, 3).reshape(batch * query_len, heads, dim)
    paging = neural.Paging(cuda(np.arange(batch + 1) * query_len, torch.int64), cuda(page_offsets, torch.int64), cuda(pages, torch.int64),
                           cuda(last, torch.int64))
    got, got_lse = neural.paged_attention(cuda(rows), cuda(kc), cuda(vc), paging, neural.AttentionOptions(scale=scale, causal=causal))
    assert np.abs(got.cpu().numpy().reshape(batch, query_len, heads, dim).transpose(0, 2, 1, 3) - out).max() <= TOLERANCE
    assert np.abs(got_lse.cpu().numpy().reshape(batch, query_len, heads).transpose(0, 2, 1) * LN2 - lse).max() <= TOLERANCE


@pytest.mark.parametrize("block_size", [1, 5, 16])
def test_block_table_decode_f32(block_size):
    q, k, v, out, lse, scale, _ = load("decode")
    batch, heads, _, dim = q.shape
    kc, vc, pages, _, _, per = page(np.random.default_rng(block_size), k, v, block_size)
    config = A.PagedKvDecodeAttentionConfig(batch, heads, k.shape[1], dim, block_size, kc.shape[0], per, scale)
    got = torch.empty((batch, heads, dim), device="cuda")
    A.paged_kv_decode_attention_f32(None, got, cuda(q[:, :, 0]), cuda(kc), cuda(vc), cuda(np.full(batch, k.shape[2]), torch.int32),
                                    cuda(pages.reshape(batch, per), torch.int32), config)
    assert np.abs(got.cpu().numpy() - out[:, :, 0]).max() <= TOLERANCE


@pytest.mark.parametrize("name,causal", [("prefix_top_left", True), ("anchor_causal", True), ("gqa_full", False)])
def test_block_table_prefill_f32(name, causal):
    q, k, v, out, lse, scale, _ = load(name)
    batch, heads, query_len, dim = q.shape
    kc, vc, pages, _, _, per = page(np.random.default_rng(3), k, v, 4)
    config = A.PagedKvPrefillAttentionConfig(batch, batch * query_len, heads, k.shape[1], dim, 4, kc.shape[0], per, causal, scale)
    got = torch.empty((batch * query_len, heads, dim), device="cuda")
    got_lse = torch.empty((batch * query_len, heads), device="cuda")
    A.paged_kv_prefill_attention_f32(None, got, got_lse, cuda(q.transpose(0, 2, 1, 3).reshape(batch * query_len, heads, dim)), cuda(kc), cuda(vc),
                                     cuda(np.full(batch, query_len), torch.int32), cuda(np.full(batch, k.shape[2]), torch.int32),
                                     cuda(np.arange(batch) * query_len, torch.int32), cuda(pages.reshape(batch, per), torch.int32), config)
    assert np.abs(got.cpu().numpy().reshape(batch, query_len, heads, dim).transpose(0, 2, 1, 3) - out).max() <= TOLERANCE
    assert np.abs(got_lse.cpu().numpy().reshape(batch, query_len, heads).transpose(0, 2, 1) - lse).max() <= TOLERANCE


@pytest.mark.parametrize("max_splits", [1, 4, 64])
def test_split_decode_and_reduce_f32(max_splits):
    q, k, v, out, lse, scale, _ = load("decode")
    batch, heads, _, dim = q.shape
    keys = k.shape[2]
    config = A.FmhaDecodeSplitKReduceConfig.contiguous(batch, keys, heads, k.shape[1], dim, max_splits, scale)
    effective = min(max_splits, keys)
    got = torch.empty((batch, heads, dim), device="cuda")
    A.fmha_decode_splitk_reduce_f32(None, got, torch.empty(batch * heads * effective * dim, device="cuda"),
                                    torch.empty(batch * heads * effective, device="cuda"), cuda(q[:, :, 0]), cuda(k.transpose(0, 2, 1, 3)),
                                    cuda(v.transpose(0, 2, 1, 3)), config)
    assert np.abs(got.cpu().numpy() - out[:, :, 0]).max() <= TOLERANCE
