"""The kernels that take any element type and head dimension, on the GPU against the CPU oracle through
the C ABI: dense scaled-dot-product attention with every option of the op (causal, window, softcap,
additive / Boolean mask, sinks, key lengths), the general paged attention, and splitk_reduce_f32.
Tolerances: f32 max-abs 1e-4; bf16 max-abs 2e-2 and mean-abs 2e-3; f16 max-abs 5e-3 (the reference's own
half tolerances, singe/src/backend/cuda/kernel_plan/source/tests.rs:549-553); base-two LSE 2e-3."""
import numpy as np
import pytest
import torch

import oracle
from singe_amd import error, neural
from singe_amd.kernel import attention as A

pytestmark = pytest.mark.gpu

TOLERANCE = {torch.float32: (1e-4, 1e-5), torch.bfloat16: (2e-2, 2e-3), torch.float16: (5e-3, 5e-4)}


def close(got, want, dtype):
    worst, mean = TOLERANCE[dtype]
    gap = np.abs(got - want)
    assert np.isfinite(got).all()
    assert gap.max(initial=0.0) <= worst, gap.max()
    assert gap.mean() <= mean if gap.size else True, gap.mean()


def tensors(shape_q, shape_k, shape_v, dtype, seed):
    gen = torch.Generator(device="cuda")
    gen.manual_seed(seed)
    return tuple(torch.randn(shape, generator=gen, device="cuda").to(dtype) for shape in (shape_q, shape_k, shape_v))


def host(tensor):
    return tensor.float().cpu().numpy()


# ---- dense ------------------------------------------------------------------------------------------

def test_f32_accuracy_anchor():
    """Dense causal [1, 8, 512, 64] f32 with scale 0.125: within 1e-4 of the CPU path."""
    q, k, v = tensors((1, 8, 512, 64), (1, 8, 512, 64), (1, 8, 512, 64), torch.float32, 1)
    out = neural.scaled_dot_product_attention(q, k, v, 0.125, True)
    want = oracle.scaled_dot_product_attention_f32(host(q), host(k), host(v), scale=0.125, causal=True, threads=8)
    close(host(out), want, torch.float32)


DENSE_SHAPES = [
    # batch, heads, kv_heads, query_len, key_len, head_dim, value_dim
    (2, 4, 2, 37, 53, 64, 64),
    (1, 6, 3, 70, 70, 80, 48),
    (2, 2, 1, 5, 130, 200, 256),
    (1, 3, 3, 129, 64, 16, 8),
]
DENSE_OPTIONS = [
    dict(),
    dict(causal=True),
    dict(causal=True, window=9, softcap=20.0),
    dict(window=33, scale=0.07),
    dict(softcap=3.0),
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", DENSE_SHAPES)
@pytest.mark.parametrize("options", DENSE_OPTIONS)
def test_dense_options(shape, options, dtype):
    batch, heads, kv_heads, query_len, key_len, head_dim, value_dim = shape
    q, k, v = tensors((batch, heads, query_len, head_dim), (batch, kv_heads, key_len, head_dim),
                      (batch, kv_heads, key_len, value_dim), dtype, 7)
    out = neural.attend(q, k, v, options=neural.AttentionOptions(**options))
    assert out.dtype == dtype and out.shape == (batch, heads, query_len, value_dim)
    want = oracle.scaled_dot_product_attention_f32(host(q), host(k), host(v), threads=8, **options)
    close(host(out), want, dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_dense_mask_sinks_and_key_lengths(dtype):
    batch, heads, kv_heads, query_len, key_len, dim = 3, 4, 2, 20, 45, 64
    q, k, v = tensors((batch, heads, query_len, dim), (batch, kv_heads, key_len, dim), (batch, kv_heads, key_len, dim), dtype, 11)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(5)
    # An additive mask broadcast over batch and heads, with some keys hidden outright.
    mask = torch.randn((query_len, key_len), generator=gen, device="cuda").to(dtype)
    mask[:, 3] = float("-inf")
    mask[7, :30] = float("-inf")
    sinks = torch.randn((heads,), generator=gen, device="cuda").to(dtype)
    options = neural.AttentionOptions(causal=False, softcap=10.0)
    out = neural.attend(q, k, v, mask, sinks, options)
    want = oracle.scaled_dot_product_attention_f32(host(q), host(k), host(v), softcap=10.0, mask=host(mask), sinks=host(sinks),
                                                   threads=8)
    close(host(out), want, dtype)
    # A mask over [batch, 1, query, key].
    mask4 = torch.randn((batch, 1, query_len, key_len), generator=gen, device="cuda").to(dtype)
    out = neural.attend(q, k, v, mask4, None, neural.AttentionOptions(causal=True))
    want = oracle.scaled_dot_product_attention_f32(host(q), host(k), host(v), causal=True, mask=host(mask4), threads=8)
    close(host(out), want, dtype)
    # A Boolean mask lets the keys where it holds take part.
    keep = torch.rand((heads, query_len, key_len), generator=gen, device="cuda") > 0.3
    keep[..., 0] = True
    out = neural.attend(q, k, v, keep, sinks)
    additive = np.where(keep.cpu().numpy(), 0.0, -np.inf).astype(np.float32)
    want = oracle.scaled_dot_product_attention_f32(host(q), host(k), host(v), mask=additive, sinks=host(sinks), threads=8)
    close(host(out), want, dtype)
    # Padded batches: a count of zero gives zeros, counts past the keys see them all.
    lengths = torch.tensor([0, 17, 99], dtype=torch.int32, device="cuda")
    out = neural.attend_padded(q, k, v, lengths, neural.AttentionOptions(causal=True))
    want = oracle.scaled_dot_product_attention_f32(host(q), host(k), host(v), causal=True, key_lengths=[0, 17, 99], threads=8)
    close(host(out), want, dtype)
    assert not host(out)[0].any()


def test_dense_bf16_at_128_takes_the_matrix_core_kernel_and_matches():
    q, k, v = tensors((2, 8, 200, 128), (2, 2, 333, 128), (2, 2, 333, 128), torch.bfloat16, 13)
    for causal in (False, True):
        out = neural.scaled_dot_product_attention(q, k, v, None, causal)
        want = oracle.scaled_dot_product_attention_f32(host(q), host(k), host(v), causal=causal, threads=8)
        close(host(out), want, torch.bfloat16)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("causal", [False, True])
def test_dense_at_128_with_sinks_and_key_lengths_on_the_matrix_core_kernel(dtype, causal):
    # Sinks and key lengths stay on the flash kernel at head dimension 128; a mask, a window or a cap do not.
    batch, heads, kv_heads, query_len, key_len = 3, 8, 2, 150, 333
    q, k, v = tensors((batch, heads, query_len, 128), (batch, kv_heads, key_len, 128), (batch, kv_heads, key_len, 128), dtype, 17)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(9)
    sinks = (torch.randn((heads,), generator=gen, device="cuda") * 3).to(dtype)
    sinks[1] = float("-inf")  # a sink that never counts
    sinks[2] = 30.0           # a sink that takes nearly all of every row
    options = neural.AttentionOptions(causal=causal)
    out = neural.attend(q, k, v, None, sinks, options)
    want = oracle.scaled_dot_product_attention_f32(host(q), host(k), host(v), causal=causal, sinks=host(sinks), threads=8)
    close(host(out), want, dtype)
    lengths = torch.tensor([0, 77, 400], dtype=torch.int32, device="cuda")
    out = neural.attend_padded(q, k, v, lengths, options)
    want = oracle.scaled_dot_product_attention_f32(host(q), host(k), host(v), causal=causal, key_lengths=[0, 77, 400], threads=8)
    close(host(out), want, dtype)
    assert not host(out)[0].any()
    # Both at once, through the C ABI's nullable operands.
    import ctypes
    from singe_amd import _native
    problem = _native.AttentionProblemC(batch, heads, kv_heads, query_len, key_len, 128, 128, (ctypes.c_int64 * 4)(0, 0, 0, 0),
                                        {torch.bfloat16: 1, torch.float16: 2}[dtype], int(causal), 0, 0, 0, 0.0, 0.0, 0)
    both = torch.empty_like(q)
    status = _native.lib().singe_hip_scaled_dot_product_attention(None, q.data_ptr(), k.data_ptr(), v.data_ptr(), None, sinks.data_ptr(),
                                                                  lengths.data_ptr(), both.data_ptr(), ctypes.byref(problem))
    assert status == 0
    want = oracle.scaled_dot_product_attention_f32(host(q), host(k), host(v), causal=causal, sinks=host(sinks), key_lengths=[0, 77, 400],
                                                   threads=8)
    close(host(both), want, dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("options", [dict(window=40), dict(causal=True, window=7), dict(softcap=3.0), dict(softcap=-2.0, causal=True),
                                     dict(causal=True, window=100, softcap=5.0, scale=-0.05), dict(window=0)])
def test_dense_at_128_with_window_and_cap_on_the_matrix_core_kernel(dtype, options):
    batch, heads, kv_heads, query_len, key_len = 2, 4, 2, 200, 333
    q, k, v = tensors((batch, heads, query_len, 128), (batch, kv_heads, key_len, 128), (batch, kv_heads, key_len, 128), dtype, 19)
    out = neural.attend(q, k, v, options=neural.AttentionOptions(**options))
    want = oracle.scaled_dot_product_attention_f32(host(q), host(k), host(v), threads=8, **options)
    close(host(out), want, dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("options", [dict(causal=True, window=300), dict(causal=True, window=129, softcap=6.0), dict(window=200),
                                     dict(causal=True, window=64), dict(causal=True, window=1000)])
def test_dense_at_128_long_windows(dtype, options):
    """Rows long enough that a wave meets all three kinds of tile: reaching back past the window, wholly
    inside it, and on the causal edge."""
    batch, heads, kv_heads, query_len, key_len = 1, 4, 2, 900, 900
    q, k, v = tensors((batch, heads, query_len, 128), (batch, kv_heads, key_len, 128), (batch, kv_heads, key_len, 128), dtype, 31)
    out = neural.attend(q, k, v, options=neural.AttentionOptions(**options))
    want = oracle.scaled_dot_product_attention_f32(host(q), host(k), host(v), threads=8, **options)
    close(host(out), want, dtype)


@pytest.mark.parametrize("causal", [False, True])
def test_dense_at_128_cap_alone_with_sinks_and_key_lengths(causal):
    """A cap without mask or window keeps the straight-line tiles of the matrix-core kernel; sinks and
    per-batch key lengths ride along."""
    batch, heads, kv_heads, query_len, key_len = 2, 4, 2, 520, 700
    dtype = torch.bfloat16
    q, k, v = tensors((batch, heads, query_len, 128), (batch, kv_heads, key_len, 128), (batch, kv_heads, key_len, 128), dtype, 29)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(5)
    sinks = torch.randn((heads,), generator=gen, device="cuda").to(dtype)
    lengths = torch.tensor([333, 700], dtype=torch.int32, device="cuda")
    import ctypes
    from singe_amd import _native
    problem = _native.AttentionProblemC(batch, heads, kv_heads, query_len, key_len, 128, 128, (ctypes.c_int64 * 4)(0, 0, 0, 0), 1,
                                        int(causal), 0, 0, 1, 0.0, 4.0, 0)
    out = torch.empty_like(q)
    status = _native.lib().singe_hip_scaled_dot_product_attention(None, q.data_ptr(), k.data_ptr(), v.data_ptr(), None, sinks.data_ptr(),
                                                                  lengths.data_ptr(), out.data_ptr(), ctypes.byref(problem))
    assert status == 0
    want = oracle.scaled_dot_product_attention_f32(host(q), host(k), host(v), causal=causal, softcap=4.0, sinks=host(sinks),
                                                   key_lengths=[333, 700], threads=8)
    close(host(out), want, dtype)


@pytest.mark.parametrize("key_len", [201, 204])  # mask rows off and on an 8-byte boundary (the packed loads)
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_dense_at_128_with_masks_on_the_matrix_core_kernel(dtype, key_len):
    batch, heads, kv_heads, query_len = 2, 4, 2, 150
    q, k, v = tensors((batch, heads, query_len, 128), (batch, kv_heads, key_len, 128), (batch, kv_heads, key_len, 128), dtype, 23)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(3)
    sinks = torch.randn((heads,), generator=gen, device="cuda").to(dtype)
    lengths = torch.tensor([170, 500], dtype=torch.int32, device="cuda")
    # broadcast over batch and heads, with hidden keys and one row hidden but for its last keys
    mask = torch.randn((query_len, key_len), generator=gen, device="cuda").to(dtype)
    mask[:, 3] = float("-inf")
    mask[7, :190] = float("-inf")
    out = neural.attend(q, k, v, mask, sinks, neural.AttentionOptions(softcap=10.0))
    want = oracle.scaled_dot_product_attention_f32(host(q), host(k), host(v), softcap=10.0, mask=host(mask), sinks=host(sinks), threads=8)
    close(host(out), want, dtype)
    # per batch and head, causal and windowed; one row has every key hidden: the CPU form divides zero by zero
    # there (NaN), the kernel writes zeros like every other row without keys
    full = torch.randn((batch, heads, query_len, key_len), generator=gen, device="cuda").to(dtype)
    full[1, 2, 5, :] = float("-inf")
    out = neural.attend(q, k, v, full, None, neural.AttentionOptions(causal=True, window=64))
    want = oracle.scaled_dot_product_attention_f32(host(q), host(k), host(v), causal=True, window=64, mask=host(full), threads=8)
    assert np.isnan(want[1, 2, 5]).all() and not host(out)[1, 2, 5].any()
    want[1, 2, 5] = 0.0
    close(host(out), want, dtype)
    # broadcast over queries ([batch, 1, 1, key]) and a Boolean mask over [heads, query, key]
    padding = torch.zeros((batch, 1, 1, key_len), device="cuda", dtype=dtype)
    padding[0, ..., 120:] = float("-inf")
    out = neural.attend(q, k, v, padding)
    want = oracle.scaled_dot_product_attention_f32(host(q), host(k), host(v), mask=host(padding), threads=8)
    close(host(out), want, dtype)
    keep = torch.rand((heads, query_len, key_len), generator=gen, device="cuda") > 0.3
    keep[..., 0] = True
    out = neural.attend(q, k, v, keep, sinks)
    want = oracle.scaled_dot_product_attention_f32(host(q), host(k), host(v), mask=np.where(keep.cpu().numpy(), 0.0, -np.inf).astype(np.float32),
                                                   sinks=host(sinks), threads=8)
    close(host(out), want, dtype)


def test_dense_shape_rules():
    q, k, v = tensors((1, 4, 8, 32), (1, 3, 8, 32), (1, 3, 8, 32), torch.float32, 1)
    with pytest.raises(error.InvalidArgument):
        neural.scaled_dot_product_attention(q, k, v)
    q, k, v = tensors((1, 4, 8, 32), (1, 2, 8, 32), (1, 2, 9, 32), torch.float32, 1)
    with pytest.raises(error.LengthMismatch):
        neural.scaled_dot_product_attention(q, k, v)
    q, k, v = tensors((1, 2, 8, 320), (1, 2, 8, 320), (1, 2, 8, 320), torch.float32, 1)
    with pytest.raises(error.UnsupportedWidth):
        neural.scaled_dot_product_attention(q, k, v)


# ---- paged --------------------------------------------------------------------------------------------

def paged_layout(sequences, page_size, extra_pages=2):
    query_offsets, page_offsets, last, needed = [0], [0], [], 0
    for queries, keys in sequences:
        query_offsets.append(query_offsets[-1] + queries)
        pages = (keys + page_size - 1) // page_size
        needed += pages
        page_offsets.append(needed)
        last.append(0 if keys == 0 else keys - (pages - 1) * page_size)
    page_count = needed + extra_pages
    table = list(np.random.default_rng(page_count).permutation(page_count)[:needed])
    return query_offsets, page_offsets, [int(p) for p in table], last, page_count


PAGED_OPTIONS = [dict(), dict(causal=True), dict(causal=True, window=12, softcap=25.0), dict(scale=0.2, softcap=4.0)]


@pytest.mark.parametrize("dtype,dim", [(torch.float32, 64), (torch.float32, 128), (torch.float32, 40), (torch.float16, 128),
                                       (torch.float16, 72), (torch.bfloat16, 64), (torch.bfloat16, 256)])
@pytest.mark.parametrize("options", PAGED_OPTIONS)
@pytest.mark.parametrize("index_dtype", [torch.int32, torch.int64])
def test_general_paged(dtype, dim, options, index_dtype):
    sequences, page_size, heads, kv_heads = [(1, 150), (70, 70), (20, 90), (3, 0), (9, 4)], 7, 6, 2
    query_offsets, page_offsets, table, last, page_count = paged_layout(sequences, page_size)
    q, kc, vc = tensors((query_offsets[-1], heads, dim), (page_count, page_size, kv_heads, dim), (page_count, page_size, kv_heads, dim),
                        dtype, 3)
    index = lambda values: torch.tensor(values, dtype=index_dtype, device="cuda")
    paging = neural.Paging(index(query_offsets), index(page_offsets), index(table), index(last))
    out, lse = neural.paged_attention(q, kc, vc, paging, neural.AttentionOptions(**options))
    assert out.dtype == dtype
    status, want, want_lse = oracle.paged_attention_f32(host(q), host(kc), host(vc), query_offsets, page_offsets, table, last,
                                                        threads=8, **options)
    assert status == 0
    close(host(out), want, dtype)
    got_lse = lse.cpu().numpy()
    empty = np.isneginf(want_lse)
    assert np.array_equal(np.isneginf(got_lse), empty)
    assert not host(out)[empty].any()
    assert np.abs(got_lse[~empty] - want_lse[~empty]).max(initial=0.0) <= 2e-3


@pytest.mark.parametrize("dtype,dim,index_dtype", [(torch.float32, 64, torch.int32), (torch.bfloat16, 48, torch.int64)])
def test_general_paged_finds_the_rows_of_many_ragged_sequences(dtype, dim, index_dtype):
    # more sequences than one wave's prefix sum covers (64), some without queries, some without keys
    rng = np.random.default_rng(dim)
    sequences = []
    for s in range(150):
        queries = int(rng.choice([0, 1, 1, 2, 3, 5, 9, 17]))
        sequences.append((queries, 0 if s % 19 == 3 else queries + int(rng.integers(0, 40))))
    heads, kv_heads, page_size = 6, 2, 5
    query_offsets, page_offsets, table, last, page_count = paged_layout(sequences, page_size)
    q, kc, vc = tensors((query_offsets[-1], heads, dim), (page_count, page_size, kv_heads, dim), (page_count, page_size, kv_heads, dim),
                        dtype, 9)
    index = lambda values: torch.tensor(values, dtype=index_dtype, device="cuda")
    paging = neural.Paging(index(query_offsets), index(page_offsets), index(table), index(last))
    out, lse = neural.paged_attention(q, kc, vc, paging, neural.AttentionOptions(causal=True))
    status, want, want_lse = oracle.paged_attention_f32(host(q), host(kc), host(vc), query_offsets, page_offsets, table, last,
                                                        threads=8, causal=True)
    assert status == 0
    close(host(out), want, dtype)
    empty = np.isneginf(want_lse)
    assert np.array_equal(np.isneginf(lse.cpu().numpy()), empty)
    assert np.abs(lse.cpu().numpy()[~empty] - want_lse[~empty]).max(initial=0.0) <= 2e-3


VALID = dict(query_offsets=[0, 1, 3], page_offsets=[0, 2, 3], pages=[1, 0, 2], last=[2, 1])
INVALID = [
    dict(pages=[1, 0, 3]), dict(pages=[1, -1, 2]), dict(last=[2, 5]), dict(last=[-1, 1]), dict(query_offsets=[0, 2, 1]),
    dict(query_offsets=[0, 1, 4]), dict(page_offsets=[0, 2, 4]), dict(page_offsets=[0, 3, 2]), dict(query_offsets=[-1, 1, 3]),
]


@pytest.mark.parametrize("change", INVALID)
def test_general_paged_reports_bad_paging_values(change):
    """The tuples of singe/tests/nn/paged_attention.rs:24-73 over a cache of 3 pages of 4 slots."""
    values = dict(VALID, **change)
    q, kc, vc = tensors((3, 2, 32), (3, 4, 1, 32), (3, 4, 1, 32), torch.float32, 1)
    index = lambda v: torch.tensor(v, dtype=torch.int64, device="cuda")
    paging = neural.Paging(index(values["query_offsets"]), index(values["page_offsets"]), index(values["pages"]), index(values["last"]))
    assert oracle.check_paged_values(values["query_offsets"], values["page_offsets"], values["pages"], values["last"], tokens=3,
                                     cache_pages=3, page_size=4) == 1
    with pytest.raises(error.IndexOutOfBounds):
        neural.paged_attention(q, kc, vc, paging)
    good = neural.Paging(index(VALID["query_offsets"]), index(VALID["page_offsets"]), index(VALID["pages"]), index(VALID["last"]))
    neural.paged_attention(q, kc, vc, good)


# ---- split-KV reduce ------------------------------------------------------------------------------------

@pytest.mark.parametrize("batch,heads,splits,dim", [(2, 3, 5, 64), (1, 8, 1, 128), (3, 2, 64, 40), (1, 1, 7, 300)])
def test_splitk_reduce(batch, heads, splits, dim):
    gen = torch.Generator(device="cuda")
    gen.manual_seed(splits)
    attn = torch.randn((batch, heads, splits, dim), generator=gen, device="cuda")
    lse = torch.randn((batch, heads, splits), generator=gen, device="cuda") * 4
    out = torch.empty((batch, heads, dim), device="cuda")
    A.splitk_reduce_f32(None, out, attn, lse, A.SplitKReduceConfig.contiguous(batch, heads, splits, dim))
    want = oracle.splitk_reduce_f32(host(attn), host(lse), batch=batch, heads=heads, splits=splits, head_dim=dim)
    assert np.abs(host(out) - want).max() <= 1e-5


def test_splitk_reduce_folds_an_actual_split():
    """Partials of disjoint key ranges reduce to the attention over all keys."""
    q, k, v = tensors((1, 4, 1, 64), (1, 4, 96, 64), (1, 4, 96, 64), torch.float32, 2)
    whole = neural.scaled_dot_product_attention(q, k, v)
    parts, lses = [], []
    for first in range(0, 96, 32):
        ks, vs = k[:, :, first:first + 32].contiguous(), v[:, :, first:first + 32].contiguous()
        parts.append(neural.scaled_dot_product_attention(q, ks, vs)[:, :, 0])
        scores = torch.einsum("bhd,bhsd->bhs", q[:, :, 0], ks) * 64 ** -0.5
        lses.append(torch.logsumexp(scores, dim=-1))
    attn = torch.stack(parts, dim=2).contiguous()
    lse = torch.stack(lses, dim=2).contiguous()
    out = torch.empty((1, 4, 64), device="cuda")
    A.splitk_reduce_f32(None, out, attn, lse, A.SplitKReduceConfig.contiguous(1, 4, 3, 64))
    assert (out - whole[:, :, 0]).abs().max().item() <= 1e-5


def test_splitk_reduce_validation():
    out, attn, lse = torch.empty(10, device="cuda"), torch.empty(100, device="cuda"), torch.empty(10, device="cuda")
    with pytest.raises(error.InvalidLength):
        A.splitk_reduce_f32(None, out, attn, lse, A.SplitKReduceConfig.contiguous(1, 0, 5, 8))
    with pytest.raises(error.LengthTooShort) as caught:
        A.splitk_reduce_f32(None, out, attn, lse, A.SplitKReduceConfig.contiguous(1, 2, 5, 8))
    assert caught.value.name == "out" and caught.value.minimum == 16


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("dim", [128, 64])
@pytest.mark.parametrize("causal", [True, False])
def test_padded_batches_on_the_two_tile_kernel(causal, dim, dtype):
    # key counts of their own for every batch entry (none, a few, a last tile that is not whole, all and more than all) on
    # the dense kernel that gives a wave two 32-row tiles
    from singe_amd import _native
    batch, heads, kv_heads, query_len, key_len = 5, 4, 2, 300, 640
    q, k, v = tensors((batch, heads, query_len, dim), (batch, kv_heads, key_len, dim), (batch, kv_heads, key_len, dim), dtype, 23)
    counts = [0, 17, 333, 640, 5000]
    lengths = torch.tensor(counts, dtype=torch.int32, device="cuda")
    _native.lib().singe_hip_set_dense_prefill_rows_per_wave(64)
    try:
        out = neural.attend_padded(q, k, v, lengths, neural.AttentionOptions(causal=causal))
    finally:
        _native.lib().singe_hip_set_dense_prefill_rows_per_wave(0)
    want = oracle.scaled_dot_product_attention_f32(host(q), host(k), host(v), causal=causal, key_lengths=counts, threads=8)
    close(host(out), want, dtype)
    assert not host(out)[0].any()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("dim", [128, 64])
def test_sinks_on_the_two_tile_kernel(dim, dtype):
    # a sink per head (one of them so large that it outweighs every key, one absent: -inf) with and without the causal
    # mask and with padded batches, on the dense kernel that gives a wave two 32-row tiles
    from singe_amd import _native
    batch, heads, kv_heads, query_len, key_len = 3, 4, 2, 300, 450
    q, k, v = tensors((batch, heads, query_len, dim), (batch, kv_heads, key_len, dim), (batch, kv_heads, key_len, dim), dtype, 29)
    sinks = torch.tensor([0.5, 30.0, float("-inf"), -2.0], device="cuda").to(dtype)
    counts = [0, 450, 129]
    lengths = torch.tensor(counts, dtype=torch.int32, device="cuda")
    _native.lib().singe_hip_set_dense_prefill_rows_per_wave(64)
    try:
        for causal in (True, False):
            out = neural.attend(q, k, v, None, sinks, neural.AttentionOptions(causal=causal))
            want = oracle.scaled_dot_product_attention_f32(host(q), host(k), host(v), causal=causal, sinks=host(sinks), threads=8)
            close(host(out), want, dtype)
        out = neural._attend_all(q, k, v, None, sinks, lengths, neural.AttentionOptions(causal=True), None)
        want = oracle.scaled_dot_product_attention_f32(host(q), host(k), host(v), causal=True, sinks=host(sinks), key_lengths=counts, threads=8)
        close(host(out), want, dtype)
    finally:
        _native.lib().singe_hip_set_dense_prefill_rows_per_wave(0)
