"""The steps either side of paged attention on the GPU against the CPU oracle, through the C ABI: the fused
rotate-and-append kernel and the CSR -> block-table paging conversion.  Integer outputs and copied values
bit for bit; rotated f32 values within 1e-5, bf16 / f16 within one unit in the last place of the output."""
import numpy as np
import pytest
import torch

import oracle
from singe_amd import error, neural
from singe_amd.kernel import attention as A

pytestmark = pytest.mark.gpu


def host(tensor):
    return tensor.float().cpu().numpy()


def rotary_case(dtype, table_dtype, index_dtype, tokens, heads, groups, dim, pages, slots, seed, norms=False, with_query=True):
    gen = torch.Generator(device="cuda")
    gen.manual_seed(seed)
    rand = lambda *shape: torch.randn(shape, generator=gen, device="cuda").to(dtype)
    q = rand(tokens, heads, dim) if with_query else None
    k, v = rand(tokens, groups, dim), rand(tokens, groups, dim)
    kc, vc = rand(pages, slots, groups, dim), rand(pages, slots, groups, dim)
    angle = torch.rand((tokens, 1, dim // 2), generator=gen, device="cuda") * 6.28
    cos, sin = torch.cos(angle).to(table_dtype), torch.sin(angle).to(table_dtype)
    rng = np.random.default_rng(seed)
    cells = rng.permutation(pages * slots)[:tokens]
    page_index, slot_index = cells // slots, cells % slots
    page_index[0] -= pages  # a negative index counts from the end
    slot_index[-1] -= slots
    query_norm = neural.RotationNorm(1e-6, rand(dim)) if norms else None
    key_norm = neural.RotationNorm(1e-5, None) if norms else None
    want_status, want_q, want_kc, want_vc = oracle.rotary_cache_write_f32(
        None if q is None else host(q), host(k), host(v), host(cos).reshape(tokens, -1), host(sin).reshape(tokens, -1), page_index,
        slot_index, host(kc), host(vc), query_norm=None if not norms else (1e-6, host(query_norm.weight)),
        key_norm=None if not norms else (1e-5, None))
    index = lambda values: torch.tensor(values, dtype=index_dtype, device="cuda")
    q_out = neural.rotary_cache_write(q, k, v, cos, sin, index(page_index), index(slot_index), kc, vc, query_norm=query_norm,
                                      key_norm=key_norm)
    torch.cuda.synchronize()
    assert want_status == 0
    ulp = {torch.float32: 2e-5, torch.bfloat16: 2 ** -7, torch.float16: 2 ** -10}[dtype]
    scale = lambda want: ulp * np.maximum(np.abs(want), 1.0)
    if q is not None:
        assert (np.abs(host(q_out) - want_q) <= scale(want_q)).all()
    else:
        assert q_out is None
    assert (np.abs(host(kc) - want_kc) <= scale(want_kc)).all()
    assert np.array_equal(host(vc), want_vc)  # copied values and untouched cells, bit for bit


@pytest.mark.parametrize("dtype,table_dtype", [(torch.float32, torch.float32), (torch.bfloat16, torch.float32),
                                               (torch.bfloat16, torch.bfloat16), (torch.float16, torch.float16)])
@pytest.mark.parametrize("index_dtype", [torch.int32, torch.int64])
def test_rotary_cache_write(dtype, table_dtype, index_dtype):
    rotary_case(dtype, table_dtype, index_dtype, tokens=37, heads=8, groups=2, dim=128, pages=9, slots=16, seed=1)
    rotary_case(dtype, table_dtype, index_dtype, tokens=5, heads=3, groups=3, dim=80, pages=4, slots=7, seed=2, norms=True)
    rotary_case(dtype, table_dtype, index_dtype, tokens=64, heads=4, groups=1, dim=64, pages=8, slots=16, seed=3, with_query=False)


@pytest.mark.parametrize("dtype,table_dtype", [(torch.float32, torch.bfloat16), (torch.bfloat16, torch.float32), (torch.float16, torch.float16)])
def test_rotary_cache_write_sixteen_bytes_at_a_time_and_element_by_element(dtype, table_dtype):
    """Head dimensions that are a whole number of 16-byte chunk pairs move a chunk of each half per lane (head_dim 96
    and 80 leave lanes of a head's group idle, 256 and 512 take 16 to 64 lanes a head); 24, 40 and 6 (bf16 / f16; 6 and
    20 in f32) are not, and go element by element, as do operands off a 16-byte boundary."""
    for seed, dim in enumerate([96, 256, 512, 32, 16, 24, 40, 6, 20]):
        rotary_case(dtype, table_dtype, torch.int32, tokens=19, heads=5, groups=2, dim=dim, pages=5, slots=4, seed=20 + seed, norms=seed % 2 == 0)
    rotary_case(dtype, table_dtype, torch.int32, tokens=700, heads=16, groups=4, dim=128, pages=50, slots=16, seed=31, norms=True)


def test_rotary_cache_write_off_a_sixteen_byte_boundary():
    gen = torch.Generator(device="cuda")
    gen.manual_seed(5)
    tokens, heads, groups, dim, pages, slots = 9, 4, 2, 64, 3, 4
    rand = lambda *shape: torch.randn(shape, generator=gen, device="cuda").to(torch.bfloat16)
    q, k, v = rand(tokens, heads, dim), rand(tokens, groups, dim), rand(tokens, groups, dim)
    angle = torch.rand((tokens * (dim // 2) + 1,), generator=gen, device="cuda") * 6.28
    cells = np.random.default_rng(5).permutation(pages * slots)[:tokens]
    index = lambda values: torch.tensor(values, dtype=torch.int32, device="cuda")
    results = []
    for shift in (0, 1):  # the same angles on and off the boundary
        table = lambda values: torch.cat([values.new_zeros(shift), values[:tokens * (dim // 2)]])[shift:].view(tokens, 1, dim // 2)
        cos, sin = table(torch.cos(angle)), table(torch.sin(angle))
        assert cos.data_ptr() % 16 == 4 * shift
        kc, vc = torch.zeros((pages, slots, groups, dim), dtype=torch.bfloat16, device="cuda"), torch.zeros((pages, slots, groups, dim), dtype=torch.bfloat16, device="cuda")
        out = neural.rotary_cache_write(q, k, v, cos, sin, index(cells // slots), index(cells % slots), kc, vc,
                                        key_norm=neural.RotationNorm(1e-5, None))
        results.append((out, kc, vc))
    torch.cuda.synchronize()
    for aligned, shifted in zip(*results):
        assert (aligned.float() - shifted.float()).abs().max().item() <= 2 ** -6  # one unit in the last place of values below 4
    assert torch.equal(results[0][2], results[1][2])


def test_rotary_cache_write_decode_step_shape():
    """One decode step of the headline shape: 32 tokens, 32 query / 8 KV heads, head_dim 128, block 16."""
    rotary_case(torch.bfloat16, torch.float32, torch.int32, tokens=32, heads=32, groups=8, dim=128, pages=64, slots=16, seed=9,
                norms=True)


def test_rotary_cache_write_reports_a_bad_cell():
    gen = torch.Generator(device="cuda")
    gen.manual_seed(4)
    rand = lambda *shape: torch.randn(shape, generator=gen, device="cuda")
    k, v, kc, vc = rand(3, 2, 16), rand(3, 2, 16), rand(2, 4, 2, 16), rand(2, 4, 2, 16)
    before = kc.clone()
    cos, sin = torch.ones(3, 1, 8, device="cuda"), torch.zeros(3, 1, 8, device="cuda")
    pages = torch.tensor([0, 2, 1], dtype=torch.int64, device="cuda")  # page 2 of 2
    slots = torch.tensor([0, 1, 3], dtype=torch.int64, device="cuda")
    with pytest.raises(error.IndexOutOfBounds):
        neural.rotary_cache_write(None, k, v, cos, sin, pages, slots, kc, vc)
    assert torch.equal(kc[0, 0], k[0]) and torch.equal(kc[1, 3], k[2])  # the good tokens landed
    untouched = torch.ones(2, 4, dtype=torch.bool, device="cuda")
    untouched[0, 0] = untouched[1, 3] = False
    assert torch.equal(kc[untouched], before[untouched])


def test_rotated_keys_feed_paged_decode():
    """Append a step's keys and values with the fused kernel, then decode over the cache: the result equals
    decode over a cache written on the host."""
    batch, heads, groups, dim, block, blocks = 4, 8, 2, 128, 16, 32
    gen = torch.Generator(device="cuda")
    gen.manual_seed(6)
    rand = lambda *shape: torch.randn(shape, generator=gen, device="cuda").to(torch.bfloat16)
    kc, vc = rand(blocks, block, groups, dim), rand(blocks, block, groups, dim)
    lens = np.array([17, 33, 1, 64], dtype=np.int32)  # lengths including the appended token
    table = np.random.default_rng(6).permutation(blocks)[:batch * 4].reshape(batch, 4).astype(np.uint32)
    q, k, v = rand(batch, heads, dim), rand(batch, groups, dim), rand(batch, groups, dim)
    angle = torch.rand((batch, 1, dim // 2), generator=gen, device="cuda") * 6.28
    cos, sin = torch.cos(angle), torch.sin(angle)
    last = lens - 1
    pages = table[np.arange(batch), last // block].astype(np.int32)
    slots = (last % block).astype(np.int32)
    _, want_q, want_kc, want_vc = oracle.rotary_cache_write_f32(host(q), host(k), host(v), host(cos).reshape(batch, -1),
                                                              host(sin).reshape(batch, -1), pages, slots, host(kc), host(vc))
    q_out = neural.rotary_cache_write(q, k, v, cos, sin, torch.from_numpy(pages).cuda(), torch.from_numpy(slots).cuda(), kc, vc)
    config = A.PagedKvDecodeAttentionConfig.contiguous(batch, heads, groups, dim, block, blocks, 4, dim ** -0.5)
    out = torch.empty((batch, heads, dim), device="cuda", dtype=torch.bfloat16)
    A.paged_kv_decode_attention_bf16(None, out, q_out, kc, vc, torch.from_numpy(lens).cuda(), torch.from_numpy(table.view(np.int32)).cuda(), config)
    torch.cuda.synchronize()
    round_bf16 = lambda a: torch.from_numpy(a).to(torch.bfloat16).float().numpy()
    want = oracle.paged_kv_decode_attention_f32(round_bf16(want_q), round_bf16(want_kc), round_bf16(want_vc), lens, table, batch=batch,
                                                heads=heads, kv_heads=groups, head_dim=dim, block_size=block,
                                                block_table_batch_stride=4, scale=dim ** -0.5, threads=8)
    gap = np.abs(host(out) - want)
    assert gap.max() <= 2e-2 and gap.mean() <= 2e-3


# ---- CSR -> block table -----------------------------------------------------------------------------------

def paging_case(query_offsets, page_offsets, pages, last, index_dtype, **problem):
    index = lambda values: torch.tensor(values, dtype=index_dtype, device="cuda")
    paging = neural.Paging(index(query_offsets), index(page_offsets), index(pages), index(last))
    status = torch.zeros(1, dtype=torch.int32, device="cuda")
    got = neural.paging_indices(paging, status=status, check=False, **problem)
    want = oracle.paging_indices(query_offsets, page_offsets, pages, last, **problem)
    assert int(status.item()) == want[0]
    for have, expected in zip(got, want[1:]):
        assert np.array_equal(have.cpu().numpy(), expected)
    return want[0]


@pytest.mark.parametrize("index_dtype", [torch.int32, torch.int64])
def test_paging_indices_bit_exact(index_dtype):
    assert paging_case([0, 1, 6, 9], [0, 3, 5, 5], [4, 0, 6, 2, 5], [2, 3, 0], index_dtype, tokens=9, page_size=4, cache_pages=7,
                       width=4, row_elements=32) == 0
    rng = np.random.default_rng(8)
    for page_size in (1, 16, 7):
        lengths = [(int(rng.integers(0, 40)), int(rng.integers(0, 300))) for _ in range(23)]
        qo, po, last = [0], [0], []
        for queries, keys in lengths:
            qo.append(qo[-1] + queries)
            n = -(-keys // page_size)
            po.append(po[-1] + n)
            last.append(0 if keys == 0 else keys - (n - 1) * page_size)
        pages = rng.permutation(po[-1] + 5)[:po[-1]].tolist()
        width = max(max(b - a for a, b in zip(po, po[1:])), 1)
        assert paging_case(qo, po, pages, last, index_dtype, tokens=qo[-1], page_size=page_size, cache_pages=po[-1] + 5, width=width,
                           row_elements=8 * 128) == 0


VALID = dict(query_offsets=[0, 1, 3], page_offsets=[0, 2, 3], pages=[1, 0, 2], last=[2, 1])
INVALID = [dict(pages=[1, 0, 3]), dict(pages=[1, -1, 2]), dict(last=[2, 5]), dict(last=[-1, 1]), dict(query_offsets=[0, 2, 1]),
           dict(query_offsets=[0, 1, 4]), dict(page_offsets=[0, 2, 4]), dict(page_offsets=[0, 3, 2]), dict(query_offsets=[-1, 1, 3])]


@pytest.mark.parametrize("change", INVALID)
def test_paging_indices_refuses_what_attention_refuses(change):
    """The tuples of singe/tests/nn/paged_attention.rs:24-73: reported, and everything written stays in range."""
    values = dict(VALID, **change)
    assert paging_case(values["query_offsets"], values["page_offsets"], values["pages"], values["last"], torch.int64, tokens=3,
                       page_size=4, cache_pages=3, width=2, row_elements=4) == 1


def test_csr_paging_bridges_to_the_block_table_kernels():
    """Paged attention in FlashInfer form equals paged_kv_prefill over the converted table when the queries
    are a sequence's first tokens (both alignments agree when queries == keys)."""
    sequences, page_size, heads, groups, dim = [(40, 40), (17, 17), (64, 64)], 16, 4, 2, 128
    qo, po, last = [0], [0], []
    for queries, keys in sequences:
        qo.append(qo[-1] + queries)
        n = -(-keys // page_size)
        po.append(po[-1] + n)
        last.append(keys - (n - 1) * page_size)
    cache_pages = po[-1] + 3
    pages = np.random.default_rng(2).permutation(cache_pages)[:po[-1]].tolist()
    gen = torch.Generator(device="cuda")
    gen.manual_seed(12)
    rand = lambda *shape: torch.randn(shape, generator=gen, device="cuda").to(torch.bfloat16)
    q, kc, vc = rand(qo[-1], heads, dim), rand(cache_pages, page_size, groups, dim), rand(cache_pages, page_size, groups, dim)
    index = lambda values: torch.tensor(values, dtype=torch.int32, device="cuda")
    paging = neural.Paging(index(qo), index(po), index(pages), index(last))
    out_csr, lse_csr = neural.paged_attention(q, kc, vc, paging, neural.AttentionOptions(causal=True))
    width = 4
    packed, query_lengths, key_lengths, table = neural.paging_indices(paging, tokens=qo[-1], page_size=page_size,
                                                                      cache_pages=cache_pages, width=width, row_elements=1)
    config = A.PagedKvPrefillAttentionConfig.contiguous(len(sequences), qo[-1], heads, groups, dim, page_size, cache_pages, width, True,
                                                        dim ** -0.5)
    out_table = torch.empty_like(q)
    lse_table = torch.empty((qo[-1], heads), device="cuda")
    A.paged_kv_prefill_attention_bf16(None, out_table, lse_table, q, kc, vc, query_lengths, key_lengths, packed[:-1].contiguous(), table,
                                      config)
    torch.cuda.synchronize()
    assert torch.equal(out_csr.view(torch.int16), out_table.view(torch.int16))
    assert (lse_csr * 0.6931471805599453 - lse_table).abs().max().item() <= 1e-4
