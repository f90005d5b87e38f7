"""The chunked paged prefill and the fp8-KV decode at their full benchmark sizes, where the CPU oracle would
take hours: each is checked against a different kernel of this library through a fact that holds at any
size.  (The small-size parity of every kernel involved is in the other GPU tests.)"""
import numpy as np
import pytest
import torch

from singe_amd import neural, synthetic
from singe_amd.kernel import attention as A

pytestmark = pytest.mark.gpu


def test_chunked_prefill_full_size_is_the_merge_of_its_prefix_and_its_chunk():
    """8 sequences append 512 tokens to prefixes of U[1024, 16384] keys, 64 query / 8 kv heads, page 16.
    Softmax over prefix + chunk keys is the LSE-weighted mean of softmax over the prefix (no mask, the paged
    kernel again on a shorter page list) and causal softmax over the chunk's own keys (the dense prefill
    kernel on the gathered keys)."""
    work = synthetic.chunked_prefill_workload()
    index = lambda values: torch.tensor(np.asarray(values), dtype=torch.int32, device="cuda")
    whole = neural.Paging(index(work.query_offsets), index(work.page_offsets), index(work.pages), index(work.last_page_lengths))
    out, lse = neural.paged_attention(work.query, work.key_cache, work.value_cache, whole, neural.AttentionOptions(causal=True))
    # The same launch again gives the same bits (the kernel reads its K operands a block ahead across LDS stage
    # hand-overs; a race there would show as a difference between runs).
    for _ in range(3):
        again, lse_again = neural.paged_attention(work.query, work.key_cache, work.value_cache, whole, neural.AttentionOptions(causal=True))
        assert torch.equal(again.view(torch.int16), out.view(torch.int16)) and torch.equal(lse_again, lse)

    size, new = work.page_size, work.new_tokens
    counts = (work.prefix + size - 1) // size
    prefix_pages = np.concatenate([work.pages[work.page_offsets[s]:work.page_offsets[s] + counts[s]] for s in range(work.sequences)])
    prefix_offsets = np.concatenate([[0], np.cumsum(counts)])
    before = neural.Paging(index(work.query_offsets), index(prefix_offsets), index(prefix_pages), index(work.prefix - (counts - 1) * size))
    out_before, lse_before = neural.paged_attention(work.query, work.key_cache, work.value_cache, before, neural.AttentionOptions())

    pages = torch.from_numpy(work.pages).cuda()
    gathered_keys, gathered_values = [], []
    for s in range(work.sequences):
        position = torch.arange(int(work.prefix[s]), int(work.prefix[s]) + new, device="cuda")
        page = pages[int(work.page_offsets[s]) + position // size]
        gathered_keys.append(work.key_cache[page, position % size])
        gathered_values.append(work.value_cache[page, position % size])
    keys, values = torch.stack(gathered_keys), torch.stack(gathered_values)          # [S, new, G, D]
    query = work.query.view(work.sequences, new, work.heads, work.head_dim)
    config = A.FmhaPrefillConfig.contiguous(work.sequences, new, new, work.heads, work.kv_heads, work.head_dim,
                                            float(1.0 / np.sqrt(np.float32(work.head_dim))), True)
    out_chunk = torch.empty_like(query)
    lse_chunk = torch.empty((work.sequences, work.heads, new), device="cuda", dtype=torch.float32)
    A.fmha_prefill_lse_bf16(None, out_chunk, lse_chunk, query, keys, values, config)
    torch.cuda.synchronize()

    lse_chunk = (lse_chunk * float(np.log2(np.e))).permute(0, 2, 1).reshape(-1, work.heads)  # natural log -> base two, [T, H]
    top = torch.maximum(lse_before, lse_chunk)
    weight_before, weight_chunk = torch.exp2(lse_before - top), torch.exp2(lse_chunk - top)
    total = weight_before + weight_chunk
    want = (weight_before[..., None] * out_before.float() + weight_chunk[..., None] * out_chunk.view_as(out).float()) / total[..., None]
    want_lse = top + torch.log2(total)
    gap = (out.float() - want).abs()
    assert torch.isfinite(out.float()).all()
    assert gap.max().item() <= 2e-3 and gap.mean().item() <= 1e-4, (gap.max().item(), gap.mean().item())
    assert (lse - want_lse).abs().max().item() <= 2e-3


def test_fp8_decode_full_size_matches_the_bf16_kernel_on_the_widened_cache():
    """Batch 64 at context 32768, 64 query / 8 kv heads, 131072 blocks of fp8 codes with per-block scales:
    the fp8 kernel's exact mode reads bf16_rne(value(code) * scale), so the bf16 decode kernel, another inner
    loop altogether, run on a cache widened that way by torch must agree up to summation order."""
    work = synthetic.paged_decode_fp8_workload()
    config = A.PagedKvDecodeAttentionConfig.contiguous(work.batch, work.heads, work.kv_heads, work.head_dim, work.block_size,
                                                       work.physical_blocks, work.block_table_batch_stride, work.scale)
    lens = torch.from_numpy(work.seq_lens).cuda()
    table = torch.from_numpy(work.block_table.view(np.int32)).cuda()
    got = torch.full((work.batch, work.heads, work.head_dim), float("nan"), device="cuda", dtype=torch.bfloat16)
    A.paged_kv_decode_attention_f8e4m3kv_bf16(None, got, work.query, work.key_cache, work.value_cache, work.key_scales,
                                              work.value_scales, lens, table, config)

    def widened(codes, scales, chunk=8192):
        wide = torch.empty(codes.shape, device="cuda", dtype=torch.bfloat16)
        for first in range(0, codes.shape[0], chunk):
            part = codes[first:first + chunk].view(torch.float8_e4m3fn).float() * scales[first:first + chunk, None, :, None]
            wide[first:first + chunk] = part.to(torch.bfloat16)
        return wide

    keys, values = widened(work.key_cache, work.key_scales), widened(work.value_cache, work.value_scales)
    want = torch.full_like(got, float("nan"))
    A.paged_kv_decode_attention_bf16(None, want, work.query, keys, values, lens, table, config)
    torch.cuda.synchronize()
    gap = (got.float() - want.float()).abs()
    assert torch.isfinite(got.float()).all()
    peak = want.float().abs().max().item()
    assert gap.max().item() <= 2 ** -7 * peak and gap.mean().item() <= 2 ** -10 * peak, (gap.max().item(), gap.mean().item(), peak)
