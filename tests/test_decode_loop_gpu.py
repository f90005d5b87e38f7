"""A decode loop end to end on the GPU: the page table places each step's tokens (singe/src/nn/decode/step.rs),
the fused kernel rotates and appends them, paged attention reads them back through the step's paging.  Checked
against dense attention over a per-sequence history the test keeps itself, so a wrong page, slot, offset or
length anywhere along the way shows as a wrong output row.  f32 within 1e-4; bf16 within 2e-2 max / 2e-3 mean."""
import numpy as np
import pytest
import torch

import oracle
from singe_amd import neural
from singe_amd.decode import PageTable

pytestmark = pytest.mark.gpu

HEADS, GROUPS, DIM = 8, 2, 128


def rotate(values, positions):
    """Half-split rotary pairs (p, p + D/2) at angle position * 10000^(-2p/D)."""
    half = values.shape[-1] // 2
    angle = positions[:, None].astype(np.float64) * (10000.0 ** (-np.arange(half) / half))[None, :]
    cos, sin = np.cos(angle)[:, None, :], np.sin(angle)[:, None, :]
    low, high = values[..., :half].astype(np.float64), values[..., half:].astype(np.float64)
    return np.concatenate([low * cos - high * sin, high * cos + low * sin], axis=-1).astype(np.float32), \
        np.cos(angle).astype(np.float32), np.sin(angle).astype(np.float32)


def run_loop(dtype, schedule, table, max_error, mean_error, seed):
    rng = np.random.default_rng(seed)
    device = "cuda"
    pages, size = table.page_count(), table.page_size()
    # The caches start as noise: lengths, not zeros, hide what a sequence has not written.
    key_cache = torch.tensor(rng.standard_normal((pages, size, GROUPS, DIM)), dtype=dtype, device=device)
    value_cache = torch.tensor(rng.standard_normal((pages, size, GROUPS, DIM)), dtype=dtype, device=device)
    history = [([], []) for _ in range(table.sequences())]
    rounded = lambda array: torch.tensor(array, dtype=dtype).float().numpy()
    compared = 0
    for action in schedule:
        if action[0] == "release":
            table.release(action[1])
            history[action[1]] = ([], [])
            continue
        counts, total = action[1], action[2]
        tokens = [list(rng.integers(1, 1000, size=n)) for n in counts]
        step = table.step_padded(device, tokens, total) if total else table.step(device, tokens)
        rows = step.tokens.numel()
        q = rounded(rng.standard_normal((rows, HEADS, DIM)).astype(np.float32))
        k = rounded(rng.standard_normal((rows, GROUPS, DIM)).astype(np.float32))
        v = rounded(rng.standard_normal((rows, GROUPS, DIM)).astype(np.float32))
        positions = step.positions.cpu().numpy()
        q_rotated, cos, sin = rotate(q, positions)
        k_rotated, _, _ = rotate(k, positions)
        to_device = lambda array, kind=dtype: torch.tensor(array, dtype=kind, device=device)
        write_pages, write_slots = step.slots()
        q_out = neural.rotary_cache_write(to_device(q), to_device(k), to_device(v), to_device(cos, torch.float32)[:, None, :],
                                          to_device(sin, torch.float32)[:, None, :], write_pages, write_slots, key_cache, value_cache)
        out, _ = neural.paged_attention(q_out, key_cache, value_cache, step.paging(), neural.AttentionOptions(causal=True))
        out = out.float().cpu().numpy()
        offsets = step.query_offsets.tolist()
        for sequence, count in enumerate(counts):
            if count == 0:
                continue
            first = offsets[sequence]
            keys, values = history[sequence]
            keys.extend(rounded(k_rotated[first:first + count]))
            values.extend(v[first:first + count])
            assert step.last_rows[sequence].item() == first + count - 1
            key_array = np.stack(keys).transpose(1, 0, 2)[None]      # [1, G, S, D]
            value_array = np.stack(values).transpose(1, 0, 2)[None]
            query_array = rounded(q_rotated[first:first + count]).transpose(1, 0, 2)[None]
            seen = key_array.shape[2]
            # Query i of the chunk sits at position seen - count + i and sees keys up to there.
            mask = np.where(np.arange(seen)[None, :] <= (seen - count + np.arange(count))[:, None], 0.0, -np.inf).astype(np.float32)
            want = oracle.scaled_dot_product_attention_f32(query_array, key_array, value_array, mask=mask[None, None])[0]
            got = out[first:first + count].transpose(1, 0, 2)
            difference = np.abs(got - want)
            assert difference.max() <= max_error and difference.mean() <= mean_error, (action, sequence, difference.max())
            compared += count
    return compared


SCHEDULE = [
    ("step", [5, 1, 9], 0),      # ragged prefill, pages taken as tokens arrive
    ("step", [1, 1, 1], 0),
    ("step", [0, 1, 1], 0),      # the first sequence holds: an idle row on the scratch page
    ("step", [3, 0, 1], 0),      # a chunk of three continues a sequence
    ("step", [1, 1, 1], 7),      # padded by four rows that read scratch pages
    ("release", 0),
    ("step", [0, 1, 1], 0),      # the released sequence has seen nothing: it reads the scratch page
    ("step", [6, 1, 1], 0),      # and starts over in pages it, or another, gave back
    ("step", [1, 1, 1], 0),
    ("step", [1, 1, 4], 0),
]


@pytest.mark.parametrize("dtype,max_error,mean_error", [(torch.float32, 1e-4, 1e-5), (torch.bfloat16, 2e-2, 2e-3)])
def test_decode_loop_through_the_page_table(dtype, max_error, mean_error):
    table = PageTable.create_shared(3, 40, 4, 64).with_padding(4)
    assert run_loop(dtype, SCHEDULE, table, max_error, mean_error, seed=11) == sum(sum(a[1]) for a in SCHEDULE if a[0] == "step")


def test_decode_loop_at_block_16_with_long_sequences():
    """32 decode steps after a 130- and a 47-token prefill at page size 16, bf16, every step checked."""
    table = PageTable.create(2, 200, 16)
    schedule = [("step", [130, 47], 0)] + [("step", [1, 1], 0)] * 32
    assert run_loop(torch.bfloat16, schedule, table, 2e-2, 2e-3, seed=12) == 130 + 47 + 64
