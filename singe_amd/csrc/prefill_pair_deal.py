"""Deals the work of one 32-key block of two 32-row tiles out over the slots behind its matrix instructions and writes
the block as the text fold_pair_block includes (prefill_pair_block_d128.inc and one for every other multiple of 16).

    python3 singe_amd/csrc/prefill_pair_deal.py          (rewrites the files beside this script)

A block at head_dim D is 2 * D / 16 score products of the NEXT block (tile A's and tile B's chains alternating, so that a
product never follows the one it accumulates onto) and 4 * ceil(D / 32) value products of this block (A's two 16-key
halves, then B's).  Behind each product sits a slot of other work, weighed in nominal issue cycles of four clocks (what
the dealing needs is an even spread and the right order, not exact costs: measured, a plain vector instruction of a
lone wave takes 4.5 clocks, an exponential 8, a matrix instruction's own issue 9): an exponential with its multiply-add
(E, 3), a running sum (T, 1, at least a slot after its exponential), a rounding of two weights into a word (W, 1, after
both exponentials and before the slot whose product reads the word), four direct-to-LDS loads of the tile (issue, 3 each),
the V^T operand reads of this block (VR, 2 each, before the value products of their half), the K operand reads of the
block after next (KR, 1 each, behind the last score product that reads the operand they replace), and in the last four
slots the row maxima of the next block's scores (three statements) and the lag test.  First fit, in that order, under a
budget per slot; the text keeps one slot a paragraph, `__builtin_amdgcn_sched_barrier(0)` behind the product and behind
the slot."""
import os
import re


def deal(steps, dim_blocks, budget, load_slots):
    products = []
    for j in range(steps):
        products.append(f"QK(a_nxt, qa, {j});")
        products.append(f"QK(b_nxt, qb, {j});")
    for tile, words in (("A", "wa"), ("B", "wb")):
        for half in range(2):
            for d in range(dim_blocks):
                products.append(f"PV({tile}, {half}, {d}, {words});")
    slots_n = len(products)
    first_value_product = 2 * steps
    # the slot whose product is the first to read the words of (tile, half)
    needed = {("wa", 0): first_value_product, ("wa", 1): first_value_product + dim_blocks,
              ("wb", 0): first_value_product + 2 * dim_blocks, ("wb", 1): first_value_product + 3 * dim_blocks}

    def softmax(scores, words, total, shift, low, high, deadline):
        out = []
        for e in range(low, high):
            out.append((3, f"E({scores}, {e}, {shift});", deadline))
            if e > low:
                out.append((1, f"T({total}, {scores}, {e - 1});", 99))
            if e % 2 == 1 and e - 2 >= low:
                out.append((1, f"W({words}, {scores}, {(e - 2) // 2});", deadline))
        out.append((1, f"T({total}, {scores}, {high - 1});", 99))
        out.append((1, f"W({words}, {scores}, {(high - 2) // 2});", deadline))
        return out

    stream = (softmax("a_cur", "wa", "total_a", "shift_a", 0, 8, needed[("wa", 0)]) + softmax("a_cur", "wa", "total_a", "shift_a", 8, 16, needed[("wa", 1)]) +
              softmax("b_cur", "wb", "total_b", "shift_b", 0, 8, needed[("wb", 0)]) + softmax("b_cur", "wb", "total_b", "shift_b", 8, 16, needed[("wb", 1)]))
    slots = [[] for _ in range(slots_n)]
    before = [[] for _ in range(slots_n)]  # what must come in front of a slot's product
    used = [0.0] * slots_n
    for n, at in enumerate(load_slots):
        slots[at].append(f"issue({n});")
        used[at] += 3
    value_reads = [(half, d) for half in range(2) for d in range(dim_blocks)]
    first_read = first_value_product - len(value_reads)  # the reads end right before the first value product
    for n, (half, d) in enumerate(value_reads):
        slots[first_read + n].append(f"VR({half}, {d});")
        used[first_read + n] += 2
    for j in range(steps):
        slots[first_value_product + j].append(f"KR({j});")
        used[first_value_product + j] += 1
    for n, text in enumerate(("ROW_MAXIMA_0;", "ROW_MAXIMA_1;", "ROW_MAXIMA_2;", "LAG_TEST;")):
        slots[slots_n - 4 + n].append(text)
        used[slots_n - 4 + n] += 8
    placed = {}

    def inputs(text):
        m = re.match(r"T\((\w+), (\w+), (\d+)\)", text)
        if m:
            return [(m.group(2), int(m.group(3)))]
        m = re.match(r"W\((\w+), (\w+), (\d+)\)", text)
        if m:
            return [(m.group(2), 2 * int(m.group(3))), (m.group(2), 2 * int(m.group(3)) + 1)]
        return []

    for cost, text, deadline in stream:
        at = 0
        for source in inputs(text):
            at = max(at, placed[source] + 1)
        while used[at] + cost > budget + 0.01 and at < min(slots_n - 1, deadline):
            at += 1
        assert at <= deadline, (text, at, deadline)
        (before if at == deadline else slots)[at].append(text)
        used[at] += cost
        m = re.match(r"E\((\w+), (\d+)", text)
        if m:
            placed[(m.group(1), int(m.group(2)))] = at
    lines = []
    for i in range(slots_n):
        lines.append(f"    // slot {i}")
        lines += ["    " + text for text in before[i]]
        lines.append("    " + products[i])
        lines.append("    __builtin_amdgcn_sched_barrier(0);")
        lines += ["    " + text for text in slots[i]]
        lines.append("    __builtin_amdgcn_sched_barrier(0);")
    return "\n".join(lines) + "\n", used


HEADER = """// One 32-key block of two 32-row tiles at head_dim {dim}, slot by slot: the text of fold_pair_block (prefill_pair.hip.h),
// written by prefill_pair_deal.py, which says what the statements are and how they were dealt.  Other work per slot, in
// issue cycles: {used}.
"""

# (head dimension, the smallest budget the dealing succeeds with, the slots of the four loads)
BLOCKS = ((128, 7.0, (0, 2, 4, 6)), (112, 8.0, (0, 2, 4, 6)), (96, 9.0, (0, 2, 4, 5)), (80, 10.0, (0, 2, 4, 6)),
          (64, 14.0, (0, 1, 2, 3)), (48, 16.0, (0, 1, 2, 3)), (32, 27.0, (0, 1, 2, 3)), (16, 36.0, (0, 1, 2, 3)))

if __name__ == "__main__":
    here = os.path.dirname(os.path.abspath(__file__))
    for dim, budget, load_slots in BLOCKS:
        body, used = deal(dim // 16, (dim + 31) // 32, budget, load_slots)
        with open(os.path.join(here, f"prefill_pair_block_d{dim}.inc"), "w") as out:
            out.write(HEADER.format(dim=dim, used=" ".join(f"{u:.0f}" for u in used)) + body)
        print(f"head_dim {dim}: {len(used)} slots, other work per slot", " ".join(f"{u:.0f}" for u in used))
