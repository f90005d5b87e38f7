"""Host-side mirror of the reference's paging producer (singe/src/nn/decode/step.rs): ``PageTable`` hands
out cache pages to sequences and writes each decode step's paging vectors, the ``DecodeStep`` that
``rotary_cache_write`` (write_pages / write_slots / positions) and ``paged_attention`` (paging) read.

Same names, argument meaning, page order (a sequence takes free pages in increasing order from page
zero) and failures as the reference; a step that fails leaves the table as it was.  The vectors are
int64 torch tensors on the device asked for (any torch device, or "cpu").
"""
from __future__ import annotations

from dataclasses import dataclass

import torch

from . import error
from .neural import Paging


@dataclass(frozen=True)
class DecodeStep:
    """One decode step's tokens, and where they fall in a paged cache (step.rs:13-30): everything that
    changes between steps is a tensor, so one captured step serves every position."""
    tokens: torch.Tensor             # [T] token ids
    positions: torch.Tensor          # [T] each token's position in its sequence
    write_pages: torch.Tensor        # [T] cache page each row writes
    write_slots: torch.Tensor        # [T] slot in that page
    query_offsets: torch.Tensor      # [S + 1]
    page_offsets: torch.Tensor       # [S + 1]
    pages: torch.Tensor              # [table_length]
    last_page_lengths: torch.Tensor  # [S]
    last_rows: torch.Tensor          # [S] row of each sequence's last real token
    real_tokens: torch.Tensor        # [S] rows that are the sequence's own tokens
    sequence_ids: torch.Tensor       # [T]

    def paging(self) -> Paging:
        """Where this step's queries and their keys sit, as attention reads them (step.rs:88-96)."""
        return Paging(self.query_offsets, self.page_offsets, self.pages, self.last_page_lengths)

    def slots(self):
        """One page and slot per token, the cells this step writes (step.rs:109-115)."""
        return self.write_pages, self.write_slots


@dataclass(frozen=True)
class PageLayout:
    """Where a page table places a step's tokens (step.rs:119-130)."""
    sequences: int
    capacity: int
    page_size: int
    scratch_page: int
    table_length: int


class PageTable:
    """Hands out cache pages to sequences, and writes each step's paging tensors (step.rs:132-146)."""

    def __init__(self, sequences: int, capacity: int, page_size: int, pool: int):
        self._page_size, self._capacity, self._pool, self._padding = page_size, capacity, pool, 0
        self._count = sequences
        self.reset()

    @classmethod
    def create(cls, sequences: int, capacity: int, page_size: int) -> "PageTable":
        """Enough pages for every sequence at once (step.rs:170-181)."""
        if sequences <= 0 or capacity <= 0 or page_size <= 0:
            raise error.InvalidArgument("page table size")
        return cls(sequences, capacity, page_size, sequences * ((capacity - 1) // page_size + 1))

    @classmethod
    def create_shared(cls, sequences: int, capacity: int, page_size: int, cache_tokens: int) -> "PageTable":
        """Pages that hold ``cache_tokens`` tokens, shared by the sequences (step.rs:183-199)."""
        if sequences <= 0 or capacity <= 0 or page_size <= 0 or cache_tokens <= 0:
            raise error.InvalidArgument("page table size")
        return cls(sequences, capacity, page_size, (cache_tokens - 1) // page_size + 1)

    def with_padding(self, padding: int) -> "PageTable":
        """Lets a step be padded by up to ``padding`` tokens (step.rs:215-219)."""
        if padding < 0:
            raise error.InvalidArgument("step padding")
        self._padding = padding
        return self

    def reset(self) -> None:
        """Forgets every sequence; the cache keeps its contents, which lengths hide (step.rs:221-228)."""
        self._free = list(range(self._pool - 1, -1, -1))  # popped from the end: page 0 first
        self._pages = [[] for _ in range(self._count)]
        self._lengths = [0] * self._count

    def release(self, sequence: int) -> None:
        """Forgets one sequence and returns its pages (step.rs:230-240)."""
        if not 0 <= sequence < self._count:
            raise error.InvalidArgument("decoder sequence out of range")
        self._free.extend(reversed(self._pages[sequence]))
        self._pages[sequence] = []
        self._lengths[sequence] = 0

    def free_pages(self) -> int:
        return len(self._free)

    def page_count(self) -> int:
        """Pages a cache needs: the pool and one scratch page (step.rs:248-252)."""
        return self._pool + 1

    def table_length(self) -> int:
        """Room for every held page, an idle row's scratch page each, and the scratch pages padding
        reads (step.rs:266-273)."""
        return self._pool + self._count + (self._padding + self._page_size - 1) // self._page_size

    def layout(self) -> PageLayout:
        return PageLayout(self._count, self._capacity, self._page_size, self._pool, self.table_length())

    def page_size(self) -> int:
        return self._page_size

    def capacity(self) -> int:
        return self._capacity

    def sequences(self) -> int:
        return self._count

    @staticmethod
    def step_tokens(tokens) -> int:
        """Rows a step takes: one per token, and one for each empty slice (step.rs:305-309)."""
        return sum(max(len(t), 1) for t in tokens)

    def step(self, device, tokens) -> DecodeStep:
        """Takes pages for ``tokens``, one slice per sequence, and writes the step that places them; an
        empty slice holds a sequence or leaves a row idle (step.rs:311-317)."""
        return self.step_padded(device, tokens, self.step_tokens(tokens))

    def step_padded(self, device, tokens, total: int) -> DecodeStep:
        """The step ``step`` would write, padded to ``total`` rows after the last sequence with tokens
        (step.rs:319-478)."""
        if len(tokens) != self._count or all(len(t) == 0 for t in tokens):
            raise error.InvalidArgument("decode step needs a slice for every sequence, and tokens in one")
        padding = total - self.step_tokens(tokens)
        if padding < 0:
            raise error.InvalidArgument("a decode step is padded to fewer rows than it has")
        if padding > self._padding:
            raise error.InvalidArgument(f"a decode step is padded by {padding} tokens, past the {self._padding} its page table allows")
        padded = max(row for row, t in enumerate(tokens) if len(t) > 0)
        for length, t in zip(self._lengths, tokens):
            if length + len(t) > self._capacity:
                raise error.InvalidArgument("decoder cache capacity out of range")
        # Checked before anything moves, so a step that overruns the pool changes nothing.
        fresh = 0
        for length, pages, t in zip(self._lengths, self._pages, tokens):
            if len(t) > 0:
                fresh += max((length + len(t) - 1) // self._page_size + 1 - len(pages), 0)
        if fresh > len(self._free):
            raise error.InvalidArgument("decoder cache pages out of range")

        size, scratch = self._page_size, self._pool
        flat, positions, write_pages, write_slots, sequence_ids = [], [], [], [], []
        query_offsets, last_rows, real_tokens, visible = [0], [], [], []
        for row, t in enumerate(tokens):
            pages = self._pages[row]
            for token in t:
                position = self._lengths[row]
                if position // size == len(pages):
                    pages.append(self._free.pop())
                flat.append(int(token))
                positions.append(position)
                write_pages.append(pages[position // size])
                write_slots.append(position % size)
                self._lengths[row] += 1
            if len(t) == 0:
                flat.append(0)
                positions.append(min(self._lengths[row], self._capacity - 1))
                write_pages.append(scratch)
                write_slots.append(0)
            last = len(flat) - 1
            keys = self._lengths[row]
            if row == padded:
                for position in range(self._lengths[row], self._lengths[row] + padding):
                    flat.append(0)
                    positions.append(min(position, self._capacity - 1))
                    write_pages.append(scratch)
                    write_slots.append(position % size)
                keys += padding
            visible.append(keys)
            sequence_ids.extend([row] * (len(flat) - len(sequence_ids)))
            query_offsets.append(len(flat))
            last_rows.append(last)
            real_tokens.append(len(t))

        # Unused trailing entries keep the table's shape, so one compiled step serves every length.
        table, page_offsets, last_page_lengths = [], [0], []
        for pages, seen in zip(self._pages, visible):
            if seen == 0:
                table.append(scratch)  # an idle row reads the scratch page, since every kernel takes a key
                last_page_lengths.append(1)
            else:
                used = (seen - 1) // size + 1
                held = min(used, len(pages))
                table.extend(pages[:held])
                table.extend([scratch] * (used - held))  # padding's keys past the sequence's own pages
                last_page_lengths.append((seen - 1) % size + 1)
            page_offsets.append(len(table))
        table.extend([0] * (self.table_length() - len(table)))

        vector = lambda values: torch.tensor(values, dtype=torch.int64, device=device)
        return DecodeStep(vector(flat), vector(positions), vector(write_pages), vector(write_slots), vector(query_offsets),
                          vector(page_offsets), vector(table), vector(last_page_lengths), vector(last_rows), vector(real_tokens),
                          vector(sequence_ids))
