"""Device storage of the cache and its link to the host bookkeeping.

Key/value groups: ``k`` of shape ``[lines, pages, kv_heads, 64, head_dim]`` and ``v``
of shape ``[lines, pages, kv_heads, head_dim, 64]`` (transposed within a page) in the
compute dtype, so one (page, kv head) is one contiguous tile of 64 keys or values and
both matrix products of attention read contiguous runs along their contraction index.
The 64 columns of a page of values hold its positions in the order the matrix cores take
them (``value_column``: position ``16a + 4g + i`` of a block of 32 sits in column
``8g + 4a + i``), which only the kernels that write and read pages need to know. The reference's layout is
``[layers, rows, kv_heads, L_cap, head_dim]`` (engine/dryft_qwen3/cache.py:3-6);
the page indirection replaces its fixed ``L_cap`` per row. State groups:
``[lines, slots, *shape]``. Storage is zero-initialised once so that bytes no
length covers can never hold a NaN (cache.py:44-47); releasing a slot resets its
length and its fixed-size state but leaves key/value bytes alone (cache.py:73-81).
"""

from __future__ import annotations

from dataclasses import dataclass

import numpy as np
import torch

from .pages import CacheFull, PageTable, SlotTable
from .spec import KVNeed, PAGE_TOKENS, StateNeed, pages_for

_STATE_DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16, "int32": torch.int32}


@dataclass
class KVLine:
    """What an attention-like mixer gets for one cache line."""

    k: torch.Tensor           # [pages, kv_heads, 64, head_dim]
    v: torch.Tensor           # [pages, kv_heads, head_dim, 64]
    page_table: torch.Tensor  # [slots, max_pages] int32, device
    max_pages: int
    window: int | None


@dataclass
class StateLine:
    """What a mixer with fixed-size state gets: ``state[slot]`` is that sequence's."""

    state: torch.Tensor       # [slots, *shape]


class KVGroup:
    def __init__(self, need: KVNeed, lines: list[int], n_pages: int, n_slots: int, max_pages: int,
                 dtype: torch.dtype, device):
        self.need, self.lines = need, list(lines)
        shape = (len(lines), n_pages, need.num_kv_heads, PAGE_TOKENS, need.head_dim)
        self.k = torch.zeros(shape, dtype=dtype, device=device)
        # values are kept transposed within a page: [.., head_dim, 64], columns in the kernels' own order
        self.v = torch.zeros(shape[:3] + (need.head_dim, PAGE_TOKENS), dtype=dtype, device=device)
        self.table = PageTable(n_slots, n_pages, max_pages, need.window)
        self.table_dev = torch.full((n_slots, max_pages), -1, dtype=torch.int32, device=device)
        self.max_pages = max_pages

    def upload(self) -> None:
        dirty = self.table.dirty
        if not dirty:
            return
        lo, hi = min(dirty), max(dirty) + 1
        self.table_dev[lo:hi].copy_(torch.from_numpy(self.table.table[lo:hi]))
        dirty.clear()

    def bytes(self) -> int:
        return 2 * self.k.numel() * self.k.element_size()


class StateGroup:
    def __init__(self, need: StateNeed, lines: list[int], n_slots: int, device):
        self.need, self.lines = need, list(lines)
        self.data = torch.zeros((len(lines), n_slots) + tuple(need.shape),
                                dtype=_STATE_DTYPES[need.dtype], device=device)

    def bytes(self) -> int:
        return self.data.numel() * self.data.element_size()


class CacheStore:
    """All groups of one model, sized by a token budget.

    ``max_tokens`` is the most tokens live sequences hold together, each
    sequence's count rounded up to whole pages; ``max_len`` bounds one sequence.
    """

    def __init__(self, needs: dict[int, KVNeed | StateNeed | dict | None], *, max_tokens: int, n_slots: int,
                 max_len: int, dtype: torch.dtype, device):
        """``needs``: per cache line what it keeps: one need, or a dictionary from names to needs for a line that keeps
        several things; ``line()`` then returns a dictionary of storage under the same names."""
        self.device = torch.device(device)
        self.dtype = dtype
        self.n_pages = max(1, pages_for(max_tokens))
        self.n_slots = int(n_slots)
        self.max_len = int(max_len)
        self.max_pages = max(1, pages_for(max_len))
        self.slots = SlotTable(self.n_slots)
        self.lengths_dev = torch.zeros(self.n_slots, dtype=torch.int32, device=self.device)
        self.kv_groups: list[KVGroup] = []
        self.state_groups: list[StateGroup] = []
        self._line: dict[object, tuple[object, int]] = {}
        self._named: dict[object, list[str]] = {}      # lines that keep several things: the names of those
        by_need: dict[object, list[object]] = {}
        for line, need in needs.items():
            if isinstance(need, dict):
                self._named[line] = list(need)
                for name, one in need.items():
                    if one is not None:
                        by_need.setdefault(one, []).append((line, name))
            elif need is not None:
                by_need.setdefault(need, []).append(line)
        for need, lines in by_need.items():
            if isinstance(need, KVNeed):
                g = KVGroup(need, lines, self.n_pages, self.n_slots, self.max_pages, dtype, self.device)
                self.kv_groups.append(g)
            elif isinstance(need, StateNeed):
                g = StateGroup(need, lines, self.n_slots, self.device)
                self.state_groups.append(g)
            else:
                raise TypeError(f"cache line {lines[0]}: unknown need {need!r}")
            for i, line in enumerate(lines):
                self._line[line] = (g, i)

    # ---- what mixers see
    def line(self, line):
        """The storage of a cache line: a ``KVLine``, a ``StateLine``, None for a line that keeps nothing, or a
        dictionary of those for a line that asked for several things by name."""
        if line in self._named:
            return {name: self._storage((line, name)) for name in self._named[line]}
        return self._storage(line)

    def _storage(self, line) -> KVLine | StateLine | None:
        entry = self._line.get(line)
        if entry is None:
            return None
        g, i = entry
        if isinstance(g, KVGroup):
            return KVLine(g.k[i], g.v[i], g.table_dev, g.max_pages, g.need.window)
        return StateLine(g.data[i])

    # ---- slots
    def acquire(self, n: int) -> list[int]:
        if n > self.slots.free_count:
            raise CacheFull(f"{n} sequences asked for, {self.slots.free_count} of {self.n_slots} slots are free")
        return [self.slots.acquire() for _ in range(n)]

    def release(self, slots: list[int]) -> None:
        if not slots:
            return
        for s in slots:
            self.slots.release(s)          # raises on a slot that is not held
            for g in self.kv_groups:
                g.table.release(s)
        idx = torch.tensor(slots, dtype=torch.long, device=self.device)
        self.lengths_dev.index_fill_(0, idx, 0)
        for g in self.state_groups:
            g.data.index_fill_(1, idx, 0)
        for g in self.kv_groups:
            g.upload()

    # ---- steps
    def begin_step(self, slots: list[int], q_lens: list[int]) -> list[int]:
        """Give every sequence room for its new tokens; returns the lengths before the step."""
        past = []
        for s, q in zip(slots, q_lens):
            self.slots.check_held(s)
            n = int(self.slots.lengths[s])
            if n + q > self.max_len:
                raise CacheFull(f"slot {s}: {n} + {q} tokens exceed the longest sequence allowed ({self.max_len})")
            past.append(n)
        try:
            for g in self.kv_groups:
                for s, q, n in zip(slots, q_lens, past):
                    if q:
                        g.table.ensure(s, n + q)
        finally:
            for g in self.kv_groups:
                g.upload()
        return past

    def end_step(self, slots: list[int], q_lens: list[int]) -> None:
        """Record that the step has appended ``q_lens`` tokens (the device advances its own copy)."""
        for s, q in zip(slots, q_lens):
            self.slots.lengths[s] += q
        trimmed = False
        for g in self.kv_groups:
            if g.need.window is not None:
                for s in slots:
                    g.table.trim(s, int(self.slots.lengths[s]))
                trimmed = True
        if trimmed:
            for g in self.kv_groups:
                g.upload()

    def reserve(self, slots: list[int], lengths: list[int]) -> None:
        """Take the pages a sequence will need up to ``lengths`` now, so later steps change no table."""
        for g in self.kv_groups:
            if g.need.window is None:
                for s, n in zip(slots, lengths):
                    g.table.ensure(s, min(n, self.max_len))
            g.upload()

    def bytes(self) -> int:
        return sum(g.bytes() for g in self.kv_groups) + sum(g.bytes() for g in self.state_groups)

    def bytes_read(self, context: float) -> float:
        """What one more token of a sequence ``context`` tokens long reads from the cache: the keys and values it
        sees on every line, and its fixed-size state."""
        total = 0.0
        for g in self.kv_groups:
            seen = min(context, g.need.window) if g.need.window else context
            total += 2.0 * len(g.lines) * g.need.num_kv_heads * g.need.head_dim * g.k.element_size() * seen
        for g in self.state_groups:
            total += g.bytes() / self.n_slots
        return total

    def lengths_host(self) -> np.ndarray:
        return self.slots.lengths.copy()
