"""Host-side bookkeeping of the cache: slots, pages and lengths. No device code.

A slot stands for one live sequence: it has a length and, per key/value group,
a row of page numbers. Pages are handed out as a sequence grows and go back to
the pool when the slot is released (or, for a windowed group, when they have
fallen out of the window). The reference keeps a fixed ``[B_cap, L_cap]`` region
per row and resets only lengths (engine/dryft_qwen3/cache.py:73-81); here too the
bytes of a returned page are left as they are, and only lengths and tables say
what is valid.
"""

from __future__ import annotations

import numpy as np

from .spec import PAGE_TOKENS, pages_for


class CacheFull(RuntimeError):
    """No free slot or page is left for what was asked."""


class CacheMisuse(RuntimeError):
    """A slot or page was released twice, or used without being held."""


class PagePool:
    """Free list of page numbers ``0..n_pages-1``."""

    def __init__(self, n_pages: int):
        self.n_pages = int(n_pages)
        self._free = list(range(self.n_pages - 1, -1, -1))  # pop() hands out low numbers first
        self._held = np.zeros(self.n_pages, dtype=bool)

    @property
    def free_count(self) -> int:
        return len(self._free)

    def take(self, n: int) -> list[int]:
        if n > len(self._free):
            raise CacheFull(f"need {n} pages, {len(self._free)} of {self.n_pages} are free")
        out = [self._free.pop() for _ in range(n)]
        self._held[out] = True
        return out

    def give_back(self, pages: list[int]) -> None:
        for p in pages:
            if not (0 <= p < self.n_pages) or not self._held[p]:
                raise CacheMisuse(f"page {p} is not held")
            self._held[p] = False
            self._free.append(p)


class PageTable:
    """Pages of one key/value group: per slot, position ``p`` lives in page ``table[slot, p // 64]``."""

    def __init__(self, n_slots: int, n_pages: int, max_pages_per_slot: int, window: int | None = None):
        self.pool = PagePool(n_pages)
        self.window = window
        self.table = np.full((n_slots, max_pages_per_slot), -1, dtype=np.int32)
        self.first = np.zeros(n_slots, dtype=np.int64)   # first page index still held
        self.count = np.zeros(n_slots, dtype=np.int64)   # one past the last page index held
        self.dirty: set[int] = set()                     # slots whose row changed since the last upload

    def ensure(self, slot: int, new_len: int) -> None:
        """Make sure positions ``[.., new_len)`` of ``slot`` have pages."""
        need = pages_for(new_len)
        if need > self.table.shape[1]:
            raise CacheFull(f"a sequence of {new_len} tokens needs {need} pages; a slot holds {self.table.shape[1]}")
        have = int(self.count[slot])
        if need > have:
            self.table[slot, have:need] = self.pool.take(need - have)
            self.count[slot] = need
            self.dirty.add(slot)

    def trim(self, slot: int, length: int) -> None:
        """Windowed groups: free pages no position of which a later token can see."""
        if self.window is None:
            return
        keep_from = max(0, length - self.window + 1) // PAGE_TOKENS   # oldest page the next token still needs
        first = int(self.first[slot])
        if keep_from > first:
            self.pool.give_back([int(p) for p in self.table[slot, first:keep_from]])
            self.table[slot, first:keep_from] = -1
            self.first[slot] = keep_from
            self.dirty.add(slot)

    def release(self, slot: int) -> None:
        first, count = int(self.first[slot]), int(self.count[slot])
        self.pool.give_back([int(p) for p in self.table[slot, first:count]])
        self.table[slot, :] = -1
        self.first[slot] = 0
        self.count[slot] = 0
        self.dirty.add(slot)

    def held_pages(self, slot: int) -> list[int]:
        return [int(p) for p in self.table[slot, int(self.first[slot]):int(self.count[slot])]]


class SlotTable:
    """Which slots are in use and how long their sequences are."""

    def __init__(self, n_slots: int):
        self.n_slots = int(n_slots)
        self._free = list(range(self.n_slots - 1, -1, -1))
        self.in_use = np.zeros(self.n_slots, dtype=bool)
        self.lengths = np.zeros(self.n_slots, dtype=np.int64)

    @property
    def free_count(self) -> int:
        return len(self._free)

    def acquire(self) -> int:
        if not self._free:
            raise CacheFull(f"all {self.n_slots} slots are in use")
        s = self._free.pop()
        self.in_use[s] = True
        self.lengths[s] = 0
        return s

    def release(self, slot: int) -> None:
        self.check_held(slot)
        self.in_use[slot] = False
        self.lengths[slot] = 0
        self._free.append(slot)

    def check_held(self, slot: int) -> None:
        if not (0 <= slot < self.n_slots) or not self.in_use[slot]:
            raise CacheMisuse(f"slot {slot} is not held")
