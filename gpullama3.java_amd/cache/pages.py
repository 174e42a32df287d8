"""Host-side bookkeeping of the cache: slots for sequences and pages for their tokens.

The reference keeps one state object per conversation whose cache is sized for the
whole context (J/inference/state/LlamaState.java:44-46, :61-64) and accepts a batch
size only to drop it (J/inference/state/State.java:69-70). Here a slot is handed to
each sequence of a batch and taken back when the sequence ends, and the tokens of a
slot live in pages of a fixed number of positions drawn from one pool, so that the
memory a sequence holds follows its own length.
"""
from __future__ import annotations


class CacheFull(RuntimeError):
    """No free slot, no free page, or a sequence beyond its longest allowed length."""


class PagePool:
    """Pages 1..n_pages-1 are handed out; page 0 is never handed out: writes of padded
    tokens land there and nobody reads it."""

    def __init__(self, n_pages):
        if n_pages < 2:
            raise ValueError("a page pool needs at least one page beside the sink")
        self.n_pages = n_pages
        self._free = list(range(n_pages - 1, 0, -1))
        self._held = set()

    @property
    def n_free(self):
        return len(self._free)

    def take(self, n):
        if n > len(self._free):
            raise CacheFull(f"{n} pages wanted, {len(self._free)} free of {self.n_pages - 1}")
        pages = [self._free.pop() for _ in range(n)]
        self._held.update(pages)
        return pages

    def give_back(self, pages):
        for p in pages:
            if p not in self._held:
                raise RuntimeError(f"page {p} is given back but not held")
        for p in pages:
            self._held.discard(p)
            self._free.append(p)


class SlotTable:
    """Slots 0..n_slots-1, each with the length of its sequence and its pages per group."""

    def __init__(self, n_slots, n_groups):
        self.n_slots = n_slots
        self._free = list(range(n_slots - 1, -1, -1))
        self.live = set()
        self.length = [0] * n_slots
        self.pages = [[[] for _ in range(n_groups)] for _ in range(n_slots)]

    @property
    def n_free(self):
        return len(self._free)

    def take(self):
        if not self._free:
            raise CacheFull(f"all {self.n_slots} slots are held")
        s = self._free.pop()
        self.live.add(s)
        self.length[s] = 0
        return s

    def give_back(self, s):
        if s not in self.live:
            raise RuntimeError(f"slot {s} is given back but not held")
        self.live.discard(s)
        self.length[s] = 0
        self._free.append(s)

    def check(self, s):
        if s not in self.live:
            raise RuntimeError(f"slot {s} is not held")
