"""The cache on the device: keys and values per run-order entry, per-slot state.

Entries of the run order with the same needs (kv heads, head size, window, storage dtype)
form a group; each group has storage, a page pool and block tables of its own (a group
with a window holds only the pages its window still reaches):
``K: [entry in group, page, kv head, position in page, head_dim]``, ``V`` the same with its
last two axes exchanged; inside a page of one head the elements lie in the tiles that the
attention kernels read as matrix operands (``layout.py``), so a page is a unit that only
kernels, and code that goes through ``layout.py``, look into. A page is
``page_size`` positions of one sequence for every entry of the group. Beside it
each entry may own a state area of fixed size per slot, ``[slot, elements]``,
zeroed when the slot is handed out; the attention of this architecture asks for
none (the reference has no such state either: J/inference/state/State.java:28-65).

Every group also keeps its block table on the device, one row per slot, ``[n_slots + 1,
pages of the longest sequence]``: a step names the rows (slot numbers) of its sequences and
uploads no page numbers. The host changes single entries when a sequence gets or returns a
page; the changes travel inside a launch (``flush_tables``). Row ``n_slots`` belongs to no
sequence and names the sink page only: entries that pad a batch to a fixed size use it, and
the matching row of every state area, so that they touch nothing a sequence owns.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import numpy as np
import torch

from .pages import CacheFull, PagePool, SlotTable


@dataclass(frozen=True)
class KVNeed:
    """What one run-order entry stores per position: keys of ``head_dim`` elements and values of
    ``v_head_dim`` for each of ``n_kv_heads`` heads. A mixer that keeps one vector per position (a
    latent that both its keys and its values are made from) asks for ``values=False`` and gets the
    first array alone."""
    n_kv_heads: int
    head_dim: int
    window: Optional[int] = None
    dtype: Optional[torch.dtype] = None      # None: the engine's; a mixer whose kernels keep something else says so
    v_head_dim: Optional[int] = None         # None: as the keys'
    values: bool = True                      # False: no second array (``layer_kv`` then gives (keys, None))

    @property
    def value_dim(self):
        return self.head_dim if self.v_head_dim is None else self.v_head_dim


@dataclass(frozen=True)
class StateNeed:
    """What one run-order entry stores per sequence, whatever its length."""
    elements: int
    dtype: torch.dtype = torch.float32


def check_layout(kv_needs, page_size):
    """The cache lies in the tiles of the attention kernels' operands (``layout.py``): pages of a multiple of 32
    positions, heads of a multiple of 16 elements. Anything else is refused here, by name, before any
    memory is taken or any weight is read; the kernels would refuse it at their first launch."""
    if isinstance(page_size, bool) or not isinstance(page_size, int) or page_size < 32 or page_size % 32:
        raise ValueError(f"page_size {page_size!r}: a page of the cache must be a positive multiple of 32 positions")
    for e, need in enumerate(kv_needs):
        if need is None:
            continue
        sizes = [("head_dim", need.head_dim)] + ([("v_head_dim", need.value_dim)] if need.values else [])
        for key, v in sizes:
            if v < 16 or v % 16:
                raise ValueError(f"run-order entry {e}: {key} {v} is not a multiple of 16; the cache keeps heads in "
                                 "tiles of 16 by 8 elements (head sizes in steps of 16)")
        if need.n_kv_heads < 1:
            raise ValueError(f"run-order entry {e}: {need.n_kv_heads} kv heads")


class CacheGroup:
    def __init__(self, need, entries, n_pages, page_size, dtype, device):
        self.need = need
        self.entries = list(entries)
        self.pool = PagePool(n_pages)
        self.page_size = page_size
        n = len(self.entries)
        dtype = need.dtype or dtype
        self.k = torch.zeros((n, n_pages, need.n_kv_heads, page_size, need.head_dim), dtype=dtype, device=device)
        # values lie transposed inside a page: the order in which the attention kernels' second
        # product reads them (and both in tiles, see layout.py)
        self.v = (torch.zeros((n, n_pages, need.n_kv_heads, need.value_dim, page_size), dtype=dtype, device=device)
                  if need.values else None)
        self.table = None            # [n_slots + 1, pages of the longest sequence] int32 on the device
        self.table_host = None       # the same on the host (numpy), the copy that the bookkeeping writes
        self.dirty = {}              # flat place in the table -> page number, not yet on the device


class Cache:
    """``kv_needs[e]`` / ``state_needs[e]`` give run-order entry e's needs (None: nothing).

    ``max_tokens``: positions that all live sequences may hold together, each
    sequence's count rounded up to whole pages. ``max_context``: longest sequence.
    """

    def __init__(self, kv_needs, state_needs, max_tokens, max_context, n_slots, dtype, device, page_size=64):
        if max_tokens < 1 or max_context < 1 or n_slots < 1:
            raise ValueError("cache sizes must be positive")
        check_layout(kv_needs, page_size)
        self.page_size = page_size
        self.max_context = max_context
        self.max_pages_per_seq = -(-max_context // page_size)
        self.dtype = dtype
        self.device = device
        n_pages = -(-max_tokens // page_size) + 1           # + the sink page
        self.groups = []
        self.group_of = {}                                   # entry -> (group index, index inside the group)
        by_need = {}
        for e, need in enumerate(kv_needs):
            if need is not None:
                by_need.setdefault(need, []).append(e)
        for need, entries in by_need.items():
            g = CacheGroup(need, entries, n_pages, page_size, dtype, device)
            for i, e in enumerate(entries):
                self.group_of[e] = (len(self.groups), i)
            self.groups.append(g)
        self.slots = SlotTable(n_slots, len(self.groups))
        self._windowed = any(g.need.window for g in self.groups)
        self.sink_slot = n_slots                             # the row of padded entries: no sequence's
        for g in self.groups:
            g.table_host = np.zeros((n_slots + 1, self.max_pages_per_seq), dtype=np.int32)
            g.table = torch.zeros((n_slots + 1, self.max_pages_per_seq), dtype=torch.int32, device=device)
        self.state = {}
        for e, need in enumerate(state_needs):
            if need is not None and need.elements > 0:
                self.state[e] = torch.zeros((n_slots + 1, need.elements), dtype=need.dtype, device=device)

    # ---- slots
    def take_slot(self):
        s = self.slots.take()
        for t in self.state.values():
            t[s].zero_()
        return s

    def give_back_slot(self, s):
        self.slots.check(s)
        for g, group in enumerate(self.groups):
            group.pool.give_back([p for p in self.slots.pages[s][g] if p])   # (0: a page given back earlier)
            self.slots.pages[s][g] = []
        self.slots.give_back(s)

    def length(self, s):
        self.slots.check(s)
        return self.slots.length[s]

    def reserve(self, wanted):
        """Make room for ``{slot: n new tokens}`` in every group, or change nothing."""
        plan = []
        for s, n in wanted.items():
            self.slots.check(s)
            new_len = self.slots.length[s] + n
            if new_len > self.max_context:
                raise CacheFull(f"slot {s}: {new_len} tokens exceed the longest sequence of {self.max_context}")
            need_pages = -(-new_len // self.page_size)
            for g in range(len(self.groups)):
                plan.append((s, g, need_pages - len(self.slots.pages[s][g])))
        for g, group in enumerate(self.groups):
            total = sum(extra for _, gg, extra in plan if gg == g and extra > 0)
            if total > group.pool.n_free:
                raise CacheFull(f"{total} more pages wanted, {group.pool.n_free} free: the cache holds "
                                f"{(group.pool.n_pages - 1) * self.page_size} tokens")
        for s, g, extra in plan:
            if extra > 0:
                pages = self.slots.pages[s][g]
                first = len(pages)
                pages.extend(self.groups[g].pool.take(extra))
                self._table_set(g, s, first, pages[first:])

    def reserve_one_each(self, slots):
        """``reserve`` for a step that brings one token per sequence: nothing to do while every
        sequence's last page has room (the usual case of a decode step)."""
        page, pages, length = self.page_size, self.slots.pages, self.slots.length
        for s in slots:
            n = length[s]
            if n >= self.max_context or any(n >= len(held) * page for held in pages[s]):
                return self.reserve({s: 1 for s in slots})

    def advance_one_each(self, slots):
        if self._windowed:
            for s in slots:
                self.advance(s, 1)
        else:
            length = self.slots.length
            for s in slots:
                length[s] += 1

    def advance(self, s, n):
        """The sequence of slot ``s`` has ``n`` more tokens. A group with a window gives back the
        pages that no later token can see: the next token, at position ``length``, reads the keys
        from ``length + 1 - window`` on. Their places in the slot's list of pages become the sink
        page, which nobody reads."""
        self.slots.length[s] += n
        for g, group in enumerate(self.groups):
            window = group.need.window
            if not window:
                continue
            pages = self.slots.pages[s][g]
            first_seen = max(0, self.slots.length[s] + 1 - window) // self.page_size
            gone = [i for i in range(min(first_seen, len(pages))) if pages[i]]
            if gone:
                group.pool.give_back([pages[i] for i in gone])
                for i in gone:
                    pages[i] = 0
                    self._table_set(g, s, i, [0])

    # ---- the block tables on the device
    def _table_set(self, g, slot, first, pages):
        group = self.groups[g]
        base = slot * self.max_pages_per_seq + first
        for i, p in enumerate(pages):
            group.table_host[slot, first + i] = p
            group.dirty[base + i] = p

    def flush_tables(self):
        """Bring the device tables up to date (on the current stream): only entries that changed since
        the last call travel, inside the launch of a small kernel."""
        for group in self.groups:
            if group.dirty:
                from ..csrc import lib as K
                K.scatter_i32(group.table, list(group.dirty.keys()), list(group.dirty.values()))
                group.dirty = {}

    def device_table(self, group):
        """``[n_slots + 1, max_pages_per_seq]`` int32: row s holds slot s's pages (call ``flush_tables``
        before a kernel reads it)."""
        return self.groups[group].table

    # ---- what the kernels read
    def layer_kv(self, entry):
        """(K, V) of one entry: K [page, kv head, position in page, head_dim], V [page, kv head, v_head_dim, position]
        (None for a need without values); the last two axes in the kernels' order (``layout.py``)."""
        g, i = self.group_of[entry]
        group = self.groups[g]
        return group.k[i], (group.v[i] if group.v is not None else None)

    def group_index(self, entry):
        return self.group_of[entry][0]

    def slot_state(self, entry):
        return self.state.get(entry)

    def tokens_free(self):
        """Positions that can still be handed out (no per-position storage: no bound but the slots)."""
        if not self.groups:
            return self.slots.n_slots * self.max_context
        return min(g.pool.n_free for g in self.groups) * self.page_size
