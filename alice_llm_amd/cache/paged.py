"""The cache: a slot per sequence, keys and values per layer in pages, and fixed-size state.

The runs of the schedule (one per layer, unless the schedule names a layer twice) are grouped by what
they need: all that keep every key form one group, all that read a window of W keys form another, each with page storage of its own
([layers of the group][page][kv head][64 positions][head_dim]) and a page table per slot.  A
windowed group gives pages back as soon as no later query can reach them.  A slot is taken when a
sequence starts and given back when it ends; its pages return to the pools and are used again
without being cleared, because reads are bounded by the slot's length.  Beside the pages, every
layer that declares state of fixed size gets one region per slot, zeroed when the slot is taken.

The reference keeps one flat [layer][position] store per sequence with a length cursor
(llama3.rs:4731-4827), a per-request paged variant with 16-token pages (llama3.rs:5059-5170),
applies the window at read time (llama3.rs:5448-5451) and keeps fixed-size recurrent state in
per-model buffers (llama3.rs:12983-13003).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Tuple

import torch

from ..parts.base import CacheNeed, KVNeed

PAGE_SIZE = 64


class CacheError(RuntimeError):
    """Capacity is exhausted, or a slot is used in a way its state does not allow."""


class SlotTable:
    """Which slots are free, which are held, and how long each held sequence is."""

    def __init__(self, n_slots: int):
        self.n_slots = n_slots
        self._free: List[int] = list(range(n_slots - 1, -1, -1))
        self._len: Dict[int, int] = {}

    def take(self) -> int:
        if not self._free:
            raise CacheError(f"all {self.n_slots} slots are held")
        s = self._free.pop()
        self._len[s] = 0
        return s

    def give_back(self, slot: int) -> None:
        if slot not in self._len:
            raise CacheError(f"slot {slot} is not held (freed twice, or never taken)")
        del self._len[slot]
        self._free.append(slot)

    def held(self) -> List[int]:
        return sorted(self._len)

    def n_free(self) -> int:
        return len(self._free)

    def length(self, slot: int) -> int:
        if slot not in self._len:
            raise CacheError(f"slot {slot} is not held")
        return self._len[slot]

    def advance(self, slot: int, n: int) -> None:
        self._len[slot] = self.length(slot) + n


class PageGroup:
    """Page storage and page tables of the layers that share one KVNeed."""

    def __init__(self, need: KVNeed, layers: Sequence[int], n_pages: int, dtype: torch.dtype, device,
                 page_size: int = PAGE_SIZE, allocate: bool = True):
        self.need = need
        self.layers = list(layers)
        self.page_size = page_size
        self.n_pages = n_pages                      # usable pages; page 0 of the pool is never handed out
        self._free: List[int] = list(range(n_pages, 0, -1))
        self._table: Dict[int, List[int]] = {}      # slot -> page id per page index, -1 once given back
        if need.page_size is not None and need.page_size != page_size:
            raise CacheError(f"the layers {self.layers} need pages of {need.page_size} positions (their kernels are "
                             f"written for that), the cache has pages of {page_size}")
        dtype = need.dtype or dtype                 # the mixer's own choice, else the run's activation dtype
        self.dtype = dtype
        shape = (len(self.layers), n_pages + 1, need.num_kv_heads, page_size)
        self.k = torch.zeros(shape + (need.head_dim,), dtype=dtype, device=device) if allocate else None
        self.v = torch.zeros(shape + (need.v_dim,), dtype=dtype, device=device) if allocate else None

    # -- bookkeeping (host only) ---------------------------------------------------------
    def open(self, slot: int) -> None:
        if slot in self._table:
            raise CacheError(f"slot {slot} already has a page table")
        self._table[slot] = []

    def pages_needed(self, slot: int, new_len: int) -> int:
        have = len(self._table[slot])
        return max(0, -(-new_len // self.page_size) - have)

    def n_free(self) -> int:
        return len(self._free)

    def grow(self, slot: int, new_len: int) -> None:
        tab = self._table[slot]
        want = -(-new_len // self.page_size)
        if want - len(tab) > len(self._free):
            raise CacheError("out of pages")
        while len(tab) < want:
            tab.append(self._free.pop())

    def trim(self, slot: int, length: int) -> None:
        """Give back the pages that no query at position >= length can reach; True if any was."""
        w = self.need.window
        if w is None:
            return False
        first_needed = max(0, length + 1 - w)        # oldest key of the next query
        tab = self._table[slot]
        changed = False
        for i in range(min(first_needed // self.page_size, len(tab))):
            if tab[i] >= 0:
                self._free.append(tab[i])
                tab[i] = -1
                changed = True
        return changed

    def close(self, slot: int) -> None:
        if slot not in self._table:
            raise CacheError(f"slot {slot} has no page table (closed twice?)")
        for p in self._table.pop(slot):
            if p >= 0:
                self._free.append(p)

    def table(self, slot: int) -> List[int]:
        return self._table[slot]

    def held_pages(self) -> List[int]:
        return [p for tab in self._table.values() for p in tab if p >= 0]


@dataclass
class LayerCache:
    """What one run of a layer sees of the cache during a step."""
    k: Optional[torch.Tensor]             # [pages, nKV, page, d] of this layer
    v: Optional[torch.Tensor]
    block_table: Optional[torch.Tensor]   # int32 [sequences of the step, pages]
    writable: bool                        # False when the run reads another layer's cache
    state: Dict[str, torch.Tensor]        # by the name of its StateNeed: [slots + 1, *shape], index with ctx.slots
    group: Optional[int] = None


class Cache:
    def __init__(self, needs: Sequence[Optional[CacheNeed]], *, max_tokens: int, dtype: torch.dtype, device,
                 max_seqs: Optional[int] = None, page_size: int = PAGE_SIZE, allocate: bool = True):
        """needs[i]: what run i of the schedule declares (None: nothing).  `max_tokens`: the most tokens that live
        sequences hold at any time, each sequence's count rounded up to a multiple of the page size."""
        self.page_size = page_size
        self.device = device
        n_pages = max(1, -(-max_tokens // page_size))
        self.max_tokens = n_pages * page_size
        n_slots = max_seqs if max_seqs is not None else min(n_pages, 4096)
        self.slots = SlotTable(n_slots)
        self.version = 0                       # bumped whenever any page table changes
        by_need: Dict[KVNeed, List[int]] = {}
        for i, need in enumerate(needs):
            if need is not None and need.kv is not None:
                by_need.setdefault(need.kv, []).append(i)
        self.groups: List[PageGroup] = [PageGroup(kv, layers, n_pages, dtype, device, page_size, allocate)
                                        for kv, layers in by_need.items()]
        self._where: Dict[int, Tuple[int, int]] = {}
        for gi, g in enumerate(self.groups):
            for li, layer in enumerate(g.layers):
                self._where[layer] = (gi, li)
        # Fixed-size state: per run of the schedule, one tensor per declared StateNeed with a row per slot and one
        # spare row (index n_slots) that the padded rows of a captured decode step read and write.
        self.spare_slot = n_slots
        self.state: Dict[int, Dict[str, torch.Tensor]] = {}
        for i, need in enumerate(needs):
            if need is not None and need.state and allocate:
                self.state[i] = {st.name: torch.zeros((n_slots + 1, *st.shape), dtype=st.dtype, device=device)
                                 for st in need.state}

    # -- slots ---------------------------------------------------------------------------
    def open(self) -> int:
        slot = self.slots.take()
        for g in self.groups:
            g.open(slot)
        for tensors in self.state.values():
            for t in tensors.values():
                t[slot].zero_()
        return slot

    def close(self, slot: int) -> None:
        self.slots.give_back(slot)
        self.version += 1
        for g in self.groups:
            g.close(slot)

    def length(self, slot: int) -> int:
        return self.slots.length(slot)

    def tokens_free(self) -> int:
        return min((g.n_free() for g in self.groups), default=self.max_tokens // self.page_size) * self.page_size

    # -- a step --------------------------------------------------------------------------
    def reserve(self, slots: Sequence[int], n_new: Sequence[int]) -> None:
        """Make room for n_new[i] more tokens in slots[i]; raises before anything changes."""
        if len(set(slots)) != len(slots):
            raise CacheError(f"a step names a slot twice: {list(slots)}")
        lens = [self.slots.length(s) for s in slots]
        if max(n_new) == 1 and min(n_new) == 1:
            # one token each: only a sequence whose length is a multiple of the page size needs a page
            P = self.page_size
            pairs = [(s, l + 1) for s, l in zip(slots, lens) if l % P == 0]
            if not pairs:
                return
        else:
            pairs = [(s, l + n) for s, l, n in zip(slots, lens, n_new)]
        for g in self.groups:
            need = sum(g.pages_needed(s, l) for s, l in pairs)
            if need > g.n_free():
                raise CacheError(
                    f"the cache is full: this step needs {need} more pages of {self.page_size} tokens in the group of "
                    f"layers {g.layers}, {g.n_free()} are free (cache sized for {self.max_tokens} tokens)")
        for g in self.groups:
            for s, l in pairs:
                if g.pages_needed(s, l):
                    self.version += 1
                g.grow(s, l)

    def commit(self, slots: Sequence[int], n_new: Sequence[int]) -> None:
        P = self.page_size
        for s, n in zip(slots, n_new):
            self.slots.advance(s, n)
            length = self.slots.length(s)
            for g in self.groups:
                w = g.need.window
                # a page of a windowed group can only fall out of reach when the oldest key that the next
                # query needs has just moved onto a new page (one token) or moved at all (several)
                if w is None or length + 1 - w <= 0 or (n == 1 and (length + 1 - w) % P != 0):
                    continue
                if g.trim(s, length):
                    self.version += 1

    def block_table_rows(self, group: int, slots: Sequence[int], width: int) -> List[List[int]]:
        g = self.groups[group]
        rows = []
        for s in slots:
            tab = g.table(s)
            rows.append([max(p, 0) for p in tab[:width]] + [0] * (width - len(tab)))   # page 0: never handed out
        return rows

    def table_width(self, slots: Sequence[int]) -> int:
        return max((len(g.table(s)) for g in self.groups for s in slots), default=1) or 1

    def view(self, layer: int, block_tables: Sequence[torch.Tensor], *, read_from: Optional[int] = None) -> LayerCache:
        src = layer if read_from is None else read_from
        k = v = bt = None
        gi = None
        if src in self._where:
            gi, li = self._where[src]
            k, v, bt = self.groups[gi].k[li], self.groups[gi].v[li], block_tables[gi]
        return LayerCache(k=k, v=v, block_table=bt, writable=read_from is None,
                          state=self.state.get(src, {}), group=gi)

    def check_consistent(self) -> None:
        """No page lost, held twice, or both free and held (for tests)."""
        for g in self.groups:
            held = g.held_pages()
            if len(set(held)) != len(held):
                raise CacheError("a page is held twice")
            if set(held) & set(g._free):
                raise CacheError("a page is both free and held")
            if len(held) + len(g._free) != g.n_pages:
                raise CacheError(f"{g.n_pages - len(held) - len(g._free)} pages are lost")
        if len(self.slots.held()) + self.slots.n_free() != self.slots.n_slots:
            raise CacheError("a slot is lost")
