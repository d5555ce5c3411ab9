"""The cache: a slot for each live sequence, pages of keys and values for each
group of layers, each sequence's own length, and fixed-size state per sequence.

Storage is paged (64 tokens a page) so that the cache is sized by the tokens that
live sequences hold, not by slots times the longest context.  A group owns one
pool ``[pages, layers of the group, K part + V part]`` and one page table
``[slots, pages per sequence]``; inside a page keys and values lie in the order in
which the attention kernels feed the matrix cores.  Pages are zeroed when handed
out, so nothing of an earlier sequence can be read.  A group with a window gives
pages back once all their tokens have left the window.

One row more than there are slots lies behind every per-slot table (page tables, lengths, sampling state,
state groups): the scratch slot, ``Cache.scratch_slot``, which is never handed out.  Its page-table entries
all point at the null page and its length stays 0.  A recorded decode step that runs more rows than there
are live sequences (its batch size rounded up to a bucket) lets the idle rows work on that slot: they write
and read the null page, which no live sequence ever reads, and change nothing else.

The reference keeps one contiguous cache per layer for a single sequence
(src/model/block.cpp:71-74) and has no per-sequence state beyond the position the
caller passes (src/model/model.cpp:66-68).
"""
from __future__ import annotations

from dataclasses import dataclass

import numpy as np
import torch

from ..tensor import Tensor
from .slots import CacheError, PagePool, SlotAllocator
from .specs import KVSpec, StateSpec

PAGE = 64
NULL_PAGE = 0


def _round_up(a: int, b: int) -> int:
    return (a + b - 1) // b * b


@dataclass
class KVView:
    """What an attention layer sees of its group: its own part of every page."""
    k: torch.Tensor            # flat view starting at this layer's keys of page 0
    v: torch.Tensor
    page_stride: int           # elements from one page to the next
    page_table: torch.Tensor   # int32 [slots, pages per sequence]
    spec: KVSpec
    round_to: torch.dtype | None = None   # keys and values take this type's values before they are stored

    def as_tuple(self):
        return (self.k, self.v, self.page_stride, self.page_table)


@dataclass
class StateView:
    state: torch.Tensor        # [slots, *shape]
    spec: StateSpec


class KVGroup:
    def __init__(self, spec: KVSpec, entries, n_slots, n_pages, max_positions, dtype, device, round_to=None):
        self.spec, self.entries, self.round_to = spec, list(entries), round_to
        self.k_elems = spec.n_kv_heads * PAGE * spec.head_dim
        self.v_elems = spec.n_kv_heads * PAGE * _round_up(spec.head_dim, 32)
        self.layer_elems = self.k_elems + self.v_elems
        self.page_elems = self.layer_elems * len(self.entries)
        self.n_pages = n_pages
        self.max_pages = (max_positions + PAGE - 1) // PAGE
        self.pool = PagePool(n_pages, first=1)
        self.table_host = np.zeros((n_slots, self.max_pages), dtype=np.int32)
        self.pages_of = [dict() for _ in range(n_slots)]            # slot -> {page index in sequence: page}
        self.device, self.dtype = device, dtype
        self._views = {}
        if device is not None:
            self.storage = Tensor.zeros((n_pages, self.page_elems), dtype, device)
            # (one row more: the scratch slot's, all null pages)
            self.page_table = Tensor.zeros((n_slots + 1, self.max_pages), torch.int32, device)
        else:
            self.storage = self.page_table = None

    def bytes_per_token(self) -> int:
        return self.page_elems // PAGE * torch.empty((), dtype=self.dtype).element_size()

    def view(self, entry: int) -> KVView:
        view = self._views.get(entry)
        if view is None:                # the storage never moves: a view is made once
            i = self.entries.index(entry)
            flat = self.storage.view(-1)
            k = flat[i * self.layer_elems:]
            v = flat[i * self.layer_elems + self.k_elems:]
            view = self._views[entry] = KVView(k, v, self.page_elems, self.page_table, self.spec, self.round_to)
        return view

    def first_needed_page(self, length: int) -> int:
        """First page that a token at position ``length`` (the next one) still reads."""
        if self.spec.window is None:
            return 0
        return max(0, length - self.spec.window + 1) // PAGE

    def reserve(self, slot: int, old_len: int, new_len: int, dirty: set, fresh: list, filled: bool = False) -> None:
        have = self.pages_of[slot]
        lo = self.first_needed_page(old_len) if self.spec.window is not None else 0
        want = range(lo, (new_len + PAGE - 1) // PAGE)
        need = [p for p in want if p not in have]
        if not need:
            return
        got = self.pool.alloc(len(need))
        for p, page in zip(need, got):
            have[p] = page
            self.table_host[slot, p] = page
            # a page that the caller fills from its first to its last token needs no clearing: only
            # what stays unwritten could reach a product as 0 x garbage
            if not (filled and old_len <= p * PAGE and new_len >= (p + 1) * PAGE):
                fresh.append(page)
        dirty.add(slot)

    def release_outside_window(self, slot: int, length: int, dirty: set) -> None:
        if self.spec.window is None:
            return
        first = self.first_needed_page(length)
        have = self.pages_of[slot]
        gone = [p for p in have if p < first]
        if gone:
            self.pool.free([have.pop(p) for p in gone])
            for p in gone:
                self.table_host[slot, p] = NULL_PAGE
            dirty.add(slot)

    def release_from(self, slot: int, length: int, dirty: set) -> None:
        """Gives back the pages that a sequence of ``length`` tokens does not reach."""
        have = self.pages_of[slot]
        gone = [p for p in have if p * PAGE >= length]
        if gone:
            self.pool.free([have.pop(p) for p in gone])
            for p in gone:
                self.table_host[slot, p] = NULL_PAGE
            dirty.add(slot)

    def release(self, slot: int) -> None:
        have = self.pages_of[slot]
        self.pool.free(list(have.values()))
        have.clear()
        self.table_host[slot, :] = NULL_PAGE

    def flush(self, dirty: set, fresh: list) -> None:
        if self.storage is None:
            return
        if fresh:
            idx = torch.tensor(sorted(fresh), dtype=torch.int64, device=self.device)
            self.storage.index_fill_(0, idx, 0)
        if dirty:
            rows = sorted(dirty)
            idx = torch.tensor(rows, dtype=torch.int64, device=self.device)
            self.page_table.index_copy_(0, idx, torch.from_numpy(self.table_host[rows]).to(self.device))


class StateGroup:
    def __init__(self, spec: StateSpec, entries, n_slots, device):
        self.spec, self.entries = spec, list(entries)
        self.device = device
        dtype = getattr(torch, spec.dtype)
        self.storage = None
        if device is not None:
            self.storage = Tensor.zeros((len(self.entries), n_slots + 1) + tuple(spec.shape), dtype, device)

    def view(self, entry: int) -> StateView:
        return StateView(self.storage[self.entries.index(entry)], self.spec)

    def reset(self, slots) -> None:
        if self.storage is not None and slots:
            idx = torch.tensor(sorted(slots), dtype=torch.int64, device=self.device)
            self.storage.index_fill_(1, idx, 0)


class Cache:
    """``specs[i]`` is what unit i asks for (a unit: one mixer of one run of a layer; None: it keeps no
    cache of its own).
    ``max_tokens`` bounds the tokens all live sequences hold together, each sequence's count
    rounded up to a whole page."""

    def __init__(self, specs, max_tokens: int, max_positions: int, dtype, device, n_slots: int | None = None,
                 kv_round=None):
        if kv_round is not None and (dtype != torch.float32 or kv_round not in (torch.float16, torch.bfloat16)):
            raise CacheError("kv_round: float16 or bfloat16, for a float32 cache (a 16-bit cache rounds to its own type)")
        self.max_positions = max_positions
        self.n_pages = max(1, (max_tokens + PAGE - 1) // PAGE) + 1          # page 0 is never handed out
        self.n_slots = n_slots or max(1, min(self.n_pages - 1, 4096))
        self.device, self.dtype = device, dtype
        self.slots = SlotAllocator(self.n_slots)
        self.scratch_slot = self.n_slots          # behind the last slot in every per-slot table; never handed out
        self.lens = [0] * self.n_slots
        self.groups = []
        self._group_of = {}
        by_spec = {}
        for i, s in enumerate(specs):
            if s is not None:
                by_spec.setdefault(s, []).append(i)
        for s, entries in by_spec.items():
            if isinstance(s, KVSpec):
                g = KVGroup(s, entries, self.n_slots, self.n_pages, max_positions, dtype, device, kv_round)
            elif isinstance(s, StateSpec):
                g = StateGroup(s, entries, self.n_slots, device)
            else:
                raise CacheError(f"unknown cache request {s!r}")
            self.groups.append(g)
            for e in entries:
                self._group_of[e] = g
        if device is not None:
            self.lens_dev = Tensor.zeros((self.n_slots + 1,), torch.int32, device)
            # fixed-size state of every sequence: key and counter of its sampling generator
            self.seq_state = Tensor.zeros((self.n_slots + 1, 2), torch.int64, device)
        else:
            self.lens_dev = self.seq_state = None

    # -- sequences ---------------------------------------------------------
    def alloc_slot(self) -> int:
        s = self.slots.alloc()
        self.lens[s] = 0
        for g in self.groups:
            if isinstance(g, StateGroup):
                g.reset([s])
        if self.lens_dev is not None:
            self.lens_dev[s] = 0
        return s

    def free_slot(self, slot: int) -> None:
        self.slots.free(slot)
        for g in self.groups:
            if isinstance(g, KVGroup):
                g.release(slot)
        self.lens[slot] = 0

    def grow(self, slots, new_lens, sync_lens: bool = True, filled: bool = False) -> None:
        """Make room for each slot to reach its new length, then record the lengths.  All page
        tables and fresh pages are updated with one small copy and one fill per group.
        ``filled``: the caller writes every position between the old and the new length before
        anything reads the cache (a step does), so pages that lie wholly in between are not cleared."""
        for slot, n in zip(slots, new_lens):
            if n > self.max_positions:
                raise CacheError(f"a sequence of {n} tokens exceeds the model's {self.max_positions} positions")
            if slot not in self.slots._held:
                raise CacheError(f"slot {slot} is not held")
        for g in self.groups:
            if not isinstance(g, KVGroup):
                continue
            dirty, fresh = set(), []
            try:
                for slot, n in zip(slots, new_lens):
                    g.reserve(slot, self.lens[slot], n, dirty, fresh, filled)
            finally:
                g.flush(dirty, fresh)
        for slot, n in zip(slots, new_lens):
            self.lens[slot] = n
        if sync_lens and self.lens_dev is not None and slots:
            idx = torch.tensor(list(slots), dtype=torch.int64, device=self.device)
            self.lens_dev.index_copy_(0, idx, torch.tensor(list(new_lens), dtype=torch.int32, device=self.device))

    def truncate(self, slots, lens) -> None:
        """Takes sequences back to earlier lengths (a step that failed after ``grow``): the lengths are
        restored and the pages beyond them given back, so that a later step finds them cleared or fills
        them itself.  State groups are not restored: what a mixer has already written into its state stays."""
        for g in self.groups:
            if isinstance(g, KVGroup):
                dirty = set()
                for slot, n in zip(slots, lens):
                    g.release_from(slot, n, dirty)
                g.flush(dirty, [])
        for slot, n in zip(slots, lens):
            self.lens[slot] = n
        if self.lens_dev is not None and slots:
            idx = torch.tensor(list(slots), dtype=torch.int64, device=self.device)
            self.lens_dev.index_copy_(0, idx, torch.tensor(list(lens), dtype=torch.int32, device=self.device))

    def trim_windows(self, slots) -> None:
        for g in self.groups:
            if isinstance(g, KVGroup) and g.spec.window is not None:
                dirty = set()
                for s in slots:
                    g.release_outside_window(s, self.lens[s], dirty)
                g.flush(dirty, [])

    # -- what the parts see --------------------------------------------------
    def view(self, entry: int):
        g = self._group_of.get(entry)
        return None if g is None else g.view(entry)

    def tokens_free(self) -> int:
        kv = [g for g in self.groups if isinstance(g, KVGroup)]
        return min((g.pool.n_free for g in kv), default=self.n_pages - 1) * PAGE

    def bytes_per_token(self) -> int:
        return sum(g.bytes_per_token() for g in self.groups if isinstance(g, KVGroup))
