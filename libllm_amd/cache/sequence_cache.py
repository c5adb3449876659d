"""The cache of a model: a slot per live sequence, keys and values per cache entry, in pages.

* A *slot* is the identity of a live sequence: its length, one row of each group's page table and
  one row of each state tensor.  Slots are taken when a request starts and given back when it
  ends; a slot that is taken again starts at length 0 with zeroed state.
* A *group* collects the cache entries whose mixers keep the same things per token (the same
  planes, for all positions or for a window of them).  Each group has storage of its own: for
  every plane that the mixers asked for a tensor ``[entries, pages + 1, *page_shape]``, whose
  page shape is the mixer's business (attention keeps a plane of keys and one of values in the
  layouts its kernels read; another mixer may keep one latent row a token), and a table
  ``[slots + 1, pages_per_sequence]`` from (slot, position // page) to a page.  The last page and
  the last slot are a sink for padding rows and belong to nobody.
* Per-sequence *state* of fixed size: for each cache entry whose mixer asks for it, a tensor
  ``[slots + 1, *shape]``.

A page holds 64 positions.  A group that keeps a window gives pages back as soon as every
position in them lies behind the window of the sequence's next token.
"""
from typing import Dict, List, Optional

import numpy as np
import torch

from ..errors import CacheError
from ..parts.base import CacheNeed, CacheView, StateNeed
from .pages import PagePool, SlotTable

PAGE = 64


def pages_for(n_tokens: int, page: int = PAGE) -> int:
    return (n_tokens + page - 1) // page



def _send(t: torch.Tensor, device) -> torch.Tensor:
    """``t`` on ``device``.  To a GPU it goes through pinned memory and without waiting: a copy
    from pageable memory holds the host until the stream gets to it, and rows of the table change
    whenever a sequence enters a new page, which with unequal lengths is on most steps."""
    if torch.device(device).type == "cuda":
        return t.pin_memory().to(device, non_blocking=True)
    return t.to(device)

class CacheGroup:
    def __init__(self, need: CacheNeed, entries: List[int], n_pages: int, n_slots: int,
                 pages_per_seq: int, dtype, device):
        self.need = need
        self.entries = list(entries)
        self.index_of = {e: i for i, e in enumerate(self.entries)}
        self.pool = PagePool(n_pages)
        self.n_pages = n_pages
        self.sink_page = n_pages
        self.pages_per_seq = pages_per_seq
        self.planes = {}
        for plane in need.planes:
            if plane.name in self.planes:
                raise CacheError("a mixer names the plane %r twice" % plane.name)
            if any(int(n) <= 0 for n in plane.page_shape):
                raise CacheError("plane %r has the page shape %s" % (plane.name, tuple(plane.page_shape)))
            self.planes[plane.name] = torch.zeros((len(entries), n_pages + 1) + tuple(plane.page_shape),
                                                  dtype=plane.dtype or dtype, device=device)
        self.table_host = np.full((n_slots + 1, pages_per_seq), self.sink_page, dtype=np.int32)
        self.table = torch.from_numpy(self.table_host.copy()).to(device)
        self.held: Dict[int, Dict[int, int]] = {}      # slot -> {page index in sequence: page}
        self.dirty = set()

    def view(self, entry: int) -> CacheView:
        i = self.index_of[entry]
        return CacheView({name: t[i] for name, t in self.planes.items()}, self.table, PAGE, self.need)

    def first_needed(self, length_after: int) -> int:
        """Index of the first page a sequence still needs once it holds ``length_after`` tokens:
        the page of the oldest key that its next token may look at."""
        if self.need.kind != "window" or self.need.window <= 0:
            return 0
        oldest = max(0, length_after + 1 - self.need.window)
        return oldest // PAGE

    def pages_missing(self, slot: int, length: int, n_new: int) -> int:
        held = self.held.get(slot, {})
        lo = self.first_needed(length)
        hi = pages_for(length + n_new)
        return sum(1 for p in range(lo, hi) if p not in held)

    def reserve(self, slot: int, length: int, n_new: int) -> None:
        held = self.held.setdefault(slot, {})
        lo = self.first_needed(length)
        hi = pages_for(length + n_new)
        if hi > self.pages_per_seq:
            raise CacheError("a sequence of %d tokens exceeds the cache's limit of %d per sequence"
                             % (length + n_new, self.pages_per_seq * PAGE))
        want = [p for p in range(lo, hi) if p not in held]
        pages = self.pool.take(len(want))
        for p, page in zip(want, pages):
            held[p] = page
            self.table_host[slot, p] = page
        if want:
            self.dirty.add(slot)

    def trim(self, slot: int, length_after: int) -> None:
        """Gives back the pages that lie wholly behind the window."""
        held = self.held.get(slot)
        if not held:
            return
        first = self.first_needed(length_after)
        dead = [p for p in held if p < first]
        if dead:
            self.pool.give_back([held.pop(p) for p in dead])
            for p in dead:
                self.table_host[slot, p] = self.sink_page
            self.dirty.add(slot)

    def release(self, slot: int) -> None:
        held = self.held.pop(slot, {})
        self.pool.give_back(list(held.values()))
        self.table_host[slot, :] = self.sink_page
        self.dirty.add(slot)

    def flush(self) -> None:
        if not self.dirty:
            return
        rows = sorted(self.dirty)
        idx = _send(torch.tensor(rows, dtype=torch.long), self.table.device)
        data = _send(torch.from_numpy(self.table_host[rows]), self.table.device)
        self.table.index_copy_(0, idx, data)
        self.dirty.clear()


class SequenceCache:
    def __init__(self, needs: List[Optional[CacheNeed]], states: List[Optional[StateNeed]],
                 max_tokens: int, max_position: int, dtype, device, max_slots: Optional[int] = None):
        if max_tokens <= 0:
            raise CacheError("max_tokens must be positive")
        self.device = device
        self.dtype = dtype
        self.n_pages = pages_for(max_tokens)
        self.pages_per_seq = max(1, min(self.n_pages, pages_for(max_position)))
        self.max_position = max_position
        n_slots = self.n_pages if max_slots is None else min(max_slots, self.n_pages)
        self.slots = SlotTable(n_slots)
        self.sink_slot = n_slots
        self.lengths: Dict[int, int] = {}
        self.groups: List[CacheGroup] = []
        self.group_of: Dict[int, CacheGroup] = {}
        by_key: Dict[tuple, List[int]] = {}
        order = []
        for entry, need in enumerate(needs):
            if need is None:
                continue
            if need.key() not in by_key:
                by_key[need.key()] = []
                order.append(need)
            by_key[need.key()].append(entry)
        for need in order:
            g = CacheGroup(need, by_key[need.key()], self.n_pages, n_slots, self.pages_per_seq,
                           dtype, device)
            self.groups.append(g)
            for e in g.entries:
                self.group_of[e] = g
        self.state: Dict[int, torch.Tensor] = {}
        for entry, need in enumerate(states):
            if need is not None:
                self.state[entry] = torch.zeros((n_slots + 1,) + tuple(need.shape),
                                                dtype=need.dtype, device=device)

    # ---- requests
    def admit(self, request) -> int:
        slot = self.slots.acquire(request)
        self.lengths[slot] = 0
        for t in self.state.values():
            t[slot].zero_()
        return slot

    def slot_of(self, request) -> int:
        return self.slots.slot_of(request)

    def holds(self, request) -> bool:
        return self.slots.holds(request)

    def length(self, slot: int) -> int:
        return self.lengths[slot]

    def can_reserve(self, plan) -> bool:
        """``plan``: list of (slot or None for a request not yet admitted, length, n_new)."""
        for g in self.groups:
            need = 0
            for slot, length, n_new in plan:
                if slot is None:
                    need += pages_for(n_new)
                else:
                    need += g.pages_missing(slot, length, n_new)
            if need > g.pool.n_free:
                return False
        return True

    def reserve(self, slot: int, n_new: int) -> None:
        """Makes room for ``n_new`` more tokens of the slot's sequence in every group; all
        groups succeed or nothing changes."""
        length = self.lengths[slot]
        if length + n_new > self.max_position:
            raise CacheError("a sequence of %d tokens exceeds max_position_embeddings %d"
                             % (length + n_new, self.max_position))
        for g in self.groups:
            missing = g.pages_missing(slot, length, n_new)
            if missing > g.pool.n_free:
                raise CacheError("the cache is full: %d pages wanted, %d of %d free (max_tokens %d)"
                                 % (missing, g.pool.n_free, g.n_pages, self.n_pages * PAGE))
            if pages_for(length + n_new) > g.pages_per_seq:
                raise CacheError("a sequence of %d tokens exceeds the cache's limit of %d per sequence"
                                 % (length + n_new, g.pages_per_seq * PAGE))
        for g in self.groups:
            g.reserve(slot, length, n_new)

    def commit(self, slot: int, n_new: int) -> None:
        self.lengths[slot] += n_new
        for g in self.groups:
            g.trim(slot, self.lengths[slot])

    def release(self, request) -> None:
        slot = self.slots.release(request)
        for g in self.groups:
            g.release(slot)
        del self.lengths[slot]

    def flush(self) -> None:
        for g in self.groups:
            g.flush()

    # ---- views for a step
    def kv_view(self, entry: int) -> Optional[CacheView]:
        g = self.group_of.get(entry)
        return None if g is None else g.view(entry)

    def tokens_held(self) -> int:
        """Tokens the live requests hold, each rounded up to whole pages (largest group)."""
        return max((g.pool.n_held for g in self.groups), default=0) * PAGE

    def check(self) -> None:
        self.slots.check()
        live = set(self.slots.live().values())
        if live != set(self.lengths):
            raise CacheError("lengths are kept for slots that are not live, or the reverse")
        for g in self.groups:
            g.pool.check()
            held = [p for s in g.held.values() for p in s.values()]
            if len(held) != len(set(held)):
                raise CacheError("a page is held by two sequences")
            if len(held) != g.pool.n_held:
                raise CacheError("%d pages are held by the pool but %d by sequences"
                                 % (g.pool.n_held, len(held)))
            if not set(g.held) <= live:
                raise CacheError("pages are held for a slot that is not live")
