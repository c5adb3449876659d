"""Host-side bookkeeping of the cache: a pool of pages and a table of slots.

Both are plain Python and know nothing of devices; every misuse (taking more than is free,
giving back what is not held, holding twice) raises CacheError and leaves the books unchanged.
"""
from typing import Dict, Hashable, List

from ..errors import CacheError


class PagePool:
    """``n_pages`` pages, handed out lowest index first so that reuse is easy to follow."""

    def __init__(self, n_pages: int):
        if n_pages <= 0:
            raise CacheError("a page pool needs at least one page")
        self.n_pages = n_pages
        self._free: List[int] = list(range(n_pages - 1, -1, -1))   # pop() yields the lowest
        self._held = [False] * n_pages

    @property
    def n_free(self) -> int:
        return len(self._free)

    @property
    def n_held(self) -> int:
        return self.n_pages - len(self._free)

    def take(self, n: int) -> List[int]:
        if n < 0:
            raise CacheError("cannot take %d pages" % n)
        if n > len(self._free):
            raise CacheError("the cache is full: %d pages wanted, %d of %d free"
                             % (n, len(self._free), self.n_pages))
        pages = [self._free.pop() for _ in range(n)]
        for p in pages:
            self._held[p] = True
        return pages

    def give_back(self, pages: List[int]) -> None:
        pages = list(pages)
        seen = set()
        for p in pages:
            if not 0 <= p < self.n_pages or not self._held[p] or p in seen:
                raise CacheError("page %r is given back but not held" % (p,))
            seen.add(p)
        for p in pages:
            self._held[p] = False
        self._free.extend(sorted(pages, reverse=True))
        self._free.sort(reverse=True)

    def check(self) -> None:
        """Every page is either free or held, exactly once."""
        free = set(self._free)
        if len(free) != len(self._free):
            raise CacheError("a page is on the free list twice")
        for p in range(self.n_pages):
            if self._held[p] == (p in free):
                raise CacheError("page %d is %s" % (p, "lost" if not self._held[p] else "held and free"))


class SlotTable:
    """Maps live requests to slots ``0 .. n_slots-1``; a slot belongs to one request at a time."""

    def __init__(self, n_slots: int):
        if n_slots <= 0:
            raise CacheError("a slot table needs at least one slot")
        self.n_slots = n_slots
        self._free: List[int] = list(range(n_slots - 1, -1, -1))
        self._slot_of: Dict[Hashable, int] = {}
        self._owner: List[object] = [None] * n_slots

    @property
    def n_free(self) -> int:
        return len(self._free)

    def live(self):
        return dict(self._slot_of)

    def holds(self, request) -> bool:
        return request in self._slot_of

    def slot_of(self, request) -> int:
        if request not in self._slot_of:
            raise CacheError("request %r holds no slot" % (request,))
        return self._slot_of[request]

    def acquire(self, request) -> int:
        if request in self._slot_of:
            raise CacheError("request %r already holds slot %d" % (request, self._slot_of[request]))
        if not self._free:
            raise CacheError("no free slot: all %d are held" % self.n_slots)
        slot = self._free.pop()
        self._slot_of[request] = slot
        self._owner[slot] = request
        return slot

    def release(self, request) -> int:
        if request not in self._slot_of:
            raise CacheError("request %r is released but holds no slot" % (request,))
        slot = self._slot_of.pop(request)
        self._owner[slot] = None
        self._free.append(slot)
        self._free.sort(reverse=True)
        return slot

    def check(self) -> None:
        free = set(self._free)
        if len(free) != len(self._free):
            raise CacheError("a slot is on the free list twice")
        held = set(self._slot_of.values())
        if len(held) != len(self._slot_of):
            raise CacheError("a slot is held by two requests")
        if free & held or len(free) + len(held) != self.n_slots:
            raise CacheError("slots lost or both free and held")
