"""Page ids: who holds them, how many are promised, which are free.

Same contract as the reference's ``BlockAllocator`` (``serving/block_allocator.py:22-140``):
a min-heap of free ids (lowest id first), a reference count per page, and a
per-owner *reservation* (pages promised but not yet handed out) with the
invariant ``free - reserved >= 0``.  Beyond the reference:

* ``allocate`` also serves an owner whose reservation is used up (or was zero),
  from pages that nobody has been promised; trace replay allocates that way,
  because it does not know a request's length in advance.
* ``free_page`` gives one page back early (a window has passed it) and can put
  it back into the owner's reservation.
"""

from __future__ import annotations

import heapq
from typing import Dict, List, Set


class PageAllocator:
    def __init__(self, num_pages: int):
        if num_pages <= 0:
            raise ValueError(f"num_pages must be positive, got {num_pages}")
        self.num_pages = num_pages
        self._free: List[int] = list(range(num_pages))
        heapq.heapify(self._free)
        self._refs = [0] * num_pages
        self._reserved: Dict[int, int] = {}
        self._owned: Dict[int, Set[int]] = {}

    # -- counts ------------------------------------------------------------
    @property
    def free_pages(self) -> int:
        return len(self._free)

    @property
    def reserved_pages(self) -> int:
        return sum(self._reserved.values())

    @property
    def available_pages(self) -> int:
        """Free pages that are promised to nobody."""
        return self.free_pages - self.reserved_pages

    def ref_count(self, page: int) -> int:
        self._check_id(page)
        return self._refs[page]

    def owners(self):
        return list(self._owned)

    def pages_of(self, owner: int) -> Set[int]:
        return set(self._owned.get(owner, ()))

    # -- reservations ------------------------------------------------------
    def can_reserve(self, owner: int, count: int) -> bool:
        if owner in self._reserved:
            raise ValueError(f"owner {owner} already has a reservation")
        return 0 <= count <= self.available_pages

    def reserve(self, owner: int, count: int) -> None:
        if count < 0:
            raise ValueError(f"count must be non-negative, got {count}")
        if not self.can_reserve(owner, count):
            raise MemoryError(f"cannot reserve {count} pages for owner {owner}: {self.available_pages} remain")
        self._reserved[owner] = count
        self._owned[owner] = set()

    # -- pages -------------------------------------------------------------
    def allocate(self, owner: int) -> int:
        if owner not in self._reserved:
            raise KeyError(f"owner {owner} has no reservation")
        if self._reserved[owner] > 0:
            if not self._free:
                raise RuntimeError("reservation invariant violated: no free page for a reserved owner")
            self._reserved[owner] -= 1
        elif self.available_pages <= 0:
            raise MemoryError(f"owner {owner} has used its reservation and no unpromised page is free")
        page = heapq.heappop(self._free)
        self._refs[page] = 1
        self._owned[owner].add(page)
        return page

    def share(self, owner: int, page: int) -> None:
        """Adds an existing page to another owner (reference: ``incref``)."""
        self._check_id(page)
        if owner not in self._reserved:
            raise KeyError(f"owner {owner} has no reservation")
        if page in self._owned[owner]:
            raise ValueError(f"owner {owner} already holds page {page}")
        if self._refs[page] == 0:
            raise ValueError(f"cannot share free page {page}")
        self._refs[page] += 1
        self._owned[owner].add(page)

    def free_page(self, owner: int, page: int, back_to_reservation: bool = False) -> None:
        if owner not in self._owned or page not in self._owned[owner]:
            raise KeyError(f"owner {owner} does not hold page {page}")
        self._owned[owner].remove(page)
        self._decref(page)
        if back_to_reservation:
            if self.available_pages <= 0:
                raise RuntimeError("reservation invariant violated while returning a page to a reservation")
            self._reserved[owner] += 1

    def release(self, owner: int) -> None:
        """Drops every page and the reservation of an owner; unknown owners are ignored."""
        owned = self._owned.pop(owner, None)
        if owned is None:
            return
        for page in owned:
            self._decref(page)
        self._reserved.pop(owner)

    # -- checks ------------------------------------------------------------
    def check(self) -> None:
        """No page lost, none held twice by one owner, none free while held."""
        free = set(self._free)
        if len(free) != len(self._free):
            raise AssertionError("a page is in the free list twice")
        counts = [0] * self.num_pages
        for pages in self._owned.values():
            for p in pages:
                counts[p] += 1
        for p in range(self.num_pages):
            if counts[p] != self._refs[p]:
                raise AssertionError(f"page {p}: {counts[p]} holders but reference count {self._refs[p]}")
            if (p in free) != (self._refs[p] == 0):
                raise AssertionError(f"page {p}: free list and reference count disagree")
        if self.available_pages < 0:
            raise AssertionError("more pages promised than free")

    def _decref(self, page: int) -> None:
        self._refs[page] -= 1
        if self._refs[page] < 0:
            raise RuntimeError(f"page {page} freed twice")
        if self._refs[page] == 0:
            heapq.heappush(self._free, page)

    def _check_id(self, page: int) -> None:
        if not 0 <= page < self.num_pages:
            raise IndexError(f"page {page} outside [0, {self.num_pages})")
