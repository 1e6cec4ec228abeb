"""The pool of page ids of one cache group: who holds which page, and what is promised to whom.

The contract is that of the reference's block allocator (``serving/block_allocator.py:22-140``):
pages are handed out lowest id first, a page may have several holders and is free again when the
last one lets go, and an owner can be *promised* pages in advance, which nobody else can then take
(the pool never promises more than it has free).  The bookkeeping is this package's own:

* Ids that were never handed out lie above a watermark; only ids that came back are kept in a
  heap.  A pool of hundreds of thousands of pages costs nothing to set up, and "lowest first"
  holds because every id below the watermark that is free is in the heap.
* Owners have *accounts* (``open`` .. ``close``).  An account whose promise is used up, or that
  was opened without one, may still ``take`` pages that are promised to nobody: trace replay
  works that way, because it does not know a request's length in advance.
* A page can also be held without an account (``pin`` / ``unpin``): the prefix cache keeps
  pages alive that way after the request that wrote them has gone.
* ``drop`` gives one page back early (a window has passed it) and can turn it back into a
  promise, so that a windowed request can never run dry.
"""

from __future__ import annotations

import heapq
from typing import Dict, FrozenSet, List, Set


class OutOfPages(MemoryError):
    """The pool cannot promise or hand out what was asked."""


class _Account:
    __slots__ = ("promised", "pages")

    def __init__(self, promised: int):
        self.promised = promised      # pages this owner may still take for certain
        self.pages: Set[int] = set()


class PagePool:
    def __init__(self, num_pages: int):
        if num_pages <= 0:
            raise ValueError(f"a pool needs at least one page, got {num_pages}")
        self.num_pages = num_pages
        self._fresh = 0                      # ids at or above it were never handed out
        self._returned: List[int] = []       # heap of free ids below the watermark
        self._held: Dict[int, int] = {}      # page in use -> accounts plus pins holding it
        self._pins: Dict[int, int] = {}
        self._accounts: Dict[int, _Account] = {}
        self._promised = 0                   # sum of the accounts' open promises

    # -- pages ---------------------------------------------------------------------------
    def take(self, owner: int) -> int:
        """The lowest free page, against the owner's promise while it lasts, else from the unpromised ones."""
        acct = self._account(owner)
        if acct.promised:
            if not self.n_free:
                raise RuntimeError("a promised page is missing: more was promised than is free")
            acct.promised -= 1
            self._promised -= 1
        elif self.n_unpromised <= 0:
            raise OutOfPages(f"owner {owner} holds no promise and every free page is promised to someone")
        page = heapq.heappop(self._returned) if self._returned else self._next_fresh()
        self._held[page] = 1
        acct.pages.add(page)
        return page

    def take_many(self, owner: int, n: int) -> List[int]:
        """``take`` n times (a long prompt's first step takes a hundred pages and more): the same pages in the same
        order; if there are not n for this owner, the error that the first missing one would have raised, and none
        is taken."""
        acct = self._account(owner)
        against_promise = min(n, acct.promised)
        if against_promise > self.n_free:
            raise RuntimeError("a promised page is missing: more was promised than is free")
        if n - against_promise > self.n_unpromised:
            raise OutOfPages(f"owner {owner} holds no promise and every free page is promised to someone")
        acct.promised -= against_promise
        self._promised -= against_promise
        held, returned, mine, taken = self._held, self._returned, acct.pages, []
        for _ in range(n):
            page = heapq.heappop(returned) if returned else self._next_fresh()
            held[page] = 1
            mine.add(page)
            taken.append(page)
        return taken

    def _next_fresh(self) -> int:
        self._fresh += 1
        return self._fresh - 1

    def adopt(self, owner: int, page: int) -> None:
        """Makes the owner one more holder of a page that is in use (the reference's ``incref``)."""
        acct = self._account(owner)
        if page in acct.pages:
            raise ValueError(f"owner {owner} holds page {page} already")
        self._hold_once_more(page, "adopted")
        acct.pages.add(page)

    def drop(self, owner: int, page: int, restore_promise: bool = False) -> None:
        """The owner lets go of one page; with ``restore_promise`` it may take one page more for certain later."""
        acct = self._accounts.get(owner)
        if acct is None or page not in acct.pages:
            raise KeyError(f"owner {owner} does not hold page {page}")
        acct.pages.discard(page)
        self._let_go(page)
        if restore_promise:
            if self.n_unpromised <= 0:
                raise RuntimeError("no unpromised page is left to turn back into a promise")
            acct.promised += 1
            self._promised += 1

    def pin(self, page: int) -> None:
        """One more holder of a page in use, outside every account."""
        self._hold_once_more(page, "pinned")
        self._pins[page] = self._pins.get(page, 0) + 1

    def unpin(self, page: int) -> None:
        left = self._pins.get(self._valid(page), 0) - 1
        if left < 0:
            raise KeyError(f"page {page} is not pinned")
        if left:
            self._pins[page] = left
        else:
            del self._pins[page]
        self._let_go(page)

    def _hold_once_more(self, page: int, how: str) -> None:
        if self._valid(page) not in self._held:
            raise ValueError(f"page {page} is free and cannot be {how}")
        self._held[page] += 1

    def _let_go(self, page: int) -> None:
        count = self._held.get(page, 0) - 1
        if count < 0:
            raise RuntimeError(f"page {page} was given back more often than it was taken")
        if count:
            self._held[page] = count
        else:
            del self._held[page]
            heapq.heappush(self._returned, page)

    # -- accounts ------------------------------------------------------------------------
    def open(self, owner: int, promise: int = 0) -> None:
        if owner in self._accounts:
            raise ValueError(f"owner {owner} has an account already")
        if promise < 0:
            raise ValueError(f"a promise cannot be negative ({promise})")
        if promise > self.n_unpromised:
            raise OutOfPages(f"{promise} pages cannot be promised to owner {owner}: {self.n_unpromised} are unpromised")
        self._accounts[owner] = _Account(promise)
        self._promised += promise

    def close(self, owner: int) -> None:
        """Lets go of every page of the owner and of what is left of its promise; an unknown owner is ignored."""
        acct = self._accounts.pop(owner, None)
        if acct is None:
            return
        self._promised -= acct.promised
        for page in acct.pages:
            self._let_go(page)

    def has(self, owner: int) -> bool:
        return owner in self._accounts

    def owners(self) -> List[int]:
        return list(self._accounts)

    def pages(self, owner: int) -> FrozenSet[int]:
        acct = self._accounts.get(owner)
        return frozenset(acct.pages) if acct else frozenset()

    def _account(self, owner: int) -> _Account:
        try:
            return self._accounts[owner]
        except KeyError:
            raise KeyError(f"owner {owner} has no account") from None

    # -- counts --------------------------------------------------------------------------
    @property
    def n_free(self) -> int:
        return self.num_pages - len(self._held)

    @property
    def n_promised(self) -> int:
        return self._promised

    @property
    def n_unpromised(self) -> int:
        """Free pages that nobody has been promised."""
        return self.n_free - self._promised

    def fits(self, promise: int) -> bool:
        return 0 <= promise <= self.n_unpromised

    def holders(self, page: int) -> int:
        return self._held.get(self._valid(page), 0)

    def _valid(self, page: int) -> int:
        if not 0 <= page < self.num_pages:
            raise IndexError(f"page {page} is outside [0, {self.num_pages})")
        return page

    # -- checks --------------------------------------------------------------------------
    def audit(self) -> None:
        """Every page is free or held, exactly as often as its count says; nothing is promised that is not there."""
        free = set(self._returned) | set(range(self._fresh, self.num_pages))
        if len(free) != len(self._returned) + self.num_pages - self._fresh or any(p >= self._fresh for p in self._returned):
            raise AssertionError("a page is in the free set twice")
        seen = dict(self._pins)
        for acct in self._accounts.values():
            for p in acct.pages:
                seen[p] = seen.get(p, 0) + 1
        if seen != self._held:
            odd = sorted(set(seen) ^ set(self._held) | {p for p in seen if seen[p] != self._held.get(p)})
            raise AssertionError(f"pages {odd[:8]} are not held as often as their counts say")
        if free & set(self._held) or len(free) + len(self._held) != self.num_pages:
            raise AssertionError("a page is both free and held, or neither")
        if self._promised != sum(a.promised for a in self._accounts.values()) or self.n_unpromised < 0:
            raise AssertionError("the promises do not add up")
