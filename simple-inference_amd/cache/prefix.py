"""Reuse of the pages of equal prompt prefixes (what the reference's ``serving/radix_cache.py:30-194`` is for).

A prompt's complete pages form a chain, and a chain is known by a running digest: the digest of the
first ``i`` pages is a hash of the digest of the first ``i - 1`` and the token ids of page ``i``.  The
cache is one table from digest to the pool page that holds such a prefix's last page of keys and
values (all slabs of it), pinned in the pool, so a request with an equal prefix takes those pages by
reference and nothing is copied.  An entry remembers its page's token ids and the digest in front of
it, and a lookup believes a digest only if both agree, so two chains that happen to hash alike are
told apart.  A lookup covers complete pages only and always leaves at least one prompt token to run,
because the first new token needs logits.

What goes when admission needs pages, or when the cache outgrows ``capacity``, is the entry that ends
a chain (nothing continues it) and was used longest ago.  Candidates wait in a heap ordered by the
time of their last use; a heap item is believed only if its entry still exists, still ends a chain
and has not been used since, so a lookup, an insertion and an eviction each cost a few heap
operations however many pages are cached.  A page that goes stays alive while a request holds it.

It needs a model whose layers all keep every key (one group, no window) and that has no per-request
state: a shared page must hold everything a later request needs of the prefix.
"""

from __future__ import annotations

import heapq
from typing import Dict, Iterator, List, Optional, Sequence, Tuple

_NOTHING = 0          # the digest of the empty prefix


def _extend(digest: int, ids: Tuple[int, ...]) -> int:
    """The digest of a prefix one page longer."""
    return hash((digest, ids)) or 1     # never the digest of the empty prefix


class _Held:
    """One cached page: the last page of the prefix whose digest is its key in the table."""

    __slots__ = ("page", "ids", "front", "heirs", "stamp")

    def __init__(self, page: int, ids: Tuple[int, ...], front: int, stamp: int):
        self.page = page        # the pool's page
        self.ids = ids          # its token ids
        self.front = front      # digest of the prefix without this page
        self.heirs = 0          # cached pages that continue this prefix
        self.stamp = stamp      # time of the last lookup or insertion that passed through


class PrefixCache:
    def __init__(self, cache, max_pages: int):
        if max_pages <= 0:
            raise ValueError(f"max_pages must be positive, got {max_pages}")
        if len(cache.groups) != 1 or cache.groups[0].need.window is not None or cache.layout.states:
            raise ValueError("prefix reuse needs one cache group without a window and no per-request state")
        self.pool = cache.groups[0].pool
        self.page_size = cache.page_size
        self.capacity = max_pages
        self._known: Dict[int, _Held] = {}
        self._ends: List[Tuple[int, int]] = []     # heap of (stamp, digest): entries that may end a chain
        self._tick = 0
        self._lookups = self._hits = self._reused = self._dropped = 0

    def __len__(self) -> int:
        return len(self._known)

    def stats(self) -> Dict[str, int]:
        held = len(self._known)
        return {"pages": held, "tokens": held * self.page_size, "lookups": self._lookups,
                "lookups_hit": self._hits, "tokens_reused": self._reused, "pages_dropped": self._dropped}

    # -- making room ---------------------------------------------------------------------
    def evict_until_available(self, required_pages: int, protected=()) -> bool:
        """Lets chain ends go, oldest first and never a ``protected`` page, until the pool has ``required_pages``
        unpromised pages; False if it cannot get there."""
        spared = frozenset(protected)
        while self.pool.n_unpromised < required_pages:
            if not self._let_oldest_end_go(spared):
                return False
        return True

    def clear(self) -> None:
        for digest in list(self._known):
            self._unpin(digest)
        del self._ends[:]
        self._lookups = self._hits = self._reused = self._dropped = 0

    def _let_oldest_end_go(self, spared) -> bool:
        passed_over = []
        gone: Optional[_Held] = None
        while self._ends and gone is None:
            stamp, digest = heapq.heappop(self._ends)
            held = self._known.get(digest)
            if held is None or held.heirs or held.stamp != stamp:
                continue                            # stale: gone, continued, or used again since
            if held.page in spared:
                passed_over.append((stamp, digest))
                continue
            gone = self._unpin(digest)
        for item in passed_over:
            heapq.heappush(self._ends, item)
        if gone is None:
            return False
        self._dropped += 1
        front = self._known.get(gone.front)
        if front is not None:
            front.heirs -= 1
            if front.heirs == 0:                    # it ends a chain now, as old as it is
                heapq.heappush(self._ends, (front.stamp, gone.front))
        return True

    def _unpin(self, digest: int) -> _Held:
        held = self._known.pop(digest)
        self.pool.unpin(held.page)
        return held

    # -- looking up and taking in ----------------------------------------------------------
    def _chain(self, tokens: Sequence[int], n_pages: int) -> Iterator[Tuple[int, int, Tuple[int, ...]]]:
        """(digest in front, digest, token ids) of each of the first ``n_pages`` pages of ``tokens``."""
        front, size = _NOTHING, self.page_size
        for first in range(0, n_pages * size, size):
            ids = tuple(tokens[first:first + size])
            digest = _extend(front, ids)
            yield front, digest, ids
            front = digest

    def _seen(self, held: _Held, digest: int) -> None:
        held.stamp = self._tick
        if held.heirs:
            return
        heapq.heappush(self._ends, (held.stamp, digest))
        if len(self._ends) > 4 * len(self._known) + 64:     # mostly stale items: start the heap afresh
            self._ends = [(h.stamp, d) for d, h in self._known.items() if not h.heirs]
            heapq.heapify(self._ends)

    def match(self, tokens) -> List[int]:
        """Pages of the longest cached chain that starts ``tokens``, at least one token left over."""
        self._tick += 1
        self._lookups += 1
        pages: List[int] = []
        for front, digest, ids in self._chain(tokens, (len(tokens) - 1) // self.page_size):
            held = self._known.get(digest)
            if held is None or held.front != front or held.ids != ids:
                break
            self._seen(held, digest)
            pages.append(held.page)
        if pages:
            self._hits += 1
            self._reused += self.page_size * len(pages)
        return pages

    def insert(self, tokens, page_table: List[int]) -> None:
        """Keeps every complete page of ``tokens`` whose keys and values are written; ``page_table[i]`` is the
        pool's page of positions ``i * page_size`` onwards."""
        whole = len(tokens) // self.page_size
        if whole > len(page_table):
            raise ValueError(f"{whole} complete pages of tokens, but a table of {len(page_table)} pages")
        self._tick += 1
        for i, (front, digest, ids) in enumerate(self._chain(tokens, whole)):
            held = self._known.get(digest)
            if held is not None and (held.front != front or held.ids != ids):
                break             # another chain with this digest is cached: this one stays out from here on
            if held is None:
                self.pool.pin(page_table[i])      # raises for a page that nobody holds: nothing is recorded then
                held = self._known[digest] = _Held(page_table[i], ids, front, self._tick)
                if front != _NOTHING:
                    self._known[front].heirs += 1
            self._seen(held, digest)
        while len(self._known) > self.capacity and self._let_oldest_end_go(frozenset()):
            pass
