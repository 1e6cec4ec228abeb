"""Reuse of the pages of equal prompt prefixes (what the reference's ``serving/radix_cache.py:30-194`` is for).

A prompt's complete pages form a chain: page ``i`` is identified by its own token ids together with
the identity of page ``i - 1``.  The cache is a flat table from ``(previous entry, token ids of a page)``
to an entry that pins one page of the pool (all slabs of it), so a request with an equal prefix takes
those pages by reference and nothing is copied.  A lookup covers complete pages only and always leaves
at least one prompt token to run, because the first new token needs logits.

What is dropped when admission needs pages, or when the cache outgrows ``capacity``, is the entry that
ends a chain (nothing continues it) and was used longest ago.  Such entries wait in a heap ordered by
their last use; the heap is cleaned lazily (an item is believed only if its entry still exists, still
ends a chain and has not been used since), so a lookup, an insertion and an eviction each cost a few
heap operations however many pages are cached.  A dropped page stays alive while a request still
holds it.

It needs a model whose layers all keep every key (one group, no window) and that has no per-request
state: a shared page must hold everything a later request needs of the prefix.
"""

from __future__ import annotations

import heapq
from typing import Dict, Iterable, List, Optional, Tuple

_ROOT = 0


class _Entry:
    __slots__ = ("uid", "page", "before", "edge", "continued_by", "used")

    def __init__(self, uid, page, before, edge, used):
        self.uid = uid                  # identity of the chain up to and including this page
        self.page = page
        self.before = before            # the entry of the page in front (None for a prompt's first page)
        self.edge = edge                # this entry's key in the table
        self.continued_by = 0           # entries that have this one in front of them
        self.used = used                # time of the last lookup or insertion that passed through


class PrefixCache:
    def __init__(self, cache, max_pages: int):
        if max_pages <= 0:
            raise ValueError(f"max_pages must be positive, got {max_pages}")
        if len(cache.groups) != 1 or cache.groups[0].need.window is not None or cache.layout.states:
            raise ValueError("prefix reuse needs one cache group without a window and no per-request state")
        self.pool = cache.groups[0].pool
        self.page_size = cache.page_size
        self.capacity = max_pages
        self._table: Dict[Tuple[int, Tuple[int, ...]], _Entry] = {}
        self._ends: List[Tuple[int, int]] = []     # heap of (last use, uid) of entries that may end a chain
        self._by_uid: Dict[int, _Entry] = {}
        self._uids = _ROOT
        self._now = 0
        self.counters = {"lookups": 0, "lookups_hit": 0, "tokens_reused": 0, "pages_dropped": 0}

    def __len__(self) -> int:
        return len(self._table)

    # -- the two ways in -----------------------------------------------------------------
    def _pages_of(self, tokens, n_tokens: int) -> Iterable[Tuple[int, ...]]:
        ps = self.page_size
        return (tuple(tokens[i:i + ps]) for i in range(0, n_tokens - ps + 1, ps))

    def _use(self, entry: _Entry) -> None:
        entry.used = self._now
        if not entry.continued_by:
            heapq.heappush(self._ends, (entry.used, entry.uid))
            if len(self._ends) > 4 * len(self._table) + 64:    # mostly stale items: start the heap afresh
                self._ends = [(e.used, e.uid) for e in self._table.values() if not e.continued_by]
                heapq.heapify(self._ends)

    def match(self, tokens) -> List[int]:
        """Pages of the longest cached chain that starts ``tokens``, at least one token left over."""
        self._now += 1
        self.counters["lookups"] += 1
        usable = (len(tokens) - 1) // self.page_size * self.page_size
        found: List[int] = []
        uid = _ROOT
        for ids in self._pages_of(tokens, usable):
            entry = self._table.get((uid, ids))
            if entry is None:
                break
            self._use(entry)
            found.append(entry.page)
            uid = entry.uid
        if found:
            self.counters["lookups_hit"] += 1
            self.counters["tokens_reused"] += len(found) * self.page_size
        return found

    def insert(self, tokens, page_table: List[int]) -> None:
        """Keeps every complete page of ``tokens`` whose keys and values are written; ``page_table[i]`` is the
        pool's page of positions ``i * page_size`` onwards."""
        self._now += 1
        whole = len(tokens) // self.page_size
        if len(page_table) < whole:
            raise ValueError(f"{whole} complete pages of tokens, but a table of {len(page_table)} pages")
        before: Optional[_Entry] = None
        for i, ids in enumerate(self._pages_of(tokens, whole * self.page_size)):
            edge = (before.uid if before else _ROOT, ids)
            entry = self._table.get(edge)
            if entry is None:
                self.pool.pin(page_table[i])      # raises for a page that nobody holds: nothing is recorded then
                self._uids += 1
                entry = _Entry(self._uids, page_table[i], before, edge, self._now)
                self._table[edge] = self._by_uid[entry.uid] = entry
                if before is not None:
                    before.continued_by += 1
            self._use(entry)
            before = entry
        while len(self._table) > self.capacity and self._drop_oldest_end(()):
            pass

    # -- the way out ---------------------------------------------------------------------
    def evict_until_available(self, required_pages: int, protected=()) -> bool:
        """Drops chain ends, oldest first and never a ``protected`` page, until the pool has ``required_pages``
        unpromised pages; False if it cannot get there."""
        protected = frozenset(protected)
        while self.pool.n_unpromised < required_pages:
            if not self._drop_oldest_end(protected):
                return False
        return True

    def _drop_oldest_end(self, protected) -> bool:
        spared = []
        victim = None
        while self._ends:
            used, uid = heapq.heappop(self._ends)
            entry = self._by_uid.get(uid)
            if entry is None or entry.continued_by or entry.used != used:
                continue                          # stale: dropped, continued or used again since
            if entry.page in protected:
                spared.append((used, uid))
                continue
            victim = entry
            break
        for item in spared:
            heapq.heappush(self._ends, item)
        if victim is None:
            return False
        self._forget(victim)
        self.counters["pages_dropped"] += 1
        if victim.before is not None:
            victim.before.continued_by -= 1
            if not victim.before.continued_by:    # it ends a chain now, with the age it has
                heapq.heappush(self._ends, (victim.before.used, victim.before.uid))
        return True

    def _forget(self, entry: _Entry) -> None:
        del self._table[entry.edge]
        del self._by_uid[entry.uid]
        self.pool.unpin(entry.page)

    def clear(self) -> None:
        for entry in list(self._table.values()):
            self._forget(entry)
        self._ends.clear()
        for key in self.counters:
            self.counters[key] = 0

    def stats(self) -> Dict[str, int]:
        return {"pages": len(self._table), "tokens": len(self._table) * self.page_size, **self.counters}
