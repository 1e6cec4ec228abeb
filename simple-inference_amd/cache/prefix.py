"""Reuse of the pages of equal prompt prefixes (reference: ``serving/radix_cache.py:30-194``).

A tree keyed by complete pages of token ids; each node pins one page (all slabs of it) through an
owner of its own in the page allocator, so a request that shares a prefix takes the pages by
reference and nothing is copied.  A match covers complete pages only and leaves at least one
prompt token to run (``((len - 1) // page) * page``), because the first new token needs logits.
Least recently used leaves are dropped when admission needs their pages or the cache outgrows
``max_pages``; a page stays alive while any request still holds it.

It needs a model whose layers all keep every key (one group, no window) and that has no
per-request state: a shared page must hold everything a later request needs of the prefix.
"""

from __future__ import annotations

from typing import Dict, List, Optional, Set, Tuple


class _Node:
    __slots__ = ("key", "page", "owner", "parent", "children", "last_used")

    def __init__(self, key=None, page=None, owner=None, parent=None):
        self.key, self.page, self.owner, self.parent = key, page, owner, parent
        self.children: Dict[Tuple[int, ...], "_Node"] = {}
        self.last_used = 0


class PrefixCache:
    def __init__(self, cache, max_pages: int):
        if max_pages <= 0:
            raise ValueError(f"max_pages must be positive, got {max_pages}")
        if len(cache.groups) != 1 or cache.groups[0].need.window is not None or cache.layout.states:
            raise ValueError("prefix reuse needs one cache group without a window and no per-request state")
        self.cache = cache
        self.allocator = cache.groups[0].allocator
        self.page_size = cache.page_size
        self.max_pages = max_pages
        self.root = _Node()
        self.cached_pages = 0
        self.hits = self.misses = self.matched_tokens = self.evictions = 0
        self._clock = 0
        self._next_owner = -1

    def _touch(self, node: _Node) -> None:
        self._clock += 1
        node.last_used = self._clock

    def match(self, tokens) -> List[int]:
        """Pages of the longest cached prefix of ``tokens`` (complete pages, at least one token left over)."""
        ps = self.page_size
        reusable = ((len(tokens) - 1) // ps) * ps
        node, pages = self.root, []
        for start in range(0, reusable, ps):
            child = node.children.get(tuple(tokens[start:start + ps]))
            if child is None:
                break
            self._touch(child)
            pages.append(child.page)
            node = child
        if pages:
            self.hits += 1
            self.matched_tokens += len(pages) * ps
        else:
            self.misses += 1
        return pages

    def insert(self, tokens, page_table: List[int]) -> None:
        """Pins every complete page of a prompt whose keys and values are written."""
        ps = self.page_size
        complete = len(tokens) // ps
        if len(page_table) < complete:
            raise ValueError(f"prompt has {complete} complete pages but the table holds {len(page_table)}")
        node = self.root
        for i in range(complete):
            key = tuple(tokens[i * ps:(i + 1) * ps])
            child = node.children.get(key)
            if child is None:
                owner = self._next_owner
                self._next_owner -= 1
                self.allocator.reserve(owner, 0)
                try:
                    self.allocator.share(owner, page_table[i])
                except Exception:
                    self.allocator.release(owner)
                    raise
                child = _Node(key, page_table[i], owner, node)
                node.children[key] = child
                self.cached_pages += 1
            self._touch(child)
            node = child
        while self.cached_pages > self.max_pages:
            if not self._evict_one(set()):
                break

    def evict_until_available(self, required_pages: int, protected: Optional[Set[int]] = None) -> bool:
        protected = protected or set()
        while self.allocator.available_pages < required_pages:
            if not self._evict_one(protected):
                return False
        return True

    def _nodes(self) -> List[_Node]:
        out, stack = [], list(self.root.children.values())
        while stack:
            n = stack.pop()
            out.append(n)
            stack.extend(n.children.values())
        return out

    def _evict_one(self, protected: Set[int]) -> bool:
        leaves = [n for n in self._nodes() if not n.children and n.page not in protected]
        if not leaves:
            return False
        victim = min(leaves, key=lambda n: n.last_used)
        del victim.parent.children[victim.key]
        self.allocator.release(victim.owner)
        self.cached_pages -= 1
        self.evictions += 1
        return True

    def clear(self) -> None:
        for n in self._nodes():
            self.allocator.release(n.owner)
        self.root.children.clear()
        self.cached_pages = 0
        self.hits = self.misses = self.matched_tokens = self.evictions = 0

    def stats(self) -> Dict[str, int]:
        return {"cached_blocks": self.cached_pages, "cached_tokens": self.cached_pages * self.page_size,
                "hits": self.hits, "misses": self.misses, "matched_tokens": self.matched_tokens,
                "evictions": self.evictions}
