"""The cache manager: pages of keys and values, block tables, and state slots.

Layers with the same cache need form a *group*; a group has pages of its own, a
page allocator of its own and, for each request, a block table of its own
(reference: one pool and one table for all layers, ``serving/paged_kv_cache.py:75-78``).
Within a group every run of a layer that writes keys and values has one *slab* of
the pool, and one page id addresses that page in all slabs.

    keys    [slabs, pages + 1, kv_heads, page_size, head_dim]
    values  [slabs, pages + 1, kv_heads, value_dim, page_size]

(``value_dim`` is ``head_dim`` unless the group's need says otherwise: a mixer may cache
rows of another width beside its keys.)

Values are stored with the positions innermost, so that the product
``probabilities x values`` reads consecutive positions as the matrix cores want
them.  The last page of a pool is a scratch page that no request owns; padded
rows of a replayed graph write there.

A group with a window keeps, for each request, only pages that a future query
can still see: before a step that starts at position ``s``, pages that lie wholly
below ``s - window + 1`` go back to the allocator, and their table entries
become -1.

Beside the pages there are *slots*: one row of fixed size per running request
and per stateful run of a layer, set to the state's initial value when a request gets its slot.  The
architecture served here has no such state; the slots still exist, every request
holds one, and the step function hands the slot ids to every mixer.
"""

from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..parts.context import LayerCache
from ..parts.model import CacheLayout
from ..parts.plan import PagedKVNeed
from .allocator import PagePool

_STATE_DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16, "int32": torch.int32}


def pages_for(tokens: int, page_size: int) -> int:
    return -(-tokens // page_size)


class PagedGroup:
    """Pages, allocator and block tables of one group of layers."""

    def __init__(self, need: PagedKVNeed, slabs: int, page_size: int, num_pages: int,
                 dtype: torch.dtype, device, allocate_storage: bool = True):
        self.need = need
        self.slabs = slabs
        self.page_size = page_size
        self.num_pages = num_pages
        self.scratch_page = num_pages
        self.pool = PagePool(num_pages)
        self.tables: Dict[int, List[int]] = {}
        # a request's entry changes whenever its table does (graph replay skips rows that did not change); the
        # numbers come from one counter, so an id that is admitted again never meets a number it had before
        self.versions: Dict[int, int] = {}
        self._version = 0
        self.k = self.v = None
        if allocate_storage:
            shape_k = (slabs, num_pages + 1, need.num_kv_heads, page_size, need.head_dim)
            shape_v = (slabs, num_pages + 1, need.num_kv_heads, need.value_dim, page_size)
            self.k = torch.zeros(shape_k, dtype=dtype, device=device)
            self.v = torch.zeros(shape_v, dtype=dtype, device=device)

    def pages_to_reserve(self, total_tokens: int, max_chunk: int) -> int:
        """Most pages a request of ``total_tokens`` holds at once, fed at most ``max_chunk`` a step."""
        full = pages_for(total_tokens, self.page_size)
        if self.need.window is None:
            return full
        # A step sees keys from (start - window + 1) to (start + chunk - 1): window + chunk - 1
        # positions, which touch at most that many / page_size pages plus one for misalignment.
        span = self.need.window + max_chunk - 1
        return min(full, pages_for(span, self.page_size) + 1)

    def begin(self, req: int, reserve: int) -> None:
        self.pool.open(req, reserve)
        self.tables[req] = []
        self._touch(req)

    def extend(self, req: int, start: int, end: int) -> None:
        """Makes the table ready for a step that writes positions ``start .. end-1``."""
        table = self.tables[req]
        if self.need.window is not None:
            first_visible = max(0, start - self.need.window + 1)
            for idx in range(min(first_visible // self.page_size, len(table))):
                if table[idx] >= 0:
                    self.pool.drop(req, table[idx], restore_promise=True)
                    table[idx] = -1
                    self._touch(req)
        more = pages_for(end, self.page_size) - len(table)
        if more > 0:
            table.extend(self.pool.take_many(req, more))
            self._touch(req)

    def _touch(self, req: int) -> None:
        self._version += 1
        self.versions[req] = self._version

    def release(self, req: int) -> None:
        self.pool.close(req)
        self.tables.pop(req, None)
        self.versions.pop(req, None)


class StateSlots:
    """One row per running request; row ``max_running`` is scratch for padded rows."""

    def __init__(self, states, max_running: int, device, allocate_storage: bool = True):
        self.max_running = max_running
        self.scratch_slot = max_running
        self._free = list(range(max_running))
        self.slot_of: Dict[int, int] = {}
        self.tensors: List[Optional[torch.Tensor]] = []
        self.initial = [need.init for need in states]
        for need in states:
            if allocate_storage:
                self.tensors.append(torch.full((max_running + 1, *need.shape), need.init,
                                               dtype=_STATE_DTYPES[need.dtype], device=device))
            else:
                self.tensors.append(None)

    @property
    def free_slots(self) -> int:
        return len(self._free)

    def take(self, req: int) -> int:
        if req in self.slot_of:
            raise ValueError(f"request {req} already has a slot")
        if not self._free:
            raise MemoryError("no free state slot")
        slot = self._free.pop(0)  # lowest first (reference: ``serving/scheduler.py:59,116``)
        self.slot_of[req] = slot
        for t, init in zip(self.tensors, self.initial):
            if t is not None:
                t[slot].fill_(init)
        return slot

    def give_back(self, req: int) -> None:
        slot = self.slot_of.pop(req, None)
        if slot is not None:
            self._free.append(slot)
            self._free.sort()


class CacheManager:
    def __init__(self, layout: CacheLayout, *, page_size: int, num_pages: int, max_running: int,
                 dtype: torch.dtype, device, allocate_storage: bool = True):
        self.layout = layout
        self.page_size = page_size
        self.groups = [
            PagedGroup(need, slabs, page_size, num_pages, dtype, device, allocate_storage)
            for need, slabs in zip(layout.kv_groups, layout.kv_slabs)
        ]
        self.slots = StateSlots(layout.states, max_running, device, allocate_storage)
        self.lengths: Dict[int, int] = {}

    # -- admission ---------------------------------------------------------
    def can_admit(self, total_tokens: Optional[int], max_chunk: int = 1, shared_pages: int = 0) -> bool:
        """Whether a slot and, in every group, the pages for ``total_tokens`` can be promised."""
        if self.slots.free_slots == 0:
            return False
        if total_tokens is None:
            return True
        return all(
            g.pages_to_reserve(total_tokens, max_chunk) - shared_pages <= g.pool.n_unpromised
            for g in self.groups)

    def admit(self, req: int, total_tokens: Optional[int] = None, max_chunk: int = 1,
              shared_pages: Optional[List[int]] = None) -> int:
        """Gives a request its slot and promises it pages; returns the slot.

        ``total_tokens`` None promises nothing: pages are then taken as the request
        grows, while unpromised pages last.  ``shared_pages`` (one group, no window)
        are pages of an equal prompt prefix that are already written.
        """
        if req in self.lengths:
            raise ValueError(f"request {req} is already admitted")
        shared = list(shared_pages or [])
        if shared and (len(self.groups) != 1 or self.groups[0].need.window is not None or self.layout.states):
            raise ValueError("shared prefix pages need exactly one group without a window and no state")
        if not self.can_admit(total_tokens, max_chunk, len(shared)):
            raise MemoryError(f"cannot admit request {req}: no slot or not enough pages")
        slot = self.slots.take(req)
        for g in self.groups:
            reserve = 0 if total_tokens is None else max(0, g.pages_to_reserve(total_tokens, max_chunk) - len(shared))
            g.begin(req, reserve)
            for page in shared:
                g.pool.adopt(req, page)
                g.tables[req].append(page)
                g._touch(req)
        self.lengths[req] = len(shared) * self.page_size
        return slot

    def extend(self, req: int, new_tokens: int) -> int:
        """Before a step: pages for ``new_tokens`` more positions. Returns the start position."""
        start = self.lengths[req]
        for g in self.groups:
            g.extend(req, start, start + new_tokens)
        self.lengths[req] = start + new_tokens
        return start

    def retract(self, req: int, tokens: int) -> None:
        """Takes back the last ``extend`` of a step that did not run after all.  Only the length goes back: the
        pages stay the request's (the next ``extend`` finds them in its table), and pages that a window had
        passed stay given back, since no later step could have seen them either."""
        if not 0 <= tokens <= self.lengths[req]:
            raise ValueError(f"request {req} holds {self.lengths[req]} tokens and cannot go back {tokens}")
        self.lengths[req] -= tokens

    def release(self, req: int) -> None:
        for g in self.groups:
            g.release(req)
        self.slots.give_back(req)
        self.lengths.pop(req, None)

    def reset(self) -> None:
        for req in list(self.lengths):
            self.release(req)

    # -- views -------------------------------------------------------------
    def slot(self, req: int) -> int:
        return self.slots.slot_of[req]

    def table(self, group: int, req: int) -> List[int]:
        return self.groups[group].tables[req]

    def max_table_len(self, reqs) -> int:
        return max((len(g.tables[r]) for g in self.groups for r in reqs), default=0)

    def layer_caches(self, block_tables: List[torch.Tensor]) -> List[LayerCache]:
        """One ``LayerCache`` per run of the order, over this step's device block tables."""
        caches = []
        for e, kv in enumerate(self.layout.run_kv):
            c = LayerCache()
            if kv is not None:
                g, slab = kv
                grp = self.groups[g]
                c.k_pages, c.v_pages = grp.k[slab], grp.v[slab]
                c.block_table = block_tables[g]
                c.page_size = grp.page_size
            si = self.layout.run_state[e]
            if si is not None:
                c.state = self.slots.tensors[si]
            caches.append(c)
        return caches

    # -- checks ------------------------------------------------------------
    def free_pages(self, group: int = 0) -> int:
        return self.groups[group].pool.n_free

    def check(self) -> None:
        for g in self.groups:
            g.pool.audit()
            for req, table in g.tables.items():
                live = [p for p in table if p >= 0]
                if len(set(live)) != len(live):
                    raise AssertionError(f"request {req} holds a page twice")
                if set(live) != g.pool.pages(req):
                    raise AssertionError(f"request {req}: table and allocator disagree")
        slots = list(self.slots.slot_of.values())
        if len(set(slots)) != len(slots):
            raise AssertionError("a state slot is held twice")
