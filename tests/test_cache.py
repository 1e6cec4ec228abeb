"""The cache manager: pages, reservations, windows, slots (no GPU)."""

import random

import pytest

from simple_inference_amd.cache import CacheManager, PagePool
from simple_inference_amd.parts.model import CacheLayout
from simple_inference_amd.parts.plan import PagedKVNeed, StateNeed
import torch


def test_pool_vector_of_the_reference_test():
    """serving/test_paged_kv_cache.py:27-43."""
    a = PagePool(4)
    a.open(1, promise=2)
    a.open(2, promise=1)
    assert not a.fits(2) and a.fits(1)
    assert (a.take(1), a.take(1)) == (0, 1)
    a.adopt(2, 0)
    assert a.holders(0) == 2
    a.close(1)
    assert a.holders(0) == 1 and a.n_free == 3
    a.close(2)
    assert a.n_free == 4
    a.audit()


def test_pool_errors():
    a = PagePool(2)
    with pytest.raises(KeyError):
        a.take(9)
    a.open(1, promise=1)
    with pytest.raises(ValueError):
        a.open(1, promise=1)
    with pytest.raises(MemoryError):
        a.open(2, promise=2)
    assert not a.has(2)
    p = a.take(1)
    a.open(2, promise=1)
    with pytest.raises(MemoryError):       # promise used up and the other page is promised
        a.take(1)
    with pytest.raises(ValueError):
        a.adopt(1, p)
    with pytest.raises(ValueError):
        a.adopt(2, 1)                      # page 1 is free
    with pytest.raises(IndexError):
        a.holders(2)
    a.drop(1, p)
    with pytest.raises(KeyError):          # given back twice
        a.drop(1, p)
    a.close(1), a.close(2), a.close(77)
    assert a.n_free == 2
    a.audit()


def test_many_pages_at_once_are_the_pages_one_by_one():
    """``take_many`` hands out what as many calls of ``take`` would, against the promise first and then from the
    unpromised pages, returned pages before fresh ones; if there are not enough, it takes none."""
    rng = random.Random(3)
    for _ in range(50):
        pools = [PagePool(40), PagePool(40)]
        promise, other = rng.randint(0, 12), rng.randint(0, 10)
        for pool in pools:
            pool.open(1, promise=promise)
            pool.open(2, promise=other)
            first = [pool.take(2) for _ in range(min(other, 6))]
            for page in first[::2]:
                pool.drop(2, page)      # returned pages, lower than the fresh ones, go out first
        n = rng.randint(0, 45)
        one_by_one, at_once = pools
        try:
            want = [one_by_one.take(1) for _ in range(n)]
        except MemoryError:
            want = None
        if want is None:
            before = (at_once.n_free, at_once.n_promised, at_once.pages(1))
            with pytest.raises(MemoryError):
                at_once.take_many(1, n)
            assert (at_once.n_free, at_once.n_promised, at_once.pages(1)) == before
        else:
            assert at_once.take_many(1, n) == want
            assert (at_once.n_free, at_once.n_promised) == (one_by_one.n_free, one_by_one.n_promised)
        at_once.audit()


def test_an_account_without_a_promise_takes_unpromised_pages_only():
    a = PagePool(3)
    a.open(1)
    a.open(2, promise=2)
    assert a.take(1) == 0                  # one page is promised to nobody
    with pytest.raises(MemoryError):
        a.take(1)
    assert (a.take(2), a.take(2)) == (1, 2)


def test_pages_come_back_lowest_first_from_below_and_above_the_watermark():
    a = PagePool(6)
    a.open(1)
    got = [a.take(1) for _ in range(4)]
    assert got == [0, 1, 2, 3]
    a.drop(1, 2), a.drop(1, 0)
    assert [a.take(1) for _ in range(3)] == [0, 2, 4]     # returned ids before ids never handed out
    a.audit()


def test_pins_keep_a_page_alive_outside_every_account():
    a = PagePool(2)
    a.open(1)
    p = a.take(1)
    a.pin(p), a.pin(p)
    a.close(1)
    assert a.n_free == 1 and a.holders(p) == 2
    a.audit()
    a.unpin(p)
    assert a.n_free == 1
    a.unpin(p)
    assert a.n_free == 2
    with pytest.raises(KeyError):
        a.unpin(p)
    with pytest.raises(ValueError):
        a.pin(p)                           # a free page
    a.audit()


def test_a_dropped_page_can_become_a_promise_again():
    a = PagePool(2)
    a.open(1, promise=2)
    p, q = a.take(1), a.take(1)
    a.drop(1, p, restore_promise=True)
    assert a.n_free == 1 and a.n_unpromised == 0 and not a.fits(1)
    assert a.take(1) == p
    a.audit()


def layout(groups, slabs=None, states=()):
    lay = CacheLayout()
    lay.kv_groups = list(groups)
    lay.kv_slabs = list(slabs or [1] * len(groups))
    lay.run_kv = [(g, 0) for g in range(len(groups))]
    lay.states = list(states)
    lay.run_state = [i if i < len(states) else None for i in range(len(groups))]
    return lay


def manager(groups, num_pages=8, page_size=2, max_running=3, states=(), storage=False):
    return CacheManager(layout(groups, states=states), page_size=page_size, num_pages=num_pages,
                        max_running=max_running, dtype=torch.float32, device="cpu", allocate_storage=storage)


FULL = PagedKVNeed(1, 4)


def test_pages_follow_growth_and_come_back_lowest_first():
    """serving/test_paged_kv_cache.py:58-89: page size 2, 4 pages."""
    m = manager([FULL], num_pages=4)
    m.admit(1)
    assert m.extend(1, 3) == 0 and m.table(0, 1) == [0, 1]
    assert m.extend(1, 2) == 3 and m.table(0, 1) == [0, 1, 2] and m.lengths[1] == 5
    m.admit(2)
    m.extend(2, 1)
    assert m.table(0, 2) == [3]
    with pytest.raises(MemoryError):
        m.extend(2, 2)
    m.release(1)
    assert m.free_pages() == 3
    m.admit(3)
    m.extend(3, 1)
    assert m.table(0, 3) == [0]            # the lowest free page is handed out again
    m.check()


def test_reservation_makes_running_out_impossible_in_mid_flight():
    m = manager([FULL], num_pages=4)
    assert m.can_admit(8) and not m.can_admit(9)
    m.admit(1, total_tokens=5)             # 3 pages promised
    assert not m.can_admit(3) and m.can_admit(2)
    m.admit(2, total_tokens=2)
    m.extend(2, 2)
    m.extend(1, 5)                         # its promised pages are there although request 2 came in between
    assert sorted(m.table(0, 1) + m.table(0, 2)) == [0, 1, 2, 3]
    with pytest.raises(MemoryError):
        m.extend(1, 2)                     # beyond what it declared, and nothing is left
    m.release(1), m.release(2)
    assert m.free_pages() == 4 and m.groups[0].pool.n_promised == 0


def test_window_group_gives_pages_back_when_the_window_has_passed():
    win = PagedKVNeed(1, 4, window=4)
    m = manager([FULL, win], num_pages=16)
    m.admit(1)
    pos = 0
    held = []
    for n in (3, 2, 1, 1, 6, 1, 1, 1, 1, 1):
        start = m.extend(1, n)
        assert start == pos
        pos += n
        table = m.table(1, 1)
        first_visible = max(0, start - 4 + 1)
        for idx, page in enumerate(table):
            if idx < first_visible // 2:
                assert page == -1                          # wholly below the window: given back
            else:
                assert page >= 0                           # still visible to this step's first query
        held.append(sum(p >= 0 for p in table))
        assert all(p >= 0 for p in m.table(0, 1))          # the full group keeps everything
        m.check()
    assert max(held) <= (4 + 6 - 1 + 1) // 2 + 1           # window + largest portion, in pages, plus one
    assert m.free_pages(1) == 16 - held[-1] and m.free_pages(0) == 16 - len(m.table(0, 1))
    m.release(1)
    assert m.free_pages(0) == 16 and m.free_pages(1) == 16


def test_window_reservation_is_small_and_sufficient():
    win = PagedKVNeed(1, 4, window=4)
    m = manager([win], num_pages=6)
    g = m.groups[0]
    assert g.pages_to_reserve(1000, max_chunk=3) == (4 + 3 - 1 + 1) // 2 + 1 == 4
    assert g.pages_to_reserve(3, max_chunk=3) == 2
    m.admit(1, total_tokens=1000, max_chunk=3)
    m.admit(2, total_tokens=3, max_chunk=3)                # 4 + 2 pages promised: the pool is full
    assert not m.can_admit(1, 1)
    for _ in range(100):
        m.extend(1, 3)                                     # never runs out although 300 positions pass
        m.check()
    m.extend(2, 3)
    m.check()


def test_slots_lowest_first_set_to_their_initial_value_and_scratch():
    m = manager([FULL], states=[StateNeed((2,), "float32"), StateNeed((3,), "float32", init=-1.5)], storage=True,
                max_running=2)
    s0, s1 = m.admit(10), m.admit(11)
    assert (s0, s1) == (0, 1) and m.slots.scratch_slot == 2
    state = m.slots.tensors[0]
    assert state.shape == (3, 2)
    state[0] = 7.0
    assert not m.can_admit(None)
    with pytest.raises(MemoryError):
        m.admit(12)
    m.release(10)
    other = m.slots.tensors[1]
    assert other.shape == (3, 3) and bool((other == -1.5).all())
    other[0] = 4.0
    assert m.admit(13) == 0 and float(state[0].abs().sum()) == 0.0   # set anew on assignment
    assert bool((other[0] == -1.5).all())
    m.check()


def test_shared_prefix_pages():
    m = manager([FULL], num_pages=6)
    m.admit(1, total_tokens=5)
    m.extend(1, 5)
    first_two = m.table(0, 1)[:2]
    m.admit(2, total_tokens=6, shared_pages=first_two)
    assert m.lengths[2] == 4 and m.table(0, 2) == first_two
    m.extend(2, 2)
    assert m.table(0, 2)[:2] == first_two and m.table(0, 2)[2] not in m.table(0, 1)
    m.release(1)
    assert m.groups[0].pool.holders(first_two[0]) == 1   # still held by request 2
    m.release(2)
    assert m.free_pages() == 6


@pytest.mark.parametrize("seed", range(5))
def test_random_orders_lose_no_page(seed):
    """Requests arrive, grow by random portions, and end in random order; after every operation no page
    is lost, held twice or freed twice, and at the end every page and slot is free."""
    rng = random.Random(seed)
    win = PagedKVNeed(2, 8, window=5)
    m = manager([FULL, win], num_pages=40, page_size=4, max_running=4)
    live, next_id = {}, 1
    for _ in range(400):
        action = rng.random()
        if action < 0.25 and len(live) < 4:
            total = rng.randint(1, 60)
            reserve = rng.random() < 0.5
            if m.can_admit(total if reserve else None, max_chunk=7):
                m.admit(next_id, total if reserve else None, max_chunk=7)
                live[next_id] = total
                next_id += 1
        elif action < 0.85 and live:
            r = rng.choice(list(live))
            room = live[r] - m.lengths[r]
            if room > 0:
                n = rng.randint(1, min(7, room))
                try:
                    m.extend(r, n)
                except MemoryError:
                    m.release(r)           # an unreserved request that found no page: give up cleanly
                    del live[r]
        elif live:
            r = rng.choice(list(live))
            m.release(r)
            del live[r]
        m.check()
        for g in m.groups:
            held = sum(len(g.pool.pages(o)) for o in g.pool.owners())
            assert held + g.pool.n_free == g.num_pages
    for r in list(live):
        m.release(r)
    m.check()
    assert all(m.free_pages(g) == 40 for g in range(2)) and m.slots.free_slots == 4
    assert all(g.pool.n_promised == 0 for g in m.groups)


def test_a_table_version_never_comes_back():
    """Graph replay keeps a block-table row while (request, version) is what it wrote.  An id that is admitted
    again after its release, with the same history of growth, must not meet a version it had before: its pages
    may be others now."""
    m = manager([FULL], num_pages=16, max_running=5)
    seen = set()
    for turn in range(3):
        m.admit(7)
        for n in (1, 3, 2):
            m.extend(7, n)
            v = (7, m.groups[0].versions[7])
            assert v not in seen
            seen.add(v)
        m.admit(100 + turn)          # takes pages in between, so that request 7 gets others next time
        m.extend(100 + turn, 2)
        m.release(7)
    m.check()
