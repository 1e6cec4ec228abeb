"""Prefix reuse: the reference's vectors for its radix cache, and the engine with it (CPU, twins)."""

import pytest
import torch

from helpers import TINIES, random_tokens, write_tiny_model
from simple_inference_amd import Engine, EngineConfig
from simple_inference_amd.cache import CacheManager, PrefixCache
from simple_inference_amd.parts.model import CacheLayout
from simple_inference_amd.parts.plan import PagedKVNeed
from twins import TwinKernels


def manager(num_pages, page_size=2, window=None):
    lay = CacheLayout()
    lay.kv_groups, lay.kv_slabs, lay.run_kv, lay.run_state = [PagedKVNeed(1, 4, window)], [1], [(0, 0)], [None]
    return CacheManager(lay, page_size=page_size, num_pages=num_pages, max_running=4, dtype=torch.float32,
                        device="cpu", allocate_storage=False)


def test_match_shares_complete_pages_and_clear_keeps_live_requests():
    """serving/test_paged_kv_cache.py:93-125: free pages 4 -> 4 -> 6."""
    m = manager(6)
    pc = PrefixCache(m, max_pages=6)
    m.admit(1, total_tokens=4)
    m.extend(1, 4)
    pc.insert([1, 2, 3, 4], m.table(0, 1))
    assert m.free_pages() == 4
    pages = pc.match([1, 2, 3, 4, 5])
    assert pages == m.table(0, 1) and pc.stats()["tokens_reused"] == 4
    assert pc.match([1, 2, 3, 4]) == m.table(0, 1)[:1]          # a token must be left to run
    assert pc.match([9, 9, 9]) == []
    m.admit(2, total_tokens=6, shared_pages=pages)
    assert m.lengths[2] == 4 and m.free_pages() == 4
    m.release(1)
    assert m.free_pages() == 4                                   # still pinned by the cache and request 2
    pc.clear()
    assert m.free_pages() == 4                                   # request 2 still holds them
    m.release(2)
    assert m.free_pages() == 6
    m.check()


def test_least_recently_used_leaf_goes_first():
    """serving/test_paged_kv_cache.py:127-156: max 2 pages; the newer path evicts the old one."""
    m = manager(8)
    pc = PrefixCache(m, max_pages=2)
    for rid, toks in ((1, [1, 2, 3, 4]), (2, [5, 6, 7, 8])):
        m.admit(rid, total_tokens=4)
        m.extend(rid, 4)
        pc.insert(toks, m.table(0, rid))
        m.release(rid)
    assert pc.match([1, 2, 3, 4, 0]) == [] and len(pc.match([5, 6, 7, 8, 0])) == 2
    assert pc.stats()["pages_dropped"] == 2 and pc.stats()["pages"] == 2 and len(pc) == 2
    assert m.free_pages() == 6
    assert pc.evict_until_available(8) and m.free_pages() == 8
    assert not pc.evict_until_available(9)


def test_the_end_of_a_chain_that_was_used_longest_ago_goes_first_and_protected_pages_stay():
    """Three prompts share their first page; what ends a chain and is oldest is dropped, an entry that others
    continue never, a protected page never, and an entry whose last continuation went becomes an end itself."""
    m = manager(16)
    pc = PrefixCache(m, max_pages=16)
    prompts = {1: [1, 2, 3, 4, 5, 6], 2: [1, 2, 7, 8], 3: [1, 2, 9, 9]}
    tables = {}
    for rid, toks in prompts.items():
        m.admit(rid, total_tokens=len(toks))
        m.extend(rid, len(toks))
        tables[rid] = list(m.table(0, rid))
        pc.insert(toks, tables[rid])
        m.release(rid)
    assert len(pc) == 5 and m.free_pages() == 16 - 7 + 2            # the two duplicates of the first page are free
    pc.match([1, 2, 3, 4, 5, 6, 0])                                   # chain 1 is the most recently used now
    shared = tables[1][0]
    # oldest end is chain 2's second page; protect it: chain 3's goes instead
    assert pc.evict_until_available(m.free_pages() + 1, protected={tables[2][1]})
    assert pc.match([1, 2, 9, 9, 0]) == [shared] and pc.match([1, 2, 7, 8, 0]) == [shared, tables[2][1]]
    # drop everything but keep the first page: its continuations go one by one, then it is an end itself
    assert pc.evict_until_available(m.free_pages() + 3, protected={shared})
    assert len(pc) == 1 and not pc.evict_until_available(m.free_pages() + 1, protected={shared})
    assert pc.evict_until_available(16) and len(pc) == 0
    m.check()


def test_the_lazy_heap_is_started_afresh_when_it_is_mostly_stale():
    m = manager(4)
    pc = PrefixCache(m, max_pages=4)
    m.admit(1, total_tokens=2)
    m.extend(1, 2)
    pc.insert([1, 2], m.table(0, 1))
    for _ in range(500):
        assert pc.match([1, 2, 3]) == m.table(0, 1)
    assert len(pc._ends) <= 4 * len(pc) + 65
    m.release(1)
    assert pc.evict_until_available(4) and m.free_pages() == 4


def test_chains_whose_digests_collide_are_told_apart(monkeypatch):
    """A prefix is known by a digest of its pages; an entry also keeps its page's ids and the digest in front, and a
    lookup believes a digest only if both agree.  With a digest that is the same for everything, nothing is ever
    found that was not put in: the first page of the first prompt is cached, whatever collides with it stays out."""
    from simple_inference_amd.cache import prefix
    monkeypatch.setattr(prefix, "_extend", lambda digest, ids: 7)
    m = manager(8)
    pc = PrefixCache(m, max_pages=8)
    for rid, toks in ((1, [1, 2, 3, 4]), (2, [5, 6, 7, 8])):
        m.admit(rid, total_tokens=4)
        m.extend(rid, 4)
        pc.insert(toks, m.table(0, rid))
    assert len(pc) == 1
    assert pc.match([1, 2, 3, 4, 0]) == m.table(0, 1)[:1]      # its second page has the digest of its first
    assert pc.match([5, 6, 7, 8, 0]) == [] and pc.match([3, 4, 0]) == []
    m.release(1)
    m.release(2)
    assert pc.evict_until_available(8) and len(pc) == 0
    m.check()


def test_refuses_models_it_cannot_serve():
    with pytest.raises(ValueError, match="window"):
        PrefixCache(manager(4, window=8), max_pages=4)


def test_engine_with_prefix_reuse_gives_the_same_tokens(tmp_path):
    """serving/test_paged_kv_cache.py:271-301 in kind: the second prompt shares pages with the first."""
    tiny = TINIES["b"]
    folder = write_tiny_model(tmp_path, tiny, seed=61)
    base = random_tokens(384, 37, seed=1)
    prompts = [base + [5, 6], base + [7], base[:20] + [9, 9, 9], random_tokens(384, 11, seed=2)]

    def run(use):
        eng = Engine.from_folder(folder, EngineConfig(
            device="cpu", dtype="float32", max_seq_len=96, block_size=8, max_running=2, chunk_tokens=16, eos_id=-1,
            num_kv_blocks=24, use_prefix_cache=use, prefix_cache_blocks=6), TwinKernels())
        out = []
        for p in prompts:                       # one after the other, so that earlier prompts are cached
            r = eng.add_request(p, max_new_tokens=4)
            eng.run()
            out.append((r.generated, r.cached_prefix_len))
        return eng, out
    _, plain_out = run(False)
    eng, cached_out = run(True)
    assert [g for g, _ in cached_out] == [g for g, _ in plain_out]
    assert [c for _, c in cached_out] == [0, 32, 16, 0]        # whole pages of 8, one token always left to run
    assert eng.prefix_cache.stats()["lookups_hit"] == 2 and eng.prefix_cache.stats()["pages"] <= 6
    eng.cache.check()
    eng.reset()
    assert eng.cache.free_pages() == 24


def test_prompts_that_arrive_together_share_what_the_first_of_them_wrote(tmp_path):
    """Several prompts with one long prefix are queued at once.  Requests enter a step only when it has room
    for their tokens, and a prompt's filled pages are cached step by step: so the later ones find the prefix,
    run their own ends only and generate what they generate without the cache."""
    tiny = TINIES["a"]
    folder = write_tiny_model(tmp_path, tiny, seed=62)
    prefix = random_tokens(tiny.config["vocab_size"], 44, seed=3)
    prompts = [prefix + random_tokens(tiny.config["vocab_size"], 3 + i, seed=10 + i) for i in range(5)]

    def run(use):
        eng = Engine.from_folder(folder, EngineConfig(
            device="cpu", dtype="float32", max_seq_len=96, block_size=4, max_running=4, chunk_tokens=16, eos_id=-1,
            num_kv_blocks=120, use_prefix_cache=use), TwinKernels())
        reqs = [eng.add_request(p, max_new_tokens=5) for p in prompts]
        eng.run()
        eng.cache.check()
        return eng, reqs
    _, plain_reqs = run(False)
    eng, reqs = run(True)
    assert [r.generated for r in reqs] == [r.generated for r in plain_reqs]
    assert reqs[0].cached_prefix_len == 0
    assert all(r.cached_prefix_len == 44 for r in reqs[1:])      # 11 whole pages of 4
    assert eng.stats["prefill_tokens"] == sum(len(p) for p in prompts) - 4 * 44
    eng.reset()
    assert eng.cache.free_pages() == 120
