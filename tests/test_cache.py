"""The cache manager on its own: no page lost, held twice or freed twice, under random orders of requests; windows give
pages back as they pass; fixed-size slots."""
from __future__ import annotations

import random

import pytest
import torch

from holon_amd.cache import CacheManager, PagePool
from holon_amd.cache.pool import OutOfPages
from holon_amd.model import Site
from holon_amd.parts.base import PagedState, SlotState


def _cache(decls, *, page_size=4, max_seqs=4, max_model_len=64, tokens=64):
    sites = [Site(run=i, layer=i) for i in range(len(decls))]
    cache = CacheManager(sites, decls, page_size=page_size, max_seqs=max_seqs, max_model_len=max_model_len,
                         tokens=tokens, device=torch.device("cpu"), dtype=torch.float32)
    return cache, sites


def test_pool_counts_references():
    pool = PagePool(5)
    assert pool.usable == 4 and pool.null == 4
    a = pool.alloc(3)
    assert a == [0, 1, 2] and pool.free == 1
    with pytest.raises(OutOfPages):
        pool.alloc(2)
    assert pool.free == 1                                     # nothing was taken
    pool.incref(a[0])
    pool.decref(a[0])
    assert pool.free == 1
    pool.decref(a[0])
    assert pool.free == 2 and pool.alloc(1) == [0]            # a freed page is used again first
    with pytest.raises(RuntimeError):
        pool.decref(a[1]) or pool.decref(a[1])
    with pytest.raises(RuntimeError):
        pool.decref(pool.null)


def test_groups_by_declaration_and_shared_caches():
    full, win = PagedState("kv", 8), PagedState("kv", 8, window=6)
    decls = [[full], [win], [full], [win], [], [SlotState("s", (3,))]]
    sites = [Site(run=i, layer=i) for i in range(6)]
    sites[4].writes, sites[4].owner = False, 0                # run 4 reads run 0's cache
    cache = CacheManager(sites, decls, page_size=4, max_seqs=2, max_model_len=32, tokens=32,
                         device=torch.device("cpu"), dtype=torch.float32)
    assert len(cache.groups) == 2
    assert [s.group for s in sites] == [0, 1, 0, 1, 0, None]
    assert sites[4].pages.data_ptr() == sites[0].pages.data_ptr()
    assert sites[0].pages.data_ptr() != sites[2].pages.data_ptr()
    assert cache.groups[0].storage.shape == (2, 9, 4 * 8)
    assert sites[5].slot_state["s"].shape == (3, 3)


def test_window_gives_pages_back_as_it_passes():
    cache, _ = _cache([[PagedState("kv", 2)], [PagedState("kv", 2, window=6)]], tokens=40, max_model_len=40)
    full, win = cache.groups
    slot = cache.admit()
    for total in range(1, 41):
        assert cache.reserve(slot, total)
        cache.advance(slot, total)
        cache.check()
        # the next query at position `total` reads keys total-5 .. total in the windowed group
        first_needed = max(0, total - 5) // 4
        assert win.first[slot] == first_needed
        assert (win.table[slot, :first_needed] == win.pool.null).all()
        assert (win.table[slot, first_needed: -(-total // 4)] != win.pool.null).all()
        assert full.first[slot] == 0
    assert win.pool.usable - win.pool.free <= 3 and full.pool.free == 0
    cache.release(slot)
    cache.check()
    assert win.pool.free == win.pool.usable and full.pool.free == full.pool.usable


def test_reserve_takes_all_or_nothing():
    cache, _ = _cache([[PagedState("kv", 2)], [PagedState("kv", 2, window=4)]], tokens=16, max_seqs=3)
    a, b = cache.admit(), cache.admit()
    assert cache.reserve(a, 12)
    before = [g.pool.free for g in cache.groups]
    assert not cache.reserve(b, 8)                            # one page short in both groups
    assert [g.pool.free for g in cache.groups] == before
    cache.check()
    assert cache.could_fit(b, 8, [a]) and not cache.could_fit(b, 20, [a])
    with pytest.raises(ValueError):
        cache.reserve(a, 65)
    cache.release(a)
    with pytest.raises(RuntimeError):
        cache.release(a)
    assert cache.reserve(b, 8)


def test_slots_are_zeroed_when_given_out():
    cache, sites = _cache([[SlotState("h", (2, 3))]], max_seqs=2)
    s = cache.admit()
    sites[0].slot_state["h"][s] += 5
    cache.release(s)
    assert cache.admit() == s and not sites[0].slot_state["h"][s].any()
    assert cache.admit() is not None and cache.admit() is None


@pytest.mark.parametrize("seed", range(8))
def test_random_orders_keep_the_books(seed):
    rng = random.Random(seed)
    cache, _ = _cache([[PagedState("kv", 2)], [PagedState("kv", 2, window=rng.choice([3, 9, 17]))], [PagedState("kv", 2)]],
                      page_size=rng.choice([1, 4, 8]), max_seqs=5, max_model_len=80, tokens=rng.choice([80, 120, 200]))
    live: dict[int, int] = {}
    for _ in range(600):
        action = rng.random()
        if action < 0.25 and (slot := cache.admit()) is not None:
            live[slot] = 0
        elif action < 0.85 and live:
            slot = rng.choice(list(live))
            total = min(80, live[slot] + rng.choice([1, 1, 1, 2, 7, 19]))
            if cache.reserve(slot, total):
                assert cache.capacity(slot) >= total
                cache.advance(slot, total)
                live[slot] = total
        elif live:
            slot = rng.choice(list(live))
            cache.release(slot)
            del live[slot]
        cache.check()
    for slot in live:
        cache.release(slot)
    cache.check()
    assert all(g.pool.free == g.pool.usable for g in cache.groups) and cache.free_slots == 5
    cache.upload()
    for g in cache.groups:
        assert torch.equal(g.table_dev, torch.from_numpy(g.table))
