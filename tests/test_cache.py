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


# -- shared prefixes ---------------------------------------------------------------------------------------------------
def _prefix_cache(**kw):
    cache, _ = _cache([[PagedState("kv", 2)], [PagedState("kv", 3)]], **kw)
    assert cache.enable_prefix(b"test")
    return cache


def _run(cache, slot, tokens, upto):
    """What a step does: reserve, compute, publish."""
    assert cache.reserve(slot, upto)
    cache.advance(slot, upto)
    cache.publish(slot, tokens)


def test_requests_that_start_alike_share_pages_and_one_token_is_always_left():
    cache = _prefix_cache()
    tokens = list(range(100, 111))                                         # 11 tokens, pages of 4
    a = cache.admit()
    assert cache.adopt(a, tokens) == 0
    _run(cache, a, tokens, 10)
    assert len(cache.prefix.entries) == 2 and cache.chain[a] and len(cache.chain[a]) == 2
    b = cache.admit()
    assert cache.adopt(b, tokens[:9] + [7, 7]) == 8                        # two whole pages, the rest is its own
    for g in cache.groups:
        assert g.table[b, :2].tolist() == g.table[a, :2].tolist() and g.count[b] == 2
        assert all(g.pool.refs(int(p)) == 3 for p in g.table[a, :2])       # a, b and the index
    c = cache.admit()
    assert cache.adopt(c, tokens[:8]) == 4                                 # 8 cached tokens, but one must be computed
    d = cache.admit()
    assert cache.adopt(d, [1] + tokens[1:]) == 0                           # another first token: nothing in common
    assert cache.tokens_saved == 12
    cache.check()
    cache.release(a)
    cache.check()
    _run(cache, b, tokens[:9] + [7, 7], 11)                                # b goes on over the shared pages
    assert all(g.pool.refs(int(g.table[b, 0])) == 3 for g in cache.groups)  # b, c and the index
    for slot in (b, c, d):
        cache.release(slot)
    cache.check()
    assert all(g.pool.free + len(cache.prefix.entries) == g.pool.usable for g in cache.groups)
    cache.flush_prefix()
    cache.check()
    assert all(g.pool.free == g.pool.usable for g in cache.groups)


def test_a_block_stored_twice_is_kept_once():
    cache = _prefix_cache()
    tokens = list(range(9))
    a, b = cache.admit(), cache.admit()
    cache.adopt(a, tokens), cache.adopt(b, tokens)
    assert cache.reserve(a, 9) and cache.reserve(b, 9)                      # both compute the same tokens side by side
    free = [g.pool.free for g in cache.groups]
    cache.advance(a, 9), cache.advance(b, 9)
    cache.publish(a, tokens)
    cache.publish(b, tokens)
    for g, before in zip(cache.groups, free):
        assert g.table[b, :2].tolist() == g.table[a, :2].tolist()          # b took a's pages for its own copies
        assert g.table[b, 2] != g.table[a, 2]                              # the page that is not full stays private
        assert g.pool.free == before + 2
        assert b in g.dirty
    cache.check()


def test_cached_pages_make_room_least_recent_leaves_first():
    cache = _prefix_cache(tokens=32, max_model_len=32)                      # 8 pages
    old, new = [1] * 9, [2] * 13
    for tokens in (old, new):
        s = cache.admit()
        cache.adopt(s, tokens)
        _run(cache, s, tokens, len(tokens))
        cache.release(s)
    assert len(cache.prefix.entries) == 5 and cache.groups[0].pool.free == 3
    s = cache.admit()
    assert cache.adopt(s, old) == 8                                        # a hit makes `old` the more recent chain
    assert cache.could_fit(s, 32, [])                                      # 6 more pages: 3 free and `new`'s 3 idle ones
    assert cache.reserve(s, 24)                                            # 4 more pages: one cached page has to go
    keys = [e.tokens for e in cache.prefix.entries.values()]
    assert keys.count((1,) * 4) == 2 and keys.count((2,) * 4) == 2         # `new` lost its leaf, its last block
    assert cache.prefix.evictions == 1
    cache.check()
    assert cache.reserve(s, 32)                                            # 2 more pages: the rest of `new` goes
    assert [e.tokens for e in cache.prefix.entries.values()] == [(1,) * 4] * 2
    other = cache.admit()
    assert not cache.could_fit(other, 1, []) and not cache.reserve(other, 1)   # `old`'s pages are in use
    assert cache.could_fit(other, 32, [s])
    cache.check()


def test_what_eviction_can_free_counts_for_preemption():
    cache = _prefix_cache(tokens=32, max_model_len=32)
    shared = [5] * 8
    a = cache.admit()
    cache.adopt(a, shared + [1] * 5)
    _run(cache, a, shared + [1] * 5, 13)                                   # 4 pages, 3 of them published
    b = cache.admit()
    assert cache.adopt(b, shared + [2] * 9) == 8
    _run(cache, b, shared + [2] * 9, 17)                                   # 3 more pages; 1 is free
    assert cache.groups[0].pool.free == 1
    c = cache.admit()
    assert cache.could_fit(c, 8, [a])                                      # a's private page and its own cached block
    assert not cache.could_fit(c, 16, [a])                                 # the shared pages stay with b
    assert cache.could_fit(c, 32, [a, b])
    cache.check()


def test_two_prefixes_under_one_key_share_nothing(monkeypatch):
    from holon_amd.cache.prefix import PrefixIndex
    monkeypatch.setattr(PrefixIndex, "key", lambda self, prev, tokens: b"same" + bytes([0 if prev is None else 1]))
    cache = _prefix_cache()
    a, b = cache.admit(), cache.admit()
    first, other = list(range(9)), list(range(50, 59))
    cache.adopt(a, first)
    _run(cache, a, first, 9)
    assert cache.adopt(b, other) == 0                                      # the key is known, the tokens differ
    _run(cache, b, other, 9)
    assert cache.chain[b] is None and len(cache.prefix.entries) == 2       # b stops publishing; a's blocks stay
    assert [e.tokens for e in cache.prefix.entries.values()] == [(0, 1, 2, 3), (4, 5, 6, 7)]
    cache.check()


def test_state_that_pages_do_not_hold_whole_is_not_shared():
    windowed, _ = _cache([[PagedState("kv", 2)], [PagedState("kv", 2, window=6)]])
    assert not windowed.enable_prefix(b"x") and windowed.prefix is None
    fixed, _ = _cache([[PagedState("kv", 2)], [SlotState("s", (3,))]])
    assert not fixed.enable_prefix(b"x")
    slot = fixed.admit()
    assert fixed.adopt(slot, list(range(20))) == 0
    fixed.publish(slot, list(range(20)))


@pytest.mark.parametrize("seed", range(8))
def test_random_orders_keep_the_books_with_shared_prefixes(seed):
    rng = random.Random(seed)
    page = rng.choice([1, 4, 8])
    cache = _prefix_cache(page_size=page, max_seqs=5, max_model_len=80, tokens=rng.choice([80, 120, 200]))
    starts = [[rng.randrange(3) for _ in range(80)] for _ in range(3)]     # few starts, so that requests often share
    live: dict[int, tuple[list[int], int]] = {}
    for _ in range(800):
        action = rng.random()
        if action < 0.25 and (slot := cache.admit()) is not None:
            base = rng.choice(starts)
            cut = rng.randrange(1, 80)
            tokens = base[:cut] + [rng.randrange(3) for _ in range(80 - cut)]
            got = cache.adopt(slot, tokens)
            assert got % page == 0 and got < 80 and cache.capacity(slot) == got
            live[slot] = (tokens, got)
        elif action < 0.85 and live:
            slot = rng.choice(list(live))
            tokens, have = live[slot]
            total = min(80, have + rng.choice([1, 1, 1, 2, 7, 19]))
            if cache.reserve(slot, total):
                cache.advance(slot, total)
                cache.publish(slot, tokens)
                live[slot] = (tokens, total)
            else:
                idle = cache.prefix.idle_pages()
                assert all(-(-total // page) - g.count[slot] > g.pool.free + idle for g in cache.groups)
        elif live:
            slot = rng.choice(list(live))
            cache.release(slot)
            del live[slot]
        cache.check()
        for slot, (tokens, have) in live.items():                         # what a request holds is what it computed
            chain = cache.chain[slot]
            assert chain is not None and len(chain) == have // page
            prev = None
            for i, key in enumerate(chain):
                e = cache.prefix.entries[key]
                assert e.tokens == tuple(tokens[i * page: (i + 1) * page]) and e.parent == prev
                assert all(g.table[slot, i] == e.pages[gid] for gid, g in enumerate(cache.groups))
                prev = key
    for slot in live:
        cache.release(slot)
    cache.check()
    assert cache.prefix.idle_pages() == len(cache.prefix.entries)
    cache.flush_prefix()
    cache.check()
    assert all(g.pool.free == g.pool.usable for g in cache.groups) and cache.free_slots == 5


def test_a_run_may_keep_several_paged_states():
    """Two states of one page geometry in one run share a group (one table, one page id for both); a state of another
    width has a group, a pool and a table of its own. Reserving and releasing moves all of them together."""
    decls = [[PagedState("k", 8), PagedState("v", 8), PagedState("gate", 1, dtype=torch.float32)],
             [PagedState("k", 8), PagedState("v", 8)], [PagedState("gate", 1, dtype=torch.float32)]]
    sites = [Site(run=i, layer=i) for i in range(3)]
    cache = CacheManager(sites, decls, page_size=4, max_seqs=3, max_model_len=32, tokens=48,
                         device=torch.device("cpu"), dtype=torch.bfloat16)
    wide, narrow = cache.groups
    assert wide.members == [(0, "k"), (0, "v"), (1, "k"), (1, "v")] and wide.sites == [0, 1]
    assert narrow.members == [(0, "gate"), (2, "gate")] and narrow.storage.dtype == torch.float32
    assert sites[0].paged["k"].group == sites[0].paged["v"].group == wide.gid and sites[0].paged["gate"].group == narrow.gid
    assert sites[0].paged["k"].pages.data_ptr() != sites[0].paged["v"].pages.data_ptr()
    assert sites[0].group == wide.gid and sites[0].pages.data_ptr() == sites[0].paged["k"].pages.data_ptr()
    assert sites[2].group == narrow.gid
    a, b = cache.admit(), cache.admit()
    assert cache.reserve(a, 9) and cache.reserve(b, 30)
    assert wide.count[a] == narrow.count[a] == 3 and cache.capacity(b) == 32
    assert not cache.reserve(a, 32)                           # all or nothing, over both groups
    assert wide.count[a] == narrow.count[a] == 3
    cache.check()
    cache.release(b)
    assert cache.reserve(a, 32)
    cache.release(a)
    cache.check()
    assert all(g.pool.free == g.pool.usable for g in cache.groups)
    with pytest.raises(ValueError, match="two states of one name"):
        CacheManager([Site(run=0, layer=0)], [[PagedState("k", 8), PagedState("k", 4)]], page_size=4, max_seqs=1,
                     max_model_len=8, tokens=8, device=torch.device("cpu"), dtype=torch.float32)
