"""The scheduler's decisions, on the real cache manager without a model (no GPU): what a step holds, the token
budget, first come first served, what happens when pages run out. core/tests/test_sched.py:13-197 is the model."""
from __future__ import annotations

import random

import pytest
import torch

from holon_amd.cache import CacheManager
from holon_amd.config import SamplingParams
from holon_amd.engine.request import Seq, Status
from holon_amd.engine.scheduler import Scheduler
from holon_amd.model import Site
from holon_amd.parts.base import PagedState


def _sched(tokens=64, page=4, max_seqs=4, max_model_len=32, max_step_tokens=16, chunk_with_decode=0, prefix=False):
    cache = CacheManager([Site(run=0, layer=0)], [[PagedState("kv", 2)]], page_size=page, max_seqs=max_seqs,
                         max_model_len=max_model_len, tokens=tokens, device=torch.device("cpu"), dtype=torch.float32)
    if prefix:
        assert cache.enable_prefix(b"sched")
    return Scheduler(cache, max_step_tokens, max_model_len, chunk_with_decode), cache


def _seq(rid, n, max_tokens=8):
    return Seq(rid=str(rid), tokens=list(range(n)), params=SamplingParams(temperature=0.0, max_tokens=max_tokens))


def _commit(sched, cache, rows):
    """What the engine does after a step: tokens are in the cache, sampled rows get a token, finished ones leave."""
    for seq, n, m in rows:
        cache.advance(seq.slot, seq.num_computed + n)
        seq.num_computed += n
        cache.publish(seq.slot, seq.tokens)
        if m:
            if seq.status is not Status.RUNNING:
                sched.prompt_done(seq)
            seq.tokens.append(0)
            if seq.length_left(sched.max_model_len) == 0:
                sched.retire(seq, "length")


def test_prompts_are_cut_under_the_token_budget_in_arrival_order():
    sched, cache = _sched(max_step_tokens=16)
    a, b, c = _seq("a", 10), _seq("b", 20), _seq("c", 3)
    for s in (a, b, c):
        sched.add(s)
    rows = sched.schedule()
    assert [(s.rid, n, m) for s, n, m in rows] == [("a", 10, 1), ("b", 6, 0)]           # b is cut where the budget ends
    _commit(sched, cache, rows)
    rows = sched.schedule()                                                             # waiting requests go first
    assert [(s.rid, n, m) for s, n, m in rows] == [("b", 14, 1), ("c", 2, 0)]
    _commit(sched, cache, rows)
    rows = sched.schedule()
    assert [(s.rid, n, m) for s, n, m in rows] == [("c", 1, 1)]
    _commit(sched, cache, rows)
    rows = sched.schedule()                                                             # nothing waits: decode everyone
    assert [(s.rid, n, m) for s, n, m in rows] == [("a", 1, 1), ("b", 1, 1), ("c", 1, 1)]
    assert all(s.status is Status.RUNNING for s in (a, b, c))


def test_mixed_steps_put_decode_rows_first_and_cap_the_portions():
    sched, cache = _sched(max_step_tokens=16, chunk_with_decode=6, max_seqs=4)
    a, b = _seq("a", 5), _seq("b", 20)
    sched.add(a)
    _commit(sched, cache, sched.schedule())
    sched.add(b)
    rows = sched.schedule()
    assert [(s.rid, n, m) for s, n, m in rows] == [("a", 1, 1), ("b", 6, 0)]
    assert sched.mixed_steps == 1
    _commit(sched, cache, rows)
    assert [(s.rid, n) for s, n, _ in sched.schedule()] == [("a", 1), ("b", 6)]


def test_no_slot_no_admission_and_nobody_skips_ahead():
    sched, cache = _sched(max_seqs=2, tokens=64)
    for s in (_seq("a", 4), _seq("b", 4), _seq("c", 4)):
        sched.add(s)
    rows = sched.schedule()
    assert [s.rid for s, _, _ in rows] == ["a", "b"]                                    # c has no slot yet
    _commit(sched, cache, rows)
    assert [s.rid for s, _, _ in sched.schedule()] == ["a", "b"]                        # c still waits: they decode


def test_when_pages_run_out_the_lowest_ranked_is_preempted_and_recomputed():
    sched, cache = _sched(tokens=24, page=4, max_model_len=24, max_step_tokens=32)      # 6 pages
    a, b = _seq("a", 11, max_tokens=12), _seq("b", 11, max_tokens=12)
    sched.add(a), sched.add(b)
    rows = sched.schedule()
    assert [(s.rid, n) for s, n, _ in rows] == [("a", 11), ("b", 11)]                   # 3 pages each: the pool is full
    _commit(sched, cache, rows)
    rows = sched.schedule()                                                             # token 12 fits the pages held
    assert len(rows) == 2
    _commit(sched, cache, rows)
    rows = sched.schedule()                                                             # token 13 needs a page: b gives way
    assert [(s.rid, n) for s, n, _ in rows] == [("a", 1)] and sched.preemptions == 1
    assert b.status is Status.PREEMPTED and b.slot == -1 and b.num_computed == 0 and sched.waiting[0] is b
    cache.check()
    _commit(sched, cache, rows)
    while a.status is not Status.FINISHED:                                              # b cannot come back while a grows
        rows = sched.schedule()
        assert all(s is a for s, _, _ in rows) or a.status is Status.FINISHED
        _commit(sched, cache, rows)
    rows = sched.schedule()                                                             # b runs its prompt and its 2 tokens again
    assert [(s.rid, n, m) for s, n, m in rows] == [("b", 13, 1)]


def test_a_request_alone_that_cannot_grow_preempts_itself_and_the_engine_would_refuse_that_setup():
    sched, cache = _sched(tokens=8, page=4, max_model_len=32)
    assert not cache.fits_alone(32)                 # the engine checks this at start and refuses (OutOfPages)
    a = _seq("a", 8, max_tokens=8)
    sched.add(a)
    _commit(sched, cache, sched.schedule())
    assert sched.schedule() is None or a.status is Status.PREEMPTED


@pytest.mark.parametrize("prefix", [False, True], ids=["", "shared-prefixes"])
@pytest.mark.parametrize("mode", [0, 5])
@pytest.mark.parametrize("seed", range(12))
def test_every_request_finishes_under_random_traffic(seed, mode, prefix):
    """Prompts are 0, 1, 2, ...: each is the start of every longer one, so with a prefix index most admissions hit."""
    rng = random.Random(seed)
    max_len = 32
    sched, cache = _sched(tokens=rng.choice([32, 40, 64, 96]), page=rng.choice([1, 4, 8]), max_seqs=rng.choice([2, 4]),
                          max_model_len=max_len, max_step_tokens=rng.choice([12, 16, 40]) if not mode else 16,
                          chunk_with_decode=mode, prefix=prefix)
    assert cache.fits_alone(max_len)
    seqs = [_seq(i, rng.randint(1, 24), max_tokens=rng.randint(1, 12)) for i in range(14)]
    pending = list(seqs)
    for step in range(2000):
        while pending and rng.random() < 0.4:
            sched.add(pending.pop(0))
        rows = sched.schedule()
        if rows is None:
            if not pending and not sched.waiting and not sched.running:
                break
            assert pending, "no progress with requests pending"
            continue
        n_decode = sum(1 for s, n, m in rows if s.status is Status.RUNNING)
        assert all(s.status is Status.RUNNING for s, _, _ in rows[:n_decode])            # decode rows first, then portions
        assert all(s.status is not Status.RUNNING for s, _, _ in rows[n_decode:])
        assert sum(n for _, n, _ in rows) <= sched.max_step_tokens
        if mode and n_decode:
            assert sum(n for _, n, _ in rows[n_decode:]) <= mode
        for s, n, m in rows:
            assert n >= 1 and s.slot >= 0 and s.num_computed + n <= cache.capacity(s.slot)
            assert m == int(s.num_computed + n == len(s.tokens))
        _commit(sched, cache, rows)
        cache.check()
    assert all(s.status is Status.FINISHED for s in seqs)
    assert all(len(s.tokens) - s.prompt_len == min(s.params.max_tokens, max_len - s.prompt_len) for s in seqs)
    if prefix:
        assert cache.tokens_saved > 0
        cache.flush_prefix()
    assert all(g.pool.free == g.pool.usable for g in cache.groups) and cache.free_slots == cache.max_seqs


def test_a_part_may_say_where_a_portion_ends():
    """`cut`: a model whose state is kept on a grid of 8 positions lets a portion that does not end the prompt end
    only there. The budget of 13 then carries 8 tokens of a long prompt; a prompt's end is free; a budget that reaches
    no grid position carries nothing of that prompt and nobody skips ahead of it."""
    def cut(start, count):
        return (start + count) // 8 * 8 - start
    cache = CacheManager([Site(run=0, layer=0)], [[PagedState("kv", 2)]], page_size=4, max_seqs=4, max_model_len=64,
                         tokens=128, device=torch.device("cpu"), dtype=torch.float32)
    sched = Scheduler(cache, 13, 64, cut=cut)
    a, b = _seq("a", 30), _seq("b", 5)
    sched.add(a), sched.add(b)
    seen = []
    for _ in range(6):
        rows = sched.schedule()
        seen.append([(s.rid, s.num_computed, n, m) for s, n, m in rows])
        _commit(sched, cache, rows)
    assert seen[:4] == [[("a", 0, 8, 0), ("b", 0, 5, 1)], [("a", 8, 8, 0)], [("a", 16, 8, 0)], [("a", 24, 6, 1)]]
    sched = Scheduler(cache, 13, 64, chunk_with_decode=5, cut=cut)      # 5 tokens beside decode rows reach no edge from 8
    c, d = _seq("c", 4), _seq("d", 30)
    sched.add(c)
    _commit(sched, cache, sched.schedule())
    sched.add(d), sched.add(_seq("e", 3))
    rows = sched.schedule()
    assert [(s.rid, n) for s, n, _ in rows] == [("c", 1)]      # (the engine refuses such a budget when it starts)
