"""Scheduling: which requests run in the next step and how many tokens each. core/holon/core/sched.py:65-217.

First come, first served. Requests are ranked running (oldest first), then waiting (queue order; a preempted request
re-enters at the front). Without mixing (`chunk_with_decode` 0) a step is either prompt portions — of as many waiting
requests as the token budget `max_step_tokens` holds, a long prompt cut where the budget ends — or one decoded token
for every running request; waiting requests go first. With mixing (`chunk_with_decode` C > 0) a step carries every
running request's decode token and then prompt portions of up to C tokens.

When pages run out: a request that cannot get the pages it needs takes them from the requests ranked below it, the
lowest first, as long as releasing those can make room (preemption by recompute: the victim gives back everything,
goes to the front of the queue and later runs its prompt and the tokens it had generated again as one prompt). When
nothing below can make room, a running request preempts itself and a waiting one ends the step's admissions. The pool
always holds one request of `max_model_len` tokens (checked when the engine starts), so the top-ranked request always
fits once everything below it is preempted, and every step makes progress.

A step may be scheduled while the one before it still runs (core/holon/core/sched.py:12-15, 98-104): a request whose
last drawn token has not reached the host (`pending`) decodes from the copy of it on the device; it counts towards the
request's length limits; a preempted request waits for it before its tokens are run again as a prompt.
"""
from __future__ import annotations

import collections

from ..cache.manager import CacheManager
from .request import Seq, Status

Row = tuple[Seq, int, int]               # (request, tokens to run, 1 if the last of them is sampled)


class Scheduler:
    def __init__(self, cache: CacheManager, max_step_tokens: int, max_model_len: int, chunk_with_decode: int = 0,
                 on_admit=None) -> None:
        self.cache, self.max_step_tokens, self.max_model_len = cache, max_step_tokens, max_model_len
        self.chunk_with_decode = chunk_with_decode
        self.on_admit = on_admit
        self.waiting: collections.deque[Seq] = collections.deque()
        self.running: list[Seq] = []
        self.preemptions = 0
        self.mixed_steps = 0

    def add(self, seq: Seq, front: bool = False) -> None:
        seq.status = Status.WAITING
        (self.waiting.appendleft if front else self.waiting.append)(seq)

    def schedule(self) -> list[Row] | None:
        """The next step's rows: decode rows first, then prompt portions. None when nothing can run."""
        cap = self.chunk_with_decode
        if not cap:
            rows = self._prefill(self.max_step_tokens) or self._decode()
        else:
            decode = self._decode()
            if decode:
                chunks = self._prefill(min(cap, self.max_step_tokens - len(decode)))
                self.mixed_steps += bool(chunks)
                rows = decode + chunks
            else:
                rows = self._prefill(self.max_step_tokens)
        return rows or None

    def _prefill(self, budget: int) -> list[Row]:
        rows: list[Row] = []
        for seq in list(self.waiting):
            if seq.pending:                                     # preempted with a token on its way: not yet
                continue
            if budget <= 0 or (seq.slot < 0 and not self._fit(seq, None)):
                break                                           # first come first served: nobody skips ahead
            n = min(len(seq.tokens) - seq.num_computed, budget, seq.portion_cap or budget)
            if not self._fit(seq, seq.num_computed + n):
                break
            rows.append((seq, n, int(seq.num_computed + n == len(seq.tokens))))
            budget -= n
        return rows

    def _decode(self) -> list[Row]:
        rows: list[Row] = []
        for seq in list(self.running):
            if seq.status is not Status.RUNNING or self.at_limit(seq):   # preempted by a row above it
                continue
            total = seq.num_computed + 1
            if total <= self.cache.capacity(seq.slot) or self._fit(seq, total):
                rows.append((seq, 1, 1))
            else:
                self._preempt(seq)
        return rows

    def at_limit(self, seq: Seq) -> bool:
        n = len(seq.tokens) + seq.pending
        return n >= self.max_model_len or (seq.params.max_tokens is not None
                                           and n - seq.prompt_len >= seq.params.max_tokens)

    def _admit(self, seq: Seq) -> bool:
        slot = self.cache.admit()
        if slot is None:
            return False
        seq.slot = slot
        if seq.share_prefix:                       # the cached start of its tokens is not run again
            seq.num_computed = self.cache.adopt(slot, seq.tokens)
        if self.on_admit is not None:
            self.on_admit(seq)
        return True

    def _fit(self, seq: Seq, total: int | None) -> bool:
        """Admit `seq` (total None) or reserve pages for its first `total` tokens, preempting requests ranked below it,
        the lowest first, while releasing them can make room."""
        while not (self._admit(seq) if total is None else self.cache.reserve(seq.slot, total)):
            ranked = self.running + list(self.waiting)
            below = [s for s in ranked[ranked.index(seq) + 1:] if s.slot >= 0]
            if not below or not self.cache.could_fit(seq.slot if seq.slot >= 0 else None, total or 0,
                                                     [s.slot for s in below]):
                return False
            self._preempt(below[-1])
        return True

    def _preempt(self, seq: Seq) -> None:
        self.cache.release(seq.slot)
        seq.slot, seq.num_computed = -1, 0
        self.preemptions += 1
        if seq.status is Status.RUNNING:
            self.running.remove(seq)
            self.waiting.appendleft(seq)
            seq.status = Status.PREEMPTED

    def finished_prefill(self, seq: Seq) -> None:
        self.waiting.remove(seq)
        seq.status = Status.RUNNING
        self.running.append(seq)

    def finish(self, seq: Seq, reason: str) -> None:
        (self.running if seq.status is Status.RUNNING else self.waiting).remove(seq)
        if seq.slot >= 0:
            self.cache.release(seq.slot)
            seq.slot = -1
        seq.status, seq.finish_reason = Status.FINISHED, reason
