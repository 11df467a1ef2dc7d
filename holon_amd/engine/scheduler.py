"""Scheduling: which requests run in the next step and how many tokens each. Policy as in the reference
(core/holon/core/sched.py:65-217); the structure is this engine's own.

One line of requests in rank order. The first `n_running` of it decode (oldest first); the rest wait for their prompt,
or for what is left of it, in arrival order. A request that ends its prompt moves to the end of the decoding part; a
preempted one moves to the head of the waiting part. Rank decides who gives way when pages run out.

Without mixing (`chunk_with_decode` 0) a step is either prompt portions, of as many waiting requests as the token
budget `max_step_tokens` holds (a long prompt is cut where the budget ends), or one decoded token for every running
request; prompts go first. With mixing (`chunk_with_decode` C > 0) a step carries every running request's token and
then prompt portions of up to C tokens in all.

A portion may also be cut short by the model: a mixer whose state is kept on a grid of positions says through `cut`
where a portion that does not end the prompt may end (core/holon/core/sched.py:149-151).

When pages run out, a request takes them from the requests ranked below it, the lowest first, as many as the cache
manager says are needed; they give back everything, wait at the head of the line and later run their prompt and the
tokens they had generated again as one prompt (preemption by recompute). If not even all of them would make room,
nobody is preempted: a running request then gives way itself, a waiting one ends the step's admissions (first come,
first served: nobody behind it skips ahead). The pool always holds one request of `max_model_len` tokens (the engine
checks that at start), so the first in line always fits once the others have given way, and every step makes
progress.

A step may be scheduled while the one before it still runs (core/holon/core/sched.py:12-15, 98-104): a request whose
last drawn token has not reached the host (`pending`) decodes from the copy of it on the device; that token counts
towards its length limits; a preempted request waits for it before its tokens are run again as a prompt.
"""
from __future__ import annotations

from collections.abc import Callable
from typing import NamedTuple

from ..cache.manager import CacheManager
from .request import Seq, Status


class Portion(NamedTuple):
    """One row of a step: `count` next tokens of `seq`; `samples`: the last of them ends what the request has, so a
    token is drawn after it."""

    seq: Seq
    count: int
    samples: bool


class Scheduler:
    def __init__(self, cache: CacheManager, max_step_tokens: int, max_model_len: int, chunk_with_decode: int = 0,
                 on_admit: Callable[[Seq], None] | None = None,
                 cut: Callable[[int, int], int] | None = None) -> None:
        self.cache, self.max_step_tokens, self.max_model_len = cache, max_step_tokens, max_model_len
        self.chunk_with_decode = chunk_with_decode
        self.on_admit = on_admit
        self.cut = cut                     # (tokens computed, tokens offered) -> tokens a portion may take (0: none now)
        self.line: list[Seq] = []
        self.n_running = 0
        self.preemptions = 0
        self.mixed_steps = 0

    # -- the line -------------------------------------------------------------------------------------------------
    @property
    def running(self) -> list[Seq]:
        return self.line[: self.n_running]

    @property
    def waiting(self) -> list[Seq]:
        return self.line[self.n_running:]

    def __len__(self) -> int:
        return len(self.line)

    def add(self, seq: Seq, front: bool = False) -> None:
        """A new request joins the waiting part: at its end, or at its head (`front`)."""
        seq.status = Status.WAITING
        self.line.insert(self.n_running if front else len(self.line), seq)

    def prompt_done(self, seq: Seq) -> None:
        """Its prompt is in the cache and its first token drawn: it decodes from now on, ranked behind those that
        already do."""
        self.line.remove(seq)
        self.line.insert(self.n_running, seq)
        self.n_running += 1
        seq.status = Status.RUNNING

    def retire(self, seq: Seq, reason: str) -> None:
        """The request leaves the line for good and gives back what it holds."""
        at = self.line.index(seq)
        del self.line[at]
        self.n_running -= at < self.n_running
        if seq.admitted:
            self.cache.release(seq.slot)
            seq.slot = -1
        seq.status, seq.finish_reason = Status.FINISHED, reason

    def _evict(self, seq: Seq) -> None:
        """Preemption by recompute: everything it holds goes back; a decoding request returns to the head of the
        waiting part, a waiting one (part of its prompt computed) keeps its place."""
        self.cache.release(seq.slot)
        seq.slot, seq.num_computed = -1, 0
        self.preemptions += 1
        at = self.line.index(seq)
        if at < self.n_running:
            del self.line[at]
            self.n_running -= 1
            self.line.insert(self.n_running, seq)
            seq.status = Status.PREEMPTED

    # -- one step -------------------------------------------------------------------------------------------------
    def schedule(self) -> list[Portion] | None:
        """The next step's rows, decode rows before prompt portions; None when nothing can run."""
        rows: list[Portion] = []
        if self.chunk_with_decode:
            self._decode_rows(rows)
            n_decode = len(rows)
            left = self.max_step_tokens - n_decode
            self._prompt_rows(rows, min(self.chunk_with_decode, left) if n_decode else left)
            self.mixed_steps += 0 < n_decode < len(rows)
        else:
            self._prompt_rows(rows, self.max_step_tokens)
            if not rows:
                self._decode_rows(rows)
        return rows or None

    def _decode_rows(self, rows: list[Portion]) -> None:
        at = 0
        while at < self.n_running:                # the part shrinks when a request gives way
            seq = self.line[at]
            if seq.length_left(self.max_model_len) == 0:          # its last token is on its way
                at += 1
            elif self._room(seq, seq.num_computed + 1):
                rows.append(Portion(seq, 1, True))
                at += 1
            else:
                self._evict(seq)                  # nothing below it can make room: it gives way itself

    def _prompt_rows(self, rows: list[Portion], budget: int) -> None:
        for seq in self.waiting:                  # a copy: those that give way below keep their places
            if seq.pending:                       # preempted with a token still on its way: not yet
                continue
            if budget <= 0 or not (seq.admitted or self._seat(seq)):
                return
            count = min(seq.uncomputed, budget, seq.portion_cap or budget)      # after admission: a cached start counts
            if self.cut is not None and count < seq.uncomputed:
                count = self.cut(seq.num_computed, count)
            if count <= 0 or not self._room(seq, seq.num_computed + count):
                return
            rows.append(Portion(seq, count, count == seq.uncomputed))
            budget -= count

    # -- room -----------------------------------------------------------------------------------------------------
    def _below(self, seq: Seq) -> list[Seq]:
        """The admitted requests ranked below `seq`, the lowest first."""
        at = self.line.index(seq)
        return [s for s in reversed(self.line[at + 1:]) if s.admitted]

    def _seat(self, seq: Seq) -> bool:
        """A slot for a waiting request (and the cached start of its tokens, which is then not run again)."""
        slot = self.cache.admit()
        if slot is None:
            below = self._below(seq)
            if not below:
                return False
            self._evict(below[0])
            slot = self.cache.admit()
        seq.slot = slot
        if seq.share_prefix:
            seq.num_computed = self.cache.adopt(slot, seq.tokens)
        if self.on_admit is not None:
            self.on_admit(seq)
        return True

    def _room(self, seq: Seq, total: int) -> bool:
        """Pages for the first `total` tokens of `seq`, taken from requests below it if need be."""
        if total <= self.cache.capacity(seq.slot) or self.cache.reserve(seq.slot, total):
            return True
        below = self._below(seq)
        need = self.cache.victims_needed(seq.slot, total, [s.slot for s in below])
        if need is None:
            return False
        for victim in below[:need]:
            self._evict(victim)
        spare = below[need:]
        while not self.cache.reserve(seq.slot, total):            # the count was of pages as they stood: hold to it
            if not spare:
                return False
            self._evict(spare.pop(0))
        return True
