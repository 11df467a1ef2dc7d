"""Requests as the engine tracks them, and what it streams back.
core/holon/api/batch.py:80-104 (`Seq`), core/holon/api/frontend.py:26-52 (`TokenDelta`)."""
from __future__ import annotations

import dataclasses
import enum
from collections.abc import Collection

from ..config.engine import SamplingParams


class Status(enum.Enum):
    WAITING = "waiting"
    RUNNING = "running"
    PREEMPTED = "preempted"
    FINISHED = "finished"


@dataclasses.dataclass(eq=False)
class Seq:
    rid: str
    tokens: list[int]                    # prompt and generated tokens
    params: SamplingParams
    prompt_len: int = 0
    slot: int = -1                       # its row in the cache's tables while admitted
    num_computed: int = 0                # tokens whose state is in the cache
    status: Status = Status.WAITING
    finish_reason: str | None = None
    pending: int = 0                     # tokens drawn for it that have not reached the host yet
    index: int = 0                       # which of its request's `n` sequences
    portion_cap: int = 0                 # most prompt tokens one step runs of it (0: what the budget allows)
    share_prefix: bool = True            # False: every position is computed, whatever the cache holds
    cached_tokens: int | None = None     # what the prefix cache served at its first admission
    reported: bool = False               # its first delta has gone out

    def __post_init__(self) -> None:
        if not self.prompt_len:
            self.prompt_len = len(self.tokens)

    @property
    def admitted(self) -> bool:
        return self.slot >= 0

    @property
    def uncomputed(self) -> int:
        """Tokens it has that the cache does not hold yet."""
        return len(self.tokens) - self.num_computed

    def length_left(self, max_model_len: int, in_flight: bool = True) -> int:
        """How many more tokens it may be given before a length limit ends it. `in_flight` counts the tokens drawn for
        it that are still on their way to the host: a request at its limit with tokens in flight is not scheduled
        again (core/holon/core/sched.py:163-170)."""
        have = len(self.tokens) + (self.pending if in_flight else 0)
        left = max_model_len - have
        if self.params.max_tokens is not None:
            left = min(left, self.params.max_tokens - (have - self.prompt_len))
        return max(left, 0)

    def verdict(self, token: int, eos: Collection[int], max_model_len: int) -> str | None:
        """Whether `token`, just appended, ends the sequence: "stop" for an end-of-sequence token (unless ignored) or
        one of the request's stop tokens, "length" at `max_tokens` or `max_model_len`. The finishing token is part
        of the output (core/holon/core/engine.py:702-709)."""
        if token in self.params.stop_token_ids or (token in eos and not self.params.ignore_eos):
            return "stop"
        return "length" if self.length_left(max_model_len, in_flight=False) == 0 else None


@dataclasses.dataclass
class Logprobs:
    """Per emitted token: its log-probability, and the ids and log-probabilities of the k most likely tokens (of the
    raw logits, before temperature: std/holon_std/sampling/sampler.py:147-152)."""

    token: list[float]
    top_ids: list[list[int]]
    top: list[list[float]]


@dataclasses.dataclass
class TokenDelta:
    """New tokens of one request; `finish_reason` ("stop" | "length" | "abort") on its last delta."""

    rid: str
    token_ids: list[int]
    finish_reason: str | None = None
    logprobs: Logprobs | None = None
    index: int = 0                       # which of the request's `n` sequences
    prompt_logprobs: Logprobs | None = None   # with the first delta: prompt positions 1 .. n-1 (the first has no context)
    cached_tokens: int | None = None     # with the first delta: tokens the prefix cache served at the first admission
