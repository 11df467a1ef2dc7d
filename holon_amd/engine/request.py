"""Requests as the engine tracks them, and what it streams back.
core/holon/api/batch.py:80-104 (`Seq`), core/holon/api/frontend.py:26-52 (`TokenDelta`)."""
from __future__ import annotations

import dataclasses
import enum

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
