"""Trace replay: feed given token ids through the model step by step and hand back the logits that are asked for.
Nothing is sampled. The replayer owns no forward pass, cache or loader: it allocates through the cache manager and
calls the step function, the same ones generation uses."""
from __future__ import annotations

import torch

from .batch import StepRow
from .loading import Loaded


class Replayer:
    def __init__(self, loaded: Loaded) -> None:
        self.loaded = loaded
        self.cache, self.runner = loaded.cache, loaded.runner
        self.slots: dict[str, int] = {}
        self.fed: dict[str, int] = {}

    def step(self, entries: list[dict], end: list[str] = ()) -> torch.Tensor | None:
        """`entries`: [{"id", "tokens", "want"}]; returns float32 logits [wanted, vocab] in the order of the entries
        and of each `want`, or None when nothing is wanted. Requests in `end` give back what they hold afterwards."""
        rows, admitted = [], []
        try:
            for e in entries:
                rid, tokens = str(e["id"]), list(e["tokens"])
                if rid not in self.slots:
                    slot = self.cache.admit()
                    if slot is None:
                        raise RuntimeError(f"request {rid}: all {self.cache.max_seqs} slots are taken")
                    self.slots[rid], self.fed[rid] = slot, 0
                    admitted.append(rid)
                slot, start = self.slots[rid], self.fed[rid]
                if not self.cache.reserve(slot, start + len(tokens)):
                    raise RuntimeError(f"request {rid}: the cache has no pages left for {start + len(tokens)} tokens")
                rows.append(StepRow(slot, start, tokens, list(e.get("want", []))))
            logits = self.runner.run(rows) if rows else None
        except Exception:
            for rid in admitted:                   # a refused step leaves no request behind that it brought
                self.cache.release(self.slots.pop(rid))
                del self.fed[rid]
            raise
        for e in entries:
            self.fed[str(e["id"])] += len(e["tokens"])
        for rid in end:
            rid = str(rid)
            if rid in self.slots:
                self.cache.release(self.slots.pop(rid))
                del self.fed[rid]
        return logits
