"""The sampler: per-slot parameters, one kernel call per step.

Semantics follow the reference (std/holon_std/sampling/reference.py:1-30, sampler.py:24-61): logits / temperature, then
top-k, then top-p over the renormalised rest (the most likely token always stays), then min-p against the largest
probability after top-k; temperature 0 is the first maximal index. The draw is an inverse CDF at a counter-based
uniform, a hash of (seed, position of the token being drawn): no generator state, so what a request draws does not
depend on batching, chunking or preemption. The inverse CDF walks a row without a filter in vocabulary order and a row
with one (top-k, top-p or min-p set) in the filters' sorted order, largest value first and equal values by index, as the
reference does (sampler.py:43-61). One difference remains on purpose: the reference sorts every row of a batch as soon
as any of its rows has a filter (sampler.py:134-141), so that an unfiltered request's draw depends on its neighbours;
here a row's order is its own.
"""
from __future__ import annotations

import numpy as np
import torch

from ..config.engine import SamplingParams

SEED_MASK = 2 ** 63 - 1


def sequence_seed(seed: int, index: int) -> int:
    """The seed of sequence `index` of a request seeded `seed`: sequence 0 keeps it (core/holon/api/batch.py:64-77)."""
    base = seed & SEED_MASK
    if index == 0:
        return base
    x = (base + index + 0x9E3779B97F4A7C15) & 0xFFFFFFFFFFFFFFFF
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9 & 0xFFFFFFFFFFFFFFFF
    x = (x ^ (x >> 27)) * 0x94D049BB133111EB & 0xFFFFFFFFFFFFFFFF
    return (x ^ (x >> 31)) & SEED_MASK


class Sampler:
    """Per-slot parameters live on the device (std/holon_std/sampling/sampler.py:64-89): a request's are written when
    it is admitted, and a step's kernel reads them by the rows' slots, so a sampled step uploads nothing but, at
    most, which slots and positions its rows have. Host mirrors decide the path (all greedy: argmax)."""

    FIELDS = (("temperature", torch.float32, 0.0), ("top_k", torch.int32, 0), ("top_p", torch.float32, 1.0),
              ("min_p", torch.float32, 0.0), ("seed", torch.int64, 0))

    def __init__(self, kernels, max_seqs: int, device: torch.device) -> None:
        self.kernels, self.device = kernels, device
        n = max_seqs + 1
        pinned = device.type == "cuda"
        self._host = {name: torch.full((n,), fill, dtype=dt, pin_memory=pinned) for name, dt, fill in self.FIELDS}
        self._dev = {name: t.to(device) for name, t in self._host.items()}
        for name, t in self._host.items():        # numpy views of the mirrors: self.temperature[slot] = ...
            setattr(self, name, t.numpy())
        self._stale = False                        # a mirror changed since the tables were last copied
        self._copied: "torch.cuda.Event | None" = None

    def admit(self, slot: int, params: SamplingParams) -> None:
        if params.seed is None:
            raise ValueError("the engine gives every request a concrete seed")
        if self._copied is not None:               # the last copy of the mirrors must have read them before they change
            self._copied.synchronize()
            self._copied = None
        self.temperature[slot], self.top_k[slot] = params.temperature, params.top_k
        self.top_p[slot], self.min_p[slot] = params.top_p, params.min_p
        self.seed[slot] = params.seed & SEED_MASK
        self._stale = True

    def _tables(self) -> list[torch.Tensor]:
        if self._stale:
            for name, host in self._host.items():
                self._dev[name].copy_(host, non_blocking=True)
            if self.device.type == "cuda":
                self._copied = torch.cuda.Event()
                self._copied.record()
            self._stale = False
        return [self._dev[name] for name, _, _ in self.FIELDS]

    def sample(self, logits: torch.Tensor, slots: np.ndarray, positions: np.ndarray,
               on_device: tuple[torch.Tensor, torch.Tensor] | None = None) -> torch.Tensor:
        """logits [R, V] float32; row r belongs to `slots[r]` and draws the token at `positions[r]`. -> [R] int32.
        `on_device`: the same slots and positions as int32 device tensors, when the step already has them there."""
        if not self.temperature[slots].any():
            return self.kernels.argmax(logits)
        if on_device is None:
            both = torch.from_numpy(np.concatenate((slots, positions)).astype(np.int32))
            if self.device.type == "cuda":
                both = both.pin_memory()
            both = both.to(self.device, non_blocking=True)
            on_device = (both[: len(slots)], both[len(slots):])
        return self.kernels.sample(logits, *self._tables(), on_device[1], on_device[0])
