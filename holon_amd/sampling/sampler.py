"""The sampler: per-slot parameters, one kernel call per step.

Semantics follow the reference (std/holon_std/sampling/reference.py:1-30, sampler.py:24-61): logits / temperature, then
top-k, then top-p over the renormalised rest (the most likely token always stays), then min-p against the largest
probability after top-k; temperature 0 is the first maximal index. The draw is an inverse CDF at a counter-based
uniform, a hash of (seed, position of the token being drawn): no generator state, so what a request draws does not
depend on batching, chunking or preemption. Where the reference walks filtered rows in sorted order, this sampler
walks every row in vocabulary order (the law is the same; the token drawn for one uniform may differ).
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
    def __init__(self, kernels, max_seqs: int, device: torch.device) -> None:
        self.kernels, self.device = kernels, device
        n = max_seqs + 1
        self.temperature = np.zeros(n, dtype=np.float32)
        self.top_k = np.zeros(n, dtype=np.int32)
        self.top_p = np.ones(n, dtype=np.float32)
        self.min_p = np.zeros(n, dtype=np.float32)
        self.seed = np.zeros(n, dtype=np.int64)

    def admit(self, slot: int, params: SamplingParams) -> None:
        if params.seed is None:
            raise ValueError("the engine gives every request a concrete seed")
        self.temperature[slot], self.top_k[slot] = params.temperature, params.top_k
        self.top_p[slot], self.min_p[slot] = params.top_p, params.min_p
        self.seed[slot] = params.seed & SEED_MASK

    def sample(self, logits: torch.Tensor, slots: np.ndarray, positions: np.ndarray) -> torch.Tensor:
        """logits [R, V] float32; row r belongs to `slots[r]` and draws the token at `positions[r]`. -> [R] int32."""
        if not self.temperature[slots].any():
            return self.kernels.argmax(logits)
        dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(self.device, non_blocking=True)
        return self.kernels.sample(logits, dev(self.temperature[slots]), dev(self.top_k[slots]),
                                   dev(self.top_p[slots]), dev(self.min_p[slots]), dev(self.seed[slots]),
                                   dev(positions.astype(np.int64)))
