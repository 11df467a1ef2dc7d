"""Plain sampling: the distribution a row is drawn from (float64) and the counter-based uniform, in Python integers.

Shares no code with `holon_amd.sampling`.
"""
from __future__ import annotations

import torch

M32 = 0xFFFFFFFF


def mix32(x: int) -> int:
    """lowbias32. std/holon_std/sampling/sampler.py:24-30."""
    x &= M32
    x ^= x >> 16
    x = (x * 0x7FEB352D) & M32
    x ^= x >> 15
    x = (x * 0x846CA68B) & M32
    x ^= x >> 16
    return x


def uniform(seed: int, position: int) -> float:
    """One uniform in (0, 1) from (seed, position), 24 bits, as a float32 value.
    std/holon_std/sampling/sampler.py:33-40."""
    h = mix32(seed & M32) ^ ((seed >> 32) & M32) ^ mix32(position & M32)
    h = mix32(h)
    u = torch.tensor(float(h >> 8), dtype=torch.float32)
    u = (u + 0.5) * torch.tensor(2.0 ** -24, dtype=torch.float32)
    return float(torch.clamp(u, max=1 - 2.0 ** -24))


def sequence_seed(seed: int, index: int) -> int:
    """core/holon/api/batch.py:64-77."""
    base = seed & (2 ** 63 - 1)
    if index == 0:
        return base
    x = (base + index + 0x9E3779B97F4A7C15) & 0xFFFFFFFFFFFFFFFF
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9 & 0xFFFFFFFFFFFFFFFF
    x = (x ^ (x >> 27)) * 0x94D049BB133111EB & 0xFFFFFFFFFFFFFFFF
    return (x ^ (x >> 31)) & (2 ** 63 - 1)


def probs(logits: torch.Tensor, temperature: float, top_k: int = 0, top_p: float = 1.0, min_p: float = 0.0
          ) -> torch.Tensor:
    """The law of one row [V] in float64: temperature, then top-k, then top-p over the renormalised rest (the most
    likely token always stays), then min-p against the largest probability after top-k; temperature 0 is one-hot at
    the first maximum. std/holon_std/sampling/reference.py:13-30. The logits are divided by the temperature in
    float32, as the reference's sampler divides them (std/holon_std/sampling/sampler.py:137): which values are equal
    after that decides ties at a filter's edge."""
    x = logits.double()
    if temperature == 0:
        return torch.nn.functional.one_hot(x.argmax(), x.numel()).double()
    x = scaled(logits, temperature)
    keep = torch.ones_like(x, dtype=torch.bool)
    order = x.argsort(descending=True, stable=True)
    if top_k > 0:
        keep[order[top_k:]] = False
    q = torch.where(keep, x, float("-inf")).softmax(-1)
    if top_p < 1:
        sorted_q = q[order]
        keep[order[sorted_q.cumsum(-1) - sorted_q > top_p]] = False
    if min_p > 0:
        keep &= q >= min_p * q.max()
    return torch.where(keep, x, float("-inf")).softmax(-1)


def scaled(logits: torch.Tensor, temperature: float) -> torch.Tensor:
    """logits / temperature as a float32 division, in float64 for what follows. The divisor is a tensor of the logits'
    shape: by a scalar, torch may multiply by the reciprocal instead, which is not the same in the last place."""
    return (logits.float() / torch.full_like(logits, temperature, dtype=torch.float32)).double()


def drawing_order(logits: torch.Tensor, temperature: float, top_k: int = 0, top_p: float = 1.0, min_p: float = 0.0
                  ) -> torch.Tensor | None:
    """The order in which a row's tokens are walked by the draw: vocabulary order (None) when no filter is set, else
    by scaled logit, largest first, equal ones by index (the sort the filters use). The reference sorts every row of a
    batch in which any row has a filter; here a row's order is its own, so that its draws do not depend on the batch.
    std/holon_std/sampling/sampler.py:43-54,134-141."""
    if temperature == 0 or not (top_k > 0 or top_p < 1 or min_p > 0):
        return None
    return scaled(logits, temperature).argsort(descending=True, stable=True)


def draw(q: torch.Tensor, u: float, order: torch.Tensor | None = None) -> int:
    """Inverse CDF over the tokens in `order` (vocabulary order when None): the first whose cumulative mass exceeds
    u * total. std/holon_std/sampling/sampler.py:57-61."""
    q = q.double()
    c = (q if order is None else q[order]).cumsum(-1)
    idx = int(torch.searchsorted(c, torch.tensor(u, dtype=torch.float64) * c[-1], right=True))
    idx = min(idx, q.numel() - 1)
    return idx if order is None else int(order[idx])
