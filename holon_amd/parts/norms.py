"""Norms. std/holon_std/ops/units.py:16-35 (`RMSNorm`), formula std/holon_std/ops/reference.py:7-18."""
from __future__ import annotations

import torch

from ..registry import register_part
from .base import Build, NormPart, PartialSums


def _term(x: "torch.Tensor | PartialSums") -> torch.Tensor:
    """What the add + norm kernel is given: a tensor, or the parts of a product that came as partial sums."""
    return x.parts if isinstance(x, PartialSums) else x


class Normed:
    """norm(h), or norm(h + delta), that has not been computed yet. A part that has folded this norm's weight into its
    own first product (`Linear.absorb`) may take `h` as it is and let that product's kernel scale the rows (few rows,
    no pending `delta`), or take the rows normed without the norm's weight (`unit_value`) for a product that reads the
    folded weights; anyone else calls `value()`. With `delta`, whichever is computed first adds it into `h` in place.
    `stats`: what the kernel that last wrote `h` left about its rows (partial sums of squares), or None."""

    def __init__(self, norm: "RMSNorm", h: torch.Tensor, stats: torch.Tensor | None = None,
                 delta: "torch.Tensor | PartialSums | None" = None) -> None:
        self.norm, self.h, self.stats, self.delta = norm, h, stats, delta
        self._value: torch.Tensor | None = None
        self._unit: torch.Tensor | None = None

    @property
    def shape(self) -> torch.Size:
        return self.h.shape

    def _take_delta(self) -> torch.Tensor | None:
        delta, self.delta = self.delta, None
        return delta

    def value(self) -> torch.Tensor:
        if self._value is None:
            delta = self._take_delta()
            self._value = self.norm(self.h) if delta is None else self.norm.add(delta, self.h)[0]
        return self._value

    def unit_value(self) -> torch.Tensor:
        """The rows normed but not multiplied by the norm's weight: what a product over folded weights reads."""
        if self._unit is None:
            self._unit = self.norm.unit(self.h, self._take_delta())
        return self._unit


@register_part("norm", "rmsnorm")
class RMSNorm(NormPart):
    """y = x * rsqrt(mean(x^2) + eps) * weight over the last `dim` values, float32 inside, rounded once."""

    graph_safe = True

    def __init__(self, build: Build, *, eps: float, dim: int) -> None:
        super().__init__(build)
        self.eps, self.dim = float(eps), dim
        self.declare("weight", (dim,), init="norm")

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return self.kernels.rmsnorm(x, self.weight, self.eps)

    __call__ = forward

    def add(self, x: "torch.Tensor | PartialSums", residual: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
        """(norm(residual + x), residual + x); the sum replaces `residual` in place."""
        return self.kernels.add_rmsnorm(_term(x), residual, self.weight, self.eps), residual

    def defer(self, h: torch.Tensor, stats: torch.Tensor | None = None, delta: torch.Tensor | None = None) -> Normed:
        """norm(h), or norm(h + delta) with the sum replacing `h`, for a reader that may do the norm, or the
        multiplication by its weight, inside its own kernel."""
        return Normed(self, h, stats, delta)

    def unit(self, h: torch.Tensor, delta: torch.Tensor | None = None) -> torch.Tensor:
        """h * rsqrt(mean(h^2) + eps), the norm without its weight; with `delta`, of h + delta, which replaces `h`."""
        if self._ones is None:
            self._ones = torch.ones_like(self.weight)
        if delta is None:
            return self.kernels.rmsnorm(h, self._ones, self.eps)
        return self.kernels.add_rmsnorm(_term(delta), h, self._ones, self.eps)

    _ones: torch.Tensor | None = None

    def fusion(self) -> dict | None:
        """What a fused kernel needs to do this norm itself."""
        return {"norm": "rmsnorm", "eps": self.eps, "weight": self.weight}

