"""Norms. std/holon_std/ops/units.py:16-35 (`RMSNorm`), formula std/holon_std/ops/reference.py:7-18."""
from __future__ import annotations

import torch

from ..registry import register_part
from .base import Build, Part


class Normed:
    """norm(h) that has not been computed yet. A part that has folded this norm's weight into its own first product
    (`Linear.absorb`) takes `h` as it is and lets that product's kernel scale the rows; anyone else calls `value()`.
    `stats`: what the kernel that last wrote `h` left about its rows (partial sums of squares), or None."""

    def __init__(self, norm: "RMSNorm", h: torch.Tensor, stats: torch.Tensor | None = None) -> None:
        self.norm, self.h, self.stats = norm, h, stats
        self._value: torch.Tensor | None = None

    @property
    def shape(self) -> torch.Size:
        return self.h.shape

    def value(self) -> torch.Tensor:
        if self._value is None:
            self._value = self.norm(self.h)
        return self._value


@register_part("norm", "rmsnorm")
class RMSNorm(Part):
    """y = x * rsqrt(mean(x^2) + eps) * weight over the last `dim` values, float32 inside, rounded once."""

    graph_safe = True

    def __init__(self, build: Build, *, eps: float, dim: int) -> None:
        super().__init__(build)
        self.eps, self.dim = float(eps), dim
        self.declare("weight", (dim,), init="norm")

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return self.kernels.rmsnorm(x, self.weight, self.eps)

    __call__ = forward

    def add(self, x: torch.Tensor, residual: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
        """(norm(residual + x), residual + x); the sum replaces `residual` in place."""
        return self.kernels.add_rmsnorm(x, residual, self.weight, self.eps), residual

    def defer(self, h: torch.Tensor, stats: torch.Tensor | None = None) -> Normed:
        """norm(h) for a reader that may do the norm inside its own kernel."""
        return Normed(self, h, stats)

    def fusion(self) -> dict | None:
        """What a fused kernel needs to do this norm itself."""
        return {"norm": "rmsnorm", "eps": self.eps, "weight": self.weight}

