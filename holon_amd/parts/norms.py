"""Norms. std/holon_std/ops/units.py:16-35 (`RMSNorm`), formula std/holon_std/ops/reference.py:7-18."""
from __future__ import annotations

import torch

from ..registry import register_part
from .base import Build, Part


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

    def fusion(self) -> dict | None:
        """What a fused kernel needs to do this norm itself."""
        return {"norm": "rmsnorm", "eps": self.eps, "weight": self.weight}

