"""Feed-forward parts. SwiGLU: std/holon_std/ffn/units.py:12-50, activation std/holon_std/ffn/reference.py:7-12."""
from __future__ import annotations

import torch

from ..registry import register_part
from .base import Build, Part
from .linear import Linear


@register_part("ffn", "swiglu")
class SwiGLU(Part):
    """down(silu(gate(x)) * up(x)); gate and up are merged into one product after loading (gate rows first)."""

    graph_safe = True

    def __init__(self, build: Build, *, inter: int, hidden: int, layer: int) -> None:
        super().__init__(build)
        self.inter, self.hidden = inter, hidden
        self.attach("gate_proj", Linear(build, inp=hidden, out=inter))
        self.attach("up_proj", Linear(build, inp=hidden, out=inter))
        self.attach("down_proj", Linear(build, inp=inter, out=hidden))
        self.gate_up: Linear | None = None

    def finalize(self) -> None:
        self.gate_up = Linear.merge(self.build, self.gate_proj, self.up_proj)
        self.drop("gate_proj")
        self.drop("up_proj")
        self._children["gate_up"] = self.gate_up

    adds_residual = True

    def forward(self, x: torch.Tensor, step=None, residual: torch.Tensor | None = None) -> torch.Tensor | None:
        y = self.kernels.linear_silu_mul(x, self.gate_up.weight, self.gate_up.tiled)   # fused for steps of few rows
        if y is None:
            y = self.kernels.silu_mul(self.gate_up(x))
        return self.down_proj(y, residual=residual)

    __call__ = forward
