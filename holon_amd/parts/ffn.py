"""Feed-forward parts. SwiGLU: std/holon_std/ffn/units.py:12-50, activation std/holon_std/ffn/reference.py:7-12."""
from __future__ import annotations

import torch

from ..registry import register_part
from .base import Build, Part, Stream
from .linear import Linear
from .norms import Normed


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

    def absorb_norm(self, norm: Part) -> bool:
        """Fold the norm in front of this part into its first product; it then takes `Normed` input."""
        return self.gate_up.absorb(norm)

    def forward(self, x: torch.Tensor | Normed, step=None, residual: Stream | None = None) -> torch.Tensor | None:
        gate_up, y = self.gate_up, None
        if gate_up.folds(x):
            y = self.kernels.linear_silu_mul(x.h, gate_up.weight, gate_up.tiled, row_scale=gate_up.row_scale(x))
        elif gate_up.reads_folded(x, gated=True):  # 17 to 64 rows: the folded copy over rows normed without the weight
            y = self.kernels.linear_silu_mul(x.unit_value(), gate_up.weight, gate_up.tiled)
        elif gate_up.folded is None:               # fused for steps of few rows
            x = x.value() if isinstance(x, Normed) else x
            y = self.kernels.linear_silu_mul(x, gate_up.weight, gate_up.tiled)
        if y is None:
            y = self.kernels.silu_mul(gate_up(x))
        return self.down_proj(y, residual=residual)

    __call__ = forward
