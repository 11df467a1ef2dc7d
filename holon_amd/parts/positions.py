"""Position encodings applied to queries and keys inside a mixer.
std/holon_std/ops/units.py:38-63 (`Rope`), formula std/holon_std/ops/reference.py:21-30, table layout
std/holon_std/ops/kernels.py:7-12."""
from __future__ import annotations

import torch

from ..registry import register_part
from .base import Build, Part


def rope_table(max_positions: int, rotary_dim: int, theta: float) -> torch.Tensor:
    """[max_positions, rotary_dim] float32: cos(p * theta^(-2i/rotary_dim)) for i < rotary_dim/2, then the sines.
    Computed on the host in float32, in the reference's order of operations."""
    inv_freq = 1.0 / (theta ** (torch.arange(0, rotary_dim, 2, dtype=torch.float32) / rotary_dim))
    angles = torch.arange(max_positions, dtype=torch.float32)[:, None] * inv_freq[None, :]
    return torch.cat((angles.cos(), angles.sin()), dim=-1).contiguous()


@register_part("position", "rope")
class Rope(Part):
    """Rotary embedding, half-split ("neox") pairing: dims (i, i + rotary_dim/2) rotate by position * theta_i; dims
    beyond `rotary_dim` pass through."""

    graph_safe = True

    def __init__(self, build: Build, *, theta: float, head_dim: int, rotary_dim: int | None = None) -> None:
        super().__init__(build)
        self.theta, self.head_dim = float(theta), head_dim
        self.rotary_dim = head_dim if rotary_dim is None else rotary_dim
        if self.rotary_dim % 2 or not 0 < self.rotary_dim <= head_dim:
            raise ValueError(f"rotary_dim {self.rotary_dim} must be even and within head_dim {head_dim}")
        self.table = rope_table(build.max_model_len, self.rotary_dim, self.theta).to(build.device)

    def apply(self, q: torch.Tensor, k: torch.Tensor | None, positions: torch.Tensor) -> None:
        """Rotate q [T, Hq, D] and k [T, Hkv, D] in place."""
        self.kernels.rope(q, positions, self.table)
        if k is not None:
            self.kernels.rope(k, positions, self.table)

    def fusion(self) -> dict | None:
        return {"position": "rope", "table": self.table}


@register_part("position", "none")
class NoPosition(Part):
    """No position encoding (order enters through the causal mask alone)."""

    graph_safe = True

    def __init__(self, build: Build, *, head_dim: int) -> None:
        super().__init__(build)

    def apply(self, q: torch.Tensor, k: torch.Tensor | None, positions: torch.Tensor) -> None:
        return None

    def fusion(self) -> dict | None:
        return {"position": "none", "table": None}
