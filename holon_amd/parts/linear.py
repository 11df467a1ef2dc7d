"""Dense projection without bias, and the merge of several into one product.
std/holon_std/ops/units.py:189-277 (`Linear`, `merge`)."""
from __future__ import annotations

import torch

from .base import Build, Part


class Linear(Part):
    graph_safe = True

    def __init__(self, build: Build, *, inp: int, out: int) -> None:
        super().__init__(build)
        self.inp, self.out = inp, out
        self.declare("weight", (out, inp))
        self.tiled: torch.Tensor | None = None    # a second copy in the layout decode steps stream fastest

    def finalize(self) -> None:
        if self.weight is not None and self.build.decode_copy:
            self.tiled = self.kernels.tile_weight(self.weight)

    def forward(self, x: torch.Tensor, out_dtype: torch.dtype | None = None, residual: torch.Tensor | None = None
                ) -> torch.Tensor | None:
        """x W^T. With `residual`, the product is added into it in place when one kernel can do both (steps of few
        rows), and None is returned; otherwise the product is returned and the add is the caller's."""
        if residual is not None and out_dtype is None and self.kernels.linear_add(x, self.weight, self.tiled, residual):
            return None
        return self.kernels.linear(x, self.weight, out_dtype, self.tiled)

    __call__ = forward

    @staticmethod
    def merge(build: Build, *parts: "Linear") -> "Linear":
        """One projection whose rows are the parts' rows in order; the parts give up their tensors."""
        merged = Linear(build, inp=parts[0].inp, out=sum(p.out for p in parts))
        merged.weight = torch.cat([p.weight for p in parts], dim=0)
        for p in parts:
            p.weight = p.tiled = None
        merged.finalize()
        return merged
