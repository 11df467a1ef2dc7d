"""Dense projection without bias, and the merge of several into one product.
std/holon_std/ops/units.py:189-277 (`Linear`, `merge`)."""
from __future__ import annotations

import torch

from .base import Build, PartialSums, Part, Stream
from .norms import Normed, RMSNorm


class Linear(Part):
    graph_safe = True

    def __init__(self, build: Build, *, inp: int, out: int) -> None:
        super().__init__(build)
        self.inp, self.out = inp, out
        self.declare("weight", (out, inp))
        self.tiled: torch.Tensor | None = None    # a second copy in the layout decode steps stream fastest
        self.folded: RMSNorm | None = None        # the norm whose weight the tiled copy has folded in, if any

    def finalize(self) -> None:
        if self.weight is not None and self.build.decode_copy:
            self.tiled = self.kernels.tile_weight(self.weight)

    def extra_tensors(self) -> list[torch.Tensor]:
        return [self.tiled] if self.tiled is not None else []

    def absorb(self, norm: Part) -> bool:
        """Fold the weight of the norm in front of this projection into the tiled copy, so that steps of few rows
        need no kernel for the norm: the product runs over the un-normed rows and scales each by the norm's factor
        (`forward` with a `Normed`). The tiled copy then serves only such input. False when this norm or this weight
        cannot be folded; nothing changes then."""
        spec = norm.fusion()
        if not self.build.decode_copy or self.weight is None or spec is None or spec.get("norm") != "rmsnorm" \
                or spec["weight"] is None:
            return False
        folded = self.kernels.tile_weight(self.weight, spec["weight"])
        if folded is None:
            return False
        self.tiled, self.folded = folded, norm
        return True

    def folds(self, x: torch.Tensor | Normed) -> bool:
        """Whether `x` is the deferred norm this projection folded, with nothing left to add to its rows, at a number
        of rows its kernel serves."""
        return isinstance(x, Normed) and x.norm is self.folded and x.delta is None and \
            self.kernels.folds_norm(x.h.shape[0], self.weight, self.tiled)

    def reads_folded(self, x: torch.Tensor | Normed, gated: bool = False) -> bool:
        """Whether `x` is the deferred norm this projection folded, at a number of rows whose product reads the folded
        copy over rows normed without the norm's weight."""
        return isinstance(x, Normed) and x.norm is self.folded and \
            self.kernels.serves_rows(x.h.shape[0], self.weight, self.tiled, gated)

    def row_scale(self, x: Normed) -> tuple[torch.Tensor, float]:
        stats = x.stats if x.stats is not None else self.kernels.row_sumsq(x.h)
        return stats, x.norm.eps

    def forward(self, x: torch.Tensor | Normed, out_dtype: torch.dtype | None = None, residual: Stream | None = None
                ) -> "torch.Tensor | PartialSums | None":
        """x W^T. With `residual`, the product is added into the stream's rows in place when one kernel can do both
        (steps of few rows), which also leaves the rows' statistics there, and None is returned; otherwise the
        product is returned and the add is the caller's. It may then come as `PartialSums` (a narrow weight at 17 to
        128 rows, or up to 1,024 where its K is well above its N: K split over blocks), which the norm that adds it
        reads as they are."""
        if isinstance(x, Normed):
            if self.folds(x):
                return self.kernels.linear(x.h, self.weight, out_dtype, self.tiled, row_scale=self.row_scale(x))
            if self.reads_folded(x):
                return self.kernels.linear(x.unit_value(), self.weight, out_dtype, self.tiled)
            x = x.value()
        tiled = self.tiled if self.folded is None else None       # a folded copy is not this weight any more
        if residual is not None and out_dtype is None:
            done = self.kernels.linear_add(x, self.weight, tiled, residual.h, want_stats=True)
            if done is not False:
                residual.stats = done if isinstance(done, torch.Tensor) else None
                return None
            parts = self.kernels.linear_parts(x, self.weight, tiled)
            if parts is not None:
                return PartialSums(parts, self.kernels, x.dtype)
        return self.kernels.linear(x, self.weight, out_dtype, tiled)

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
