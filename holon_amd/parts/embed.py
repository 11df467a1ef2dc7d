"""Token embedding and the output head. std/holon_std/ops/units.py:280-348 (`Embedding`, `LMHead`)."""
from __future__ import annotations

import torch

from ..registry import register_part
from .base import Build, EmbedPart, Part


@register_part("embed", "table")
class Embedding(EmbedPart):
    graph_safe = True

    def __init__(self, build: Build, *, vocab: int, hidden: int) -> None:
        super().__init__(build)
        self.declare("weight", (vocab, hidden))

    def rows(self, ids: torch.Tensor) -> torch.Tensor:
        return self.kernels.embedding(ids, self.weight)

    def forward(self, ids: torch.Tensor, take: tuple[torch.Tensor, torch.Tensor] | None = None,
                want_stats: bool = False):
        """Rows of the table; `take`: where a token is still on the device, see the kernel contract. With
        `want_stats`: (rows, their statistics for a norm that follows, or None)."""
        return self.kernels.embedding(ids, self.weight, take, want_stats)

    __call__ = forward


@register_part("head", "linear")
class LMHead(Part):
    """Logits in float32. A tied head owns no tensor: it reads the embedding's."""

    graph_safe = True

    def __init__(self, build: Build, *, vocab: int, hidden: int, tied: bool, embed: Embedding) -> None:
        super().__init__(build)
        self.tied = tied
        self._embed = [embed]                     # in a list: the embedding part keeps the one owner of the tensor
        self.tiled: torch.Tensor | None = None
        if not tied:
            self.declare("weight", (vocab, hidden))

    def _weight(self) -> torch.Tensor:
        return self._embed[0].weight if self.tied else self.weight

    def finalize(self) -> None:
        if self.build.decode_copy and self._weight() is not None:
            self.tiled = self.kernels.tile_weight(self._weight())

    def extra_tensors(self) -> list[torch.Tensor]:
        return [self.tiled] if self.tiled is not None else []

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        return self.kernels.linear(h, self._weight(), torch.float32, self.tiled)

    __call__ = forward
