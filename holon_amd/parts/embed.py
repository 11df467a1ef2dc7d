"""Token embedding and the output head. std/holon_std/ops/units.py:280-348 (`Embedding`, `LMHead`)."""
from __future__ import annotations

import torch

from ..registry import register_part
from .base import Build, Part


@register_part("embed", "table")
class Embedding(Part):
    def __init__(self, build: Build, *, vocab: int, hidden: int) -> None:
        super().__init__(build)
        self.declare("weight", (vocab, hidden))

    def forward(self, ids: torch.Tensor) -> torch.Tensor:
        return self.kernels.embedding(ids, self.weight)

    __call__ = forward


@register_part("head", "linear")
class LMHead(Part):
    """Logits in float32. A tied head owns no tensor: it reads the embedding's."""

    def __init__(self, build: Build, *, vocab: int, hidden: int, tied: bool, embed: Embedding) -> None:
        super().__init__(build)
        self.tied = tied
        self._embed = [embed]                     # in a list: the embedding part keeps the one owner of the tensor
        if not tied:
            self.declare("weight", (vocab, hidden))

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        weight = self._embed[0].weight if self.tied else self.weight
        return self.kernels.linear(h, weight, torch.float32)

    __call__ = forward
