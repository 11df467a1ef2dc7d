"""How a layer's parts are wired. Pre-norm residual block: std/holon_std/blocks/units.py:8-25."""
from __future__ import annotations

import torch

from ..registry import register_part
from ..spec import PartRef
from .base import Build, Part


@register_part("block", "prenorm")
class PreNorm(Part):
    """a = mixer(input_norm(h)); h += a; x = post_norm(h); h += ffn(x). Every add is fused into the norm that reads
    its sum (the block's last add into the next reader's norm: `delta` is a term not yet added to `h`); all adds are
    in the activation dtype."""

    graph_safe = True

    def __init__(self, build: Build, *, layer: int, hidden: int, mixer: PartRef, ffn: PartRef, norm: PartRef) -> None:
        super().__init__(build)
        self.attach("input_norm", build.make(norm, dim=hidden))
        self.attach("mixer", build.make(mixer, layer=layer, hidden=hidden))
        self.attach("post_norm", build.make(norm, dim=hidden))
        self.attach("ffn", build.make(ffn, layer=layer, hidden=hidden))

    def forward(self, h: torch.Tensor, delta: torch.Tensor | None, step, site
                ) -> tuple[torch.Tensor, torch.Tensor | None]:
        """The residual stream is `h + delta` on entry and on return; `h` is updated in place. A part that can add
        its result into `h` inside its own kernel (`adds_residual`) is given `h`; it returns None when it did."""
        a = self.input_norm(h) if delta is None else self.input_norm.add(delta, h)[0]
        mixed = self.mixer(a, step, site, **({"residual": h} if self.mixer.adds_residual else {}))
        x = self.post_norm(h) if mixed is None else self.post_norm.add(mixed, h)[0]
        return h, self.ffn(x, step, **({"residual": h} if self.ffn.adds_residual else {}))

    __call__ = forward
