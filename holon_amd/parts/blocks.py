"""How a layer's parts are wired. Pre-norm residual block: std/holon_std/blocks/units.py:8-25."""
from __future__ import annotations

import torch

from ..registry import register_part
from ..spec import PartRef
from .base import Build, Part, Stream


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

    def finalize(self) -> None:
        """A mixer or feed-forward that can fold the norm in front of it into its own first product does so now (its
        weights are loaded and merged); it is then handed the norm deferred (`Normed`) instead of its result."""
        self._mixer_defers = self.input_norm.defer is not None and bool(self.mixer.absorb_norm(self.input_norm))
        self._ffn_defers = self.post_norm.defer is not None and bool(self.ffn.absorb_norm(self.post_norm))

    _mixer_defers = _ffn_defers = False

    def forward(self, stream: Stream, step, site) -> Stream:
        """The residual stream is `stream.h + stream.delta` on entry and on return; `h` is updated in place. A part
        that can add its result into `h` inside its own kernel (`adds_residual`) is given the stream; it returns None
        when it did (and the kernel leaves the rows' statistics in `stream.stats` for the norm that follows)."""
        h = stream.h
        if self._mixer_defers:
            a = self.input_norm.defer(h, stream.stats, stream.delta)
        elif stream.delta is not None:
            a = self.input_norm.add(stream.delta, h)[0]
        else:
            a = self.input_norm(h)
        stream.delta = stream.stats = None
        mixed = self.mixer(a, step, site, **({"residual": stream} if self.mixer.adds_residual else {}))
        if self._ffn_defers:
            x = self.post_norm.defer(h, stream.stats, mixed)
        elif mixed is not None:
            x = self.post_norm.add(mixed, h)[0]
        else:
            x = self.post_norm(h)
        stream.stats = None
        stream.delta = self.ffn(x, step, **({"residual": stream} if self.ffn.adds_residual else {}))
        return stream

    __call__ = forward
