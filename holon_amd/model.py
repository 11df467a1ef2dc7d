"""A model built from a spec: embedding, blocks in run order, final norm, head.
core/holon/core/build.py:273-314 (`Model`, `build_model`)."""
from __future__ import annotations

import dataclasses

import torch

from .parts.base import Build, PagedState, Part, SlotState, Stream
from .spec import ModelSpec


@dataclasses.dataclass
class SitePages:
    """One paged state of one run: the group whose block table addresses it, and its storage."""

    group: int
    pages: torch.Tensor                           # [num_pages, P * elems]


@dataclasses.dataclass
class Site:
    """One entry of the run order as the cache sees it: which layer runs, which cache it uses and whether it writes
    it. The cache manager fills `paged` and `slot_state` when it allocates: one entry for every state the run's mixer
    declares, by the declaration's name. `group` and `pages` are those of the first paged state declared (all there
    is for a mixer that keeps one)."""

    run: int
    layer: int
    writes: bool = True
    owner: int | None = None                      # the run whose cache this one reads (None: its own)
    group: int | None = None                      # paged group id
    pages: torch.Tensor | None = None             # this site's page storage [num_pages, P * elems]
    paged: dict[str, SitePages] = dataclasses.field(default_factory=dict)
    slot_state: dict[str, torch.Tensor] = dataclasses.field(default_factory=dict)   # name -> [S+1, *shape]

    def detach(self) -> None:
        """Forget the storage a cache manager gave (before another one is made for the same model)."""
        self.group, self.pages, self.paged, self.slot_state = None, None, {}, {}


class Model(Part):
    graph_safe = True

    def __init__(self, spec: ModelSpec, build: Build) -> None:
        super().__init__(build)
        self.spec = spec
        self.attach("embed", build.make(spec.embed, vocab=spec.vocab, hidden=spec.hidden))
        self.blocks: list[Part] = []
        for i, layer in enumerate(spec.layers):
            block = build.make(layer.block, layer=i, hidden=spec.hidden, mixer=layer.mixer, ffn=layer.ffn,
                               norm=layer.norm)
            self.blocks.append(self.attach(f"layers.{i}", block))
        self.attach("norm", build.make(spec.norm, dim=spec.hidden))
        self.attach("lm_head", build.make(spec.head, vocab=spec.vocab, hidden=spec.hidden, embed=self.embed))
        self.sites = [Site(run=at, layer=r.layer, writes=r.reads is None, owner=r.reads)
                      for at, r in enumerate(spec.order)]

    def state_decls(self) -> list[list[PagedState | SlotState]]:
        """Per run, what its mixer keeps between steps (empty for a run that reads another's cache)."""
        out = []
        for site in self.sites:
            mixer = getattr(self.blocks[site.layer], "mixer", None)
            out.append(list(mixer.state()) if mixer is not None and site.writes else [])
        return out

    def cut(self, start: int, count: int) -> int:
        """Where a prompt portion of `count` tokens from position `start` may end, by every part's own `cut`."""
        for part in self.walk():
            if part is not self and count > 0:
                count = min(count, max(0, part.cut(start, count)))
        return count

    def trunk(self, step) -> tuple[torch.Tensor, torch.Tensor | None]:
        """The residual stream after every run, as (h, delta) with h + delta the stream [T, hidden]."""
        h, stats = self.embed(step.token_ids, step.token_take, want_stats=True)
        stream = Stream(h, stats=stats)
        for site in self.sites:
            stream = self.blocks[site.layer](stream, step, site)
        return stream.h, stream.delta

    def head(self, h: torch.Tensor, delta: torch.Tensor | None) -> torch.Tensor:
        """Final norm and head on the given rows -> float32 logits [R, vocab]. The rows are consumed."""
        x = self.norm(h) if delta is None else self.norm.add(delta, h)[0]
        return self.lm_head(x)


def build_model(spec: ModelSpec, build: Build) -> Model:
    return Model(spec, build)
