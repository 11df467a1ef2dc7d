"""Token mixers. Grouped-query attention over the paged cache:
std/holon_std/mixers/gqa/units.py:108-294 (`GQA`), formulas std/holon_std/mixers/gqa/reference.py:26-60, 91-101."""
from __future__ import annotations

import torch

from ..registry import register_part
from ..spec import PartRef
from .base import Build, PagedState, Part, Stream
from .linear import Linear
from .norms import Normed


@register_part("mixer", "gqa")
class GQA(Part):
    """q/k/v projections (merged into one product after loading), optional per-head norm on q and k, optional
    position encoding on q and k, keys and values written to the cache, causal attention over the cache (optionally
    within a window), output projection. `heads * head_dim` need not equal `hidden`.

    A run that reads another run's cache (`site.writes` false) projects and encodes queries only."""

    graph_safe = True

    def __init__(self, build: Build, *, heads: int, kv_heads: int, head_dim: int, hidden: int, layer: int,
                 qk_norm: PartRef | None = None, position: PartRef | None = None, window: int = 0,
                 scale: float | None = None) -> None:
        super().__init__(build)
        if heads % kv_heads:
            raise ValueError(f"gqa: {heads} heads are not a multiple of {kv_heads} kv heads")
        if build.kernels is not None:             # a size no attention kernel serves is refused now, not at the first step
            build.kernels.check_attention(head_dim, build.page_size, build.dtype)
        self.heads, self.kv_heads, self.head_dim, self.hidden, self.layer = heads, kv_heads, head_dim, hidden, layer
        self.window = int(window)
        self.scale = float(scale) if scale is not None else head_dim ** -0.5
        self.attach("q_proj", Linear(build, inp=hidden, out=heads * head_dim))
        self.attach("k_proj", Linear(build, inp=hidden, out=kv_heads * head_dim))
        self.attach("v_proj", Linear(build, inp=hidden, out=kv_heads * head_dim))
        self.attach("o_proj", Linear(build, inp=heads * head_dim, out=hidden))
        self.q_norm = self.k_norm = None
        if qk_norm is not None:
            self.attach("q_norm", build.make(qk_norm, dim=head_dim))
            self.attach("k_norm", build.make(qk_norm, dim=head_dim))
        self.position = None
        if position is not None:
            self.attach("position", build.make(position, head_dim=head_dim))
        self.qkv: Linear | None = None
        self._fused: dict | None = None

    def state(self) -> list[PagedState]:
        return [PagedState("kv", elems=2 * self.kv_heads * self.head_dim, window=self.window)]

    def finalize(self) -> None:
        self.qkv = Linear.merge(self.build, self.q_proj, self.k_proj, self.v_proj)
        for name in ("q_proj", "k_proj", "v_proj"):
            self.drop(name)
        self._children["qkv"] = self.qkv
        # One fused kernel does norm, rotation and the cache write when the injected parts can describe themselves.
        norm = self.q_norm.fusion() if self.q_norm is not None else {"norm": "none", "eps": 0.0, "weight": None}
        pos = self.position.fusion() if self.position is not None else {"position": "none", "table": None}
        if norm is not None and pos is not None and norm["norm"] in ("rmsnorm", "none") \
                and pos["position"] in ("rope", "none"):
            self._fused = {"eps": norm["eps"], "table": pos["table"]}

    adds_residual = True

    def absorb_norm(self, norm: Part) -> bool:
        """Fold the norm in front of this mixer into its merged q/k/v product; it then takes `Normed` input."""
        return self.qkv is not None and self.qkv.absorb(norm)

    def forward(self, x: "torch.Tensor | Normed", step, site, residual: Stream | None = None) -> torch.Tensor | None:
        k = self.kernels
        t, hq, hkv, d = x.shape[0], self.heads, self.kv_heads, self.head_dim
        view = step.paged[site.group]
        pages = site.pages.view(-1, 2, hkv, view.page_size * d)
        qkv = self.qkv(x)
        if self._fused is not None:
            out = k.qkv_attention(
                qkv, hq, hkv, d, self.q_norm.weight if self.q_norm is not None else None,
                self.k_norm.weight if self.k_norm is not None else None, self._fused["eps"], self._fused["table"],
                step.positions, pages, view.table, view.write_page, view.write_off, step.rows, view.page_size,
                self.scale, self.window, writes=site.writes)
            return self.o_proj(out.view(t, hq * d), residual=residual)
        else:
            q = qkv[:, : hq * d].contiguous().view(t, hq, d)
            kk = qkv[:, hq * d: (hq + hkv) * d].contiguous().view(t, hkv, d) if site.writes else None
            if self.q_norm is not None:
                q = self.q_norm(q)
                kk = self.k_norm(kk) if kk is not None else None
            if self.position is not None:
                self.position.apply(q, kk, step.positions)
            if site.writes:
                v = qkv[:, (hq + hkv) * d:].contiguous().view(t, hkv, d)
                k.kv_write(kk, v, pages, view.write_page, view.write_off, view.page_size)
        out = k.paged_attention(q, pages, view.table, step.rows, view.page_size, self.scale, self.window)
        return self.o_proj(out.view(t, hq * d), residual=residual)

    __call__ = forward
