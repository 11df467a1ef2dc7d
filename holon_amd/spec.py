"""What a model is made of, as data: parts by kind name and parameters, layers, and the order they run in.

An architecture's recipe turns its typed configuration into a `ModelSpec`; the builder (`holon_amd.model`) turns the
spec into parts with weights. Nothing here knows an architecture. The shape follows the reference's contracts
(core/holon/api/model.py:27-81 `ModelSpec`/`LayerDecl`, core/holon/api/terms.py:23-63 `Ref`), with one addition: the
run order is a list of its own, so a layer may run twice or read the cache another run wrote.
"""
from __future__ import annotations

import dataclasses
import hashlib
import json
import re
from typing import Any


@dataclasses.dataclass(frozen=True)
class PartRef:
    """A part by registry kind and name, with its sizes and constants: `PartRef("mixer", "gqa", heads=32, ...)`.
    Parameters may hold other PartRefs (a mixer's norm and position encoding)."""

    family: str                                  # which registry: mixer | ffn | norm | position | block | embed | head
    kind: str
    params: tuple[tuple[str, Any], ...] = ()

    def __init__(self, family: str, kind: str, **params: Any) -> None:
        object.__setattr__(self, "family", family)
        object.__setattr__(self, "kind", kind)
        object.__setattr__(self, "params", tuple(sorted(params.items())))

    def get(self) -> dict[str, Any]:
        return dict(self.params)

    def canonical(self) -> Any:
        return {"family": self.family, "kind": self.kind,
                "params": {k: v.canonical() if isinstance(v, PartRef) else v for k, v in self.params}}


@dataclasses.dataclass(frozen=True)
class LayerSpec:
    """One layer's parts: how they are wired (block), what mixes tokens, what feeds forward, which norm."""

    block: PartRef
    mixer: PartRef
    ffn: PartRef
    norm: PartRef


@dataclasses.dataclass(frozen=True)
class Run:
    """One entry of the run order: layer `layer` runs here. `reads` names an earlier entry of the order whose cache
    this run reads instead of writing one of its own (None: it has its own)."""

    layer: int
    reads: int | None = None


@dataclasses.dataclass(frozen=True)
class WeightRule:
    """A checkpoint tensor name pattern and the parameter path it fills: `{i}` matches digits, any other `{name}` one
    or more characters, the whole name must match (core/holon/core/build.py:317-337).

    `stack` names a capture of digits that is no part of the target: the tensor then fills slice number `stack` of
    the target parameter's first dimension, so that one tensor per expert fills a parameter `[experts, ...]`
    (core/holon/core/build.py:351-369): `WeightRule("layers.{i}.mlp.experts.{e}.up.weight", "layers.{i}.ffn.up", "e")`."""

    pattern: str
    target: str
    stack: str | None = None

    def __post_init__(self) -> None:
        if self.stack is not None and ("{" + self.stack + "}" not in self.pattern or "{" + self.stack + "}" in self.target):
            raise ValueError(f"rule {self.pattern!r}: the stacking capture {{{self.stack}}} must be in the pattern and "
                             "not in the target")

    def compile(self) -> re.Pattern[str]:
        parts = re.split(r"(\{\w+\})", self.pattern)
        out = []
        for p in parts:
            if p.startswith("{") and p.endswith("}"):
                out.append(f"(?P<{p[1:-1]}>" + (r"\d+" if p in ("{i}", "{" + str(self.stack) + "}") else ".+") + ")")
            else:
                out.append(re.escape(p))
        return re.compile("".join(out) + r"\Z")


@dataclasses.dataclass(frozen=True)
class ModelSpec:
    hidden: int
    vocab: int
    layers: tuple[LayerSpec, ...]
    order: tuple[Run, ...]
    embed: PartRef
    norm: PartRef
    head: PartRef
    rules: tuple[WeightRule, ...]
    skip: tuple[str, ...] = ()                   # checkpoint name prefixes that are read past (a tied model's head)
    trained_context: int | None = None
    eos_token_ids: tuple[int, ...] = ()

    def __post_init__(self) -> None:
        for at, run in enumerate(self.order):
            if not 0 <= run.layer < len(self.layers):
                raise ValueError(f"run {at} names layer {run.layer}; the model has {len(self.layers)}")
            if run.reads is not None and not (0 <= run.reads < at and self.order[run.reads].reads is None):
                raise ValueError(f"run {at} reads run {run.reads}: it must be an earlier run with a cache of its own")

    def identity(self) -> str:
        """A hash of everything that decides the computation (core/holon/api/terms.py:98-100)."""
        doc = {"hidden": self.hidden, "vocab": self.vocab,
               "layers": [[getattr(l, f).canonical() for f in ("block", "mixer", "ffn", "norm")] for l in self.layers],
               "order": [[r.layer, r.reads] for r in self.order],
               "embed": self.embed.canonical(), "norm": self.norm.canonical(), "head": self.head.canonical()}
        return hashlib.sha256(json.dumps(doc, sort_keys=True).encode()).hexdigest()[:16]


def in_order(n_layers: int) -> tuple[Run, ...]:
    """Every layer once, first to last."""
    return tuple(Run(i) for i in range(n_layers))
