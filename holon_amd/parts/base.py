"""What every part is: an object that declares its tensors and sub-parts, is filled by the weight loader, and is called
with the step's context. Parts know their own sizes and constants and nothing of the model they are in.

State a mixer keeps between steps is declared, not allocated: `PagedState` grows with the sequence and lives in
pages; `SlotState` has a fixed size per request and lives in the request's slot. The cache manager allocates both
(core/holon/api/state.py:27-53 is the reference's form of the two shapes).
"""
from __future__ import annotations

import dataclasses
from collections.abc import Iterator
from typing import Any

import torch

from ..registry import part_class
from ..spec import PartRef

MODEL, FLOAT32, INT32 = "model", "float32", "int32"


@dataclasses.dataclass(frozen=True)
class ParamDecl:
    """A tensor a part owns. `kind`: "model" is kept in the engine's dtype; "float32" is kept in 32-bit whatever the
    engine's dtype; "int32" is an integer table."""

    shape: tuple[int, ...]
    kind: str = MODEL
    init: str = "linear"                          # how random weights draw it: linear | norm


@dataclasses.dataclass(frozen=True)
class PagedState:
    """State that grows by `elems` values per token. Sites whose declarations are equal share a page pool and a block
    table; a window W > 0 says that tokens more than W-1 behind the newest are never read again."""

    name: str
    elems: int
    window: int = 0
    dtype: torch.dtype | None = None              # None: the engine's dtype


@dataclasses.dataclass(frozen=True)
class SlotState:
    """State of fixed shape per request, addressed by the request's slot; zeroed when the slot is given out."""

    name: str
    shape: tuple[int, ...]
    dtype: torch.dtype | None = None


class PartialSums:
    """A product [T, N] that exists as float32 sums over shares of its inner dimension, `parts` [S, T, N]: the product
    is their sum in order, rounded once to the activation dtype. A projection may hand this out instead of a tensor,
    but only to a caller that passed it the residual stream (so one that goes on to add the product into the stream):
    a norm's `add` reads the parts itself; anyone else calls `value()`."""

    def __init__(self, parts: torch.Tensor, kernels: Any, dtype: torch.dtype) -> None:
        self.parts, self.kernels, self.dtype = parts, kernels, dtype

    @property
    def shape(self) -> torch.Size:
        return self.parts.shape[1:]

    def value(self) -> torch.Tensor:
        return self.kernels.sum_parts(self.parts, self.dtype)

    def index_select(self, dim: int, index: torch.Tensor) -> "PartialSums":
        """Rows of the product (dim 0 alone)."""
        if dim != 0:
            raise ValueError("PartialSums.index_select: rows only (dim 0)")
        return PartialSums(self.parts.index_select(1, index), self.kernels, self.dtype)


@dataclasses.dataclass
class Stream:
    """The residual stream between blocks: `h` [T, hidden], updated in place; `delta`, a term not yet added to it (the
    next norm's kernel fuses the add; a tensor or `PartialSums`) or None; `stats`, what the kernel that last wrote `h`
    left about its rows for a norm that follows (partial sums of squares, see the kernel contract) or None when
    nothing is known. Whoever changes `h` sets `stats` anew or to None."""

    h: torch.Tensor
    delta: "torch.Tensor | PartialSums | None" = None
    stats: torch.Tensor | None = None


@dataclasses.dataclass
class Build:
    """What a part may know of the engine while it is built."""

    kernels: Any
    device: torch.device
    dtype: torch.dtype
    page_size: int = 16
    max_model_len: int = 8192
    max_seqs: int = 64
    max_step_tokens: int = 4096
    decode_copy: bool = True                      # keep a second, tiled copy of every projection for decode steps

    def make(self, ref: PartRef, **site: Any) -> "Part":
        return part_class(ref)(self, **ref.get(), **site)


class Part:
    """Base of all parts. Subclasses call `declare` for tensors and `attach` for sub-parts in `__init__`."""

    adds_residual = False     # its forward accepts `residual=h`: it may add its result into h and return None
    graph_safe = False        # True: a captured step may be replayed over it. Its forward then reads nothing on the
                              # host that changes from step to step (no `step.h_*`, no `.item()`, no shapes that depend
                              # on values) and launches the same kernels on the same buffers whatever the rows are.
                              # A model with one part that does not say so runs every step eagerly.

    def __init__(self, build: Build) -> None:
        self.build = build
        self.kernels = build.kernels
        self._decls: dict[str, ParamDecl] = {}
        self._children: dict[str, Part] = {}

    def declare(self, name: str, shape: tuple[int, ...], kind: str = MODEL, init: str = "linear") -> None:
        self._decls[name] = ParamDecl(tuple(int(s) for s in shape), kind, init)
        setattr(self, name, None)

    def attach(self, name: str, part: "Part") -> "Part":
        self._children[name] = part
        setattr(self, name, part)
        return part

    def drop(self, name: str) -> None:
        """Forget a sub-part (its weights were merged into another tensor)."""
        self._children.pop(name)
        setattr(self, name, None)

    def named_params(self, prefix: str = "") -> Iterator[tuple[str, "Part", str, ParamDecl]]:
        for name, decl in self._decls.items():
            yield prefix + name, self, name, decl
        for cname, child in self._children.items():
            yield from child.named_params(f"{prefix}{cname}.")

    def walk(self) -> Iterator["Part"]:
        """Children first."""
        for child in list(self._children.values()):
            yield from child.walk()
        yield self

    def finalize(self) -> None:
        """Called once after every tensor is loaded, children before parents (merge weights, build tables)."""

    def state(self) -> list[PagedState | SlotState]:
        """What this part keeps between steps (mixers)."""
        return []

    def cut(self, start: int, count: int) -> int:
        """How many of the next `count` tokens, the first at position `start`, a prompt portion that does not end the
        prompt may take (0: none, offer more). A mixer whose state is only right on a grid of positions ends portions
        there; the scheduler asks every part of the model and takes the smallest answer. Default: all of them."""
        return count

    def absorb_norm(self, norm: "Part") -> bool:
        """A mixer or feed-forward whose first product can take the norm in front of it into its own kernel folds the
        norm's weight into its weights now and answers True; it is from then on handed the norm deferred
        (`norm.defer(...)`) instead of the norm's result. Default: it cannot."""
        return False

    def extra_tensors(self) -> list[torch.Tensor]:
        """Device tensors this part holds beside its declared parameters (copies in another layout, tables): what
        `nbytes` counts on top of them."""
        return []

    def nbytes(self) -> int:
        total = 0
        for part in self.walk():
            held = [getattr(part, name) for name in part._decls] + list(part.extra_tensors())
            total += sum(t.numel() * t.element_size() for t in held if t is not None)
        return total


class NormPart(Part):
    """What the model and the blocks ask of a norm. A norm implements `forward`; the rest has defaults that run it as
    a kernel of its own. A norm that fused kernels can take over describes itself in `fusion` and may hand out its
    result deferred (`defer`)."""

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError

    def __call__(self, x: torch.Tensor) -> torch.Tensor:
        return self.forward(x)

    def add(self, x: "torch.Tensor | PartialSums", residual: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
        """(norm(residual + x), residual + x); the sum, rounded to the residual's dtype, replaces `residual` in place."""
        residual.add_(x.value() if isinstance(x, PartialSums) else x)
        return self.forward(residual), residual

    def fusion(self) -> dict | None:
        """What a fused kernel needs to do this norm itself ({"norm": kind, "eps": ..., "weight": ...}); None: no
        kernel takes it over, it always runs by itself."""
        return None

    defer = None              # a norm that can be folded into the product that reads it offers
                              # defer(h, stats, delta) -> an object with value() (see norms.Normed)


class EmbedPart(Part):
    """What the model asks of the part that turns token ids into rows of the residual stream. A part implements
    `rows(ids)`; `forward` adds what the step function may ask for beside it."""

    def rows(self, ids: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError

    def forward(self, ids: torch.Tensor, take: tuple[torch.Tensor, torch.Tensor] | None = None,
                want_stats: bool = False):
        """ids [T] int32 -> rows [T, hidden]. `take` = (take_slot [T], last_token [slots]): where take_slot[t] >= 0
        the token is last_token[take_slot[t]], one that the step before drew and left on the device. With
        `want_stats` the answer is (rows, statistics of the rows for a norm that follows, or None): a part whose
        kernel leaves none answers None."""
        if take is not None:
            slot, last = take
            ids = torch.where(slot >= 0, last[slot.clamp(min=0).long()], ids)
        out = self.rows(ids)
        return (out, None) if want_stats else out

    def __call__(self, *args, **kwargs):
        return self.forward(*args, **kwargs)
