"""Toy parts and a toy architecture that tests register, build and step without touching the framework's files. None
of them is a model of anyone's: each exists to use one seam of the framework (a portion grid, several paged states
in one run, stacked expert tensors, steps that must not be replayed from a graph)."""
from __future__ import annotations

import dataclasses

import torch

from holon_amd.parts import Build, Part, SlotState
from holon_amd.parts.base import PagedState
from holon_amd.parts.linear import Linear
from holon_amd.spec import LayerSpec, ModelSpec, PartRef, WeightRule, in_order


class GridRunningMean(Part):
    """y[t] = W (mean of x[0..t]); the running sum is kept per request in its slot (float32). Its prompt path stands
    for a kernel that works on a grid of `grid` positions: a portion of more than one token must start on the grid,
    so portions that do not end the prompt must end there, which `cut` tells the scheduler. Single tokens may come
    anywhere. It plans on the host (it reads `step.h_*`), so it does not declare `graph_safe`."""

    def __init__(self, build: Build, *, hidden: int, layer: int, grid: int) -> None:
        super().__init__(build)
        self.hidden, self.grid = hidden, grid
        self.attach("proj", Linear(build, inp=hidden, out=hidden))
        self.portions: list[tuple[int, int]] = []         # (start, count) of every row it has run, for the test

    def state(self):
        return [SlotState("sum", (self.hidden,), torch.float32)]

    def cut(self, start: int, count: int) -> int:
        return max(0, (start + count) // self.grid * self.grid - start)

    def forward(self, x, step, site):
        state = site.slot_state["sum"]
        mixed = torch.empty_like(x, dtype=torch.float32)
        at = 0
        for slot, start, n in zip(step.h_slots.tolist(), step.h_starts.tolist(), step.h_counts.tolist()):
            if n > 1 and start % self.grid:
                raise AssertionError(f"a portion of {n} tokens starts at {start}, off the grid of {self.grid}")
            self.portions.append((start, n))
            s = torch.zeros_like(state[slot]) if start == 0 else state[slot].clone()
            for i in range(n):
                s = s + x[at + i].float()
                mixed[at + i] = s / (start + i + 1)
            state[slot] = s
            at += n
        return self.proj(mixed.to(x.dtype))

    __call__ = forward


class TwoCaches(Part):
    """A toy mixer that keeps two paged states of different widths: every token's input `x` (the model's dtype, `hidden`
    values a token) and a positive weight `w` = 1 + x[0]^2 (float32, one value a token). y[t] = W (sum_j<=t w_j x_j /
    sum_j<=t w_j), read back through each state's own block table."""

    def __init__(self, build: Build, *, hidden: int, layer: int) -> None:
        super().__init__(build)
        self.hidden = hidden
        self.attach("proj", Linear(build, inp=hidden, out=hidden))

    def state(self):
        return [PagedState("x", self.hidden), PagedState("w", 1, dtype=torch.float32)]

    def forward(self, x, step, site):
        px, pw = site.paged["x"], site.paged["w"]
        vx, vw = step.paged[px.group], step.paged[pw.group]
        page = vx.page_size
        xs, ws = px.pages.view(-1, page, self.hidden), pw.pages.view(-1, page, 1)
        xs[vx.write_page.long(), vx.write_off.long()] = x
        ws[vw.write_page.long(), vw.write_off.long()] = 1 + x[:, :1].float() ** 2
        out = []
        for slot, start, n in zip(step.h_slots.tolist(), step.h_starts.tolist(), step.h_counts.tolist()):
            total = start + n
            held = -(-total // page)
            keys = xs[vx.table[slot, :held].long()].reshape(-1, self.hidden)[:total].float()
            weights = ws[vw.table[slot, :held].long()].reshape(-1, 1)[:total]
            out.append(((weights * keys).cumsum(0) / weights.cumsum(0))[start:])
        return self.proj(torch.cat(out).to(x.dtype))

    __call__ = forward


class StackedTopOne(Part):
    """A toy routed feed-forward whose experts' weights are two stacked parameters, `gate_up` [experts, 2 inter,
    hidden] and `down` [experts, hidden, inter], filled one expert's tensor at a time by a stacking weight rule. The
    router is float32; each token goes to its best expert."""

    def __init__(self, build: Build, *, hidden: int, layer: int, inter: int, experts: int) -> None:
        super().__init__(build)
        self.inter, self.n_experts = inter, experts
        self.attach("router", Linear(build, inp=hidden, out=experts))
        self.declare("gate_up", (experts, 2 * inter, hidden))
        self.declare("down", (experts, hidden, inter))

    def forward(self, x, step=None):
        choice = self.router(x, torch.float32).argmax(-1)
        out = torch.zeros_like(x)
        for e in range(self.n_experts):
            idx = torch.nonzero(choice == e)[:, 0]
            if len(idx):
                gu = self.kernels.linear(x[idx].contiguous(), self.gate_up[e])
                out[idx] = self.kernels.linear(self.kernels.silu_mul(gu), self.down[e])
        return out

    __call__ = forward


STACKED_RULES = (
    WeightRule("model.layers.{i}.mlp.experts.{e}.gate_up.weight", "layers.{i}.ffn.gate_up", stack="e"),
    WeightRule("model.layers.{i}.mlp.experts.{e}.down.weight", "layers.{i}.ffn.down", stack="e"),
    WeightRule("model.layers.{i}.mlp.router.weight", "layers.{i}.ffn.router.weight"),
    WeightRule("model.{rest}", "{rest}"),
)


@dataclasses.dataclass(frozen=True)
class ToyConfig:
    """The configuration of the toy architecture, from its own config.json keys."""

    width: int
    tokens: int
    depth: int
    grid: int
    eps: float
    eos_token_ids: tuple[int, ...] = ()

    @classmethod
    def from_dict(cls, c, generation=None) -> "ToyConfig":
        return cls(width=c["width"], tokens=c["tokens"], depth=c["depth"], grid=c["grid"], eps=c["eps"])

    def to_dict(self) -> dict:
        return {"architectures": ["ToyGridModel"], **{k: getattr(self, k) for k in ("width", "tokens", "depth", "grid", "eps")}}


def toy_recipe(c: ToyConfig) -> ModelSpec:
    norm = PartRef("norm", "rmsnorm", eps=c.eps)
    layer = LayerSpec(block=PartRef("block", "prenorm"), mixer=PartRef("mixer", "test-grid-mean", grid=c.grid),
                      ffn=PartRef("ffn", "swiglu", inter=2 * c.width), norm=norm)
    return ModelSpec(hidden=c.width, vocab=c.tokens, layers=(layer,) * c.depth, order=in_order(c.depth),
                     embed=PartRef("embed", "table"), norm=norm, head=PartRef("head", "linear", tied=True),
                     rules=(WeightRule("toy.{rest}", "{rest}"),))


# -- a toy mixer that brings a kernel of its own ---------------------------------------------------------------------
DECAY_SCAN_SOURCE = __import__("pathlib").Path(__file__).resolve().parent / "kernels" / "decay_scan.hip"


def decay_scan_plain(x, state, slots, starts, query_start, n_rows, decay):
    """y[t] = s_t, s_t = decay * s_(t-1) + x[t] along each row's tokens; `state[slot]` (float32) holds a row's s between
    steps and is updated in place; a row that starts at position 0 starts from zero."""
    y = torch.empty_like(x)
    qs, slot_of, start_of = query_start.tolist(), slots.tolist(), starts.tolist()
    for b in range(n_rows):
        s = torch.zeros_like(state[slot_of[b]]) if start_of[b] == 0 else state[slot_of[b]].clone()
        for t in range(qs[b], qs[b + 1]):
            s = decay * s + x[t].float()
            y[t] = s.to(x.dtype)
        state[slot_of[b]] = s
    return y


def _decay_scan_hip(launch, x, state, slots, starts, query_start, n_rows, decay):
    if not (x.is_cuda and x.is_contiguous() and state.dtype == torch.float32 and state.shape[1] == x.shape[1]):
        raise ValueError("decay_scan: contiguous rows on the GPU and float32 state of their width")
    y = torch.empty_like(x)
    launch(x.data_ptr(), y.data_ptr(), state.data_ptr(), slots.data_ptr(), starts.data_ptr(), query_start.data_ptr(),
           n_rows, x.shape[1], float(decay), {torch.float32: 0, torch.bfloat16: 1}[x.dtype])
    return y


def decay_scan_op():
    """The operation as the toy mixer registers it: plain form, HIP symbol, argument types, and the source it is
    built from (a file under tests/, compiled into a library of its own)."""
    import ctypes

    from holon_amd.kernels.registry import KernelOp
    p, i, f = ctypes.c_void_p, ctypes.c_int, ctypes.c_float
    return KernelOp(name="decay_scan", plain=decay_scan_plain, symbol="toy_decay_scan",
                    argtypes=[p, p, p, p, p, p, i, i, f, i], call=_decay_scan_hip, source=DECAY_SCAN_SOURCE)


class DecayScan(Part):
    """A toy mixer whose arithmetic is a kernel it registers itself (`decay_scan`): a decaying running sum of the
    inputs, kept per request in its slot, then a projection. It reads nothing on the host, so steps over it may be
    replayed from graphs."""

    graph_safe = True

    def __init__(self, build: Build, *, hidden: int, layer: int, decay: float) -> None:
        super().__init__(build)
        self.hidden, self.decay = hidden, float(decay)
        self.attach("proj", Linear(build, inp=hidden, out=hidden))

    def state(self):
        return [SlotState("s", (self.hidden,), torch.float32)]

    def forward(self, x, step, site):
        y = self.kernels.decay_scan(x, site.slot_state["s"], step.slots, step.starts, step.query_start, step.n_rows,
                                    self.decay)
        return self.proj(y)

    __call__ = forward


@dataclasses.dataclass(frozen=True)
class ToyScanConfig:
    width: int
    tokens: int
    depth: int
    decay: float
    eps: float
    eos_token_ids: tuple[int, ...] = ()

    @classmethod
    def from_dict(cls, c, generation=None) -> "ToyScanConfig":
        return cls(width=c["width"], tokens=c["tokens"], depth=c["depth"], decay=c["decay"], eps=c["eps"])

    def to_dict(self) -> dict:
        return {"architectures": ["ToyScanModel"], **{k: getattr(self, k) for k in ("width", "tokens", "depth", "decay", "eps")}}


def toy_scan_recipe(c: ToyScanConfig) -> ModelSpec:
    norm = PartRef("norm", "rmsnorm", eps=c.eps)
    layer = LayerSpec(block=PartRef("block", "prenorm"), mixer=PartRef("mixer", "test-decay-scan", decay=c.decay),
                      ffn=PartRef("ffn", "swiglu", inter=2 * c.width), norm=norm)
    return ModelSpec(hidden=c.width, vocab=c.tokens, layers=(layer,) * c.depth, order=in_order(c.depth),
                     embed=PartRef("embed", "table"), norm=norm, head=PartRef("head", "linear", tied=True),
                     rules=(WeightRule("toy.{rest}", "{rest}"),))
