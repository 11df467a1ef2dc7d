"""The step function: a batch of (request, its next tokens) in, logits at the wanted places out.

It runs only the tokens it is given, as one flat batch, against the cache that earlier steps left: portions of
prompts beside single decoded tokens, cut anywhere. core/holon/core/executor.py:357-430 (`Executor.launch`), :497-564
(host half of the inputs), :460-470 (logits only where wanted), :316-354 (graphs for decode steps).

Decode-only steps (one token a row, every row sampled) may be replayed from a HIP graph: rows are padded to a
batch-size bucket with rows on the padding slot (whose block-table row is all null pages, so they read and write only
the null page), inputs are copied into buffers of fixed address, and the captured launch sequence is replayed. The
first step of a bucket runs eagerly on those buffers, the second captures, later ones replay.
"""
from __future__ import annotations

import dataclasses
import sys

import numpy as np
import torch

from ..cache.manager import CacheManager
from ..kernels.api import AttnRows
from ..model import Model
from .batch import PagedView, Step, StepRow

BUCKETS = (1, 2, 4, 8, 16, 24, 32, 48, 64, 96, 128, 192, 256)    # core/holon/core/executor.py:28
LEN_BUCKET_MIN = 1024


@dataclasses.dataclass
class _Graph:
    arena: torch.Tensor                           # int32 inputs at a fixed address
    step: Step
    logits: torch.Tensor | None = None
    graph: torch.cuda.CUDAGraph | None = None
    runs: int = 0


class StepRunner:
    def __init__(self, model: Model, cache: CacheManager, kernels, device: torch.device, *, max_step_tokens: int,
                 max_seqs: int, graphs: bool = False) -> None:
        self.model, self.cache, self.kernels, self.device = model, cache, kernels, device
        self.max_step_tokens, self.max_seqs = max_step_tokens, max_seqs
        self.vocab = model.spec.vocab
        self.steps = 0
        self.pinned = device.type == "cuda"
        self._stages: list[tuple[torch.Tensor, torch.cuda.Event] | None] = [None, None]
        self._turn = 0
        # the token last drawn for each slot, for a row whose token has not reached the host when it is scheduled
        self.last_token = torch.zeros(max_seqs + 1, dtype=torch.int32, device=device)
        self.last_slots: torch.Tensor | None = None       # the last step's rows' slots on the device
        self.last_lens: torch.Tensor | None = None        # and how many tokens each then holds
        # a captured step is replayed without any part's Python code: only over parts that say they allow it
        self.not_graph_safe = sorted({type(p).__name__ for p in model.walk() if not p.graph_safe})
        self.use_graphs = graphs and device.type == "cuda" and not self.not_graph_safe
        if graphs and device.type == "cuda" and self.not_graph_safe:
            print(f"holon_amd: steps run eagerly, not from graphs: {', '.join(self.not_graph_safe)} "
                  "do not declare graph_safe", file=sys.stderr)
        self.graphs: dict[tuple[int, int], _Graph] = {}
        self.graph_replays = 0

    # -- inputs ---------------------------------------------------------------------------------------------------
    def _arrays(self, slots: np.ndarray, starts: np.ndarray, counts: np.ndarray, tokens: np.ndarray,
                take: np.ndarray, wanted: np.ndarray | None = None) -> tuple[list[np.ndarray], dict]:
        """The int32 arrays of a step, in a fixed order, and the host-side facts about them. `wanted` (the flat places
        whose logits are asked for) rides behind the cache groups' write targets when given."""
        cache = self.cache
        total, n = int(counts.sum()), len(slots)
        if total == n:                             # one token a row: the step's shape is the batch's
            rows = np.arange(n + 1)
            qstart, token_row, positions, decode, chunk = rows, rows[:n], starts, rows[:n], rows[:0]
        else:
            qstart = np.concatenate(([0], np.cumsum(counts)))
            token_row = np.repeat(np.arange(n), counts)
            positions = np.repeat(starts, counts) + (np.arange(total) - np.repeat(qstart[:-1], counts))
            decode = np.flatnonzero(counts == 1)
            chunk = np.flatnonzero(counts > 1)
        lens = starts + counts
        arrays = [tokens, positions, token_row, slots, starts, lens, qstart, decode, chunk, take]
        for g in cache.groups:
            page, off = cache.write_targets(g.gid, slots[token_row], positions)
            arrays += [page, off]
        if wanted is not None:
            arrays.append(wanted)
        fixed = len(arrays)
        dirty = cache.take_dirty()                  # block-table rows that changed: they ride the same copy
        for _, rows, contents in dirty:
            arrays += [rows, contents]
        facts = dict(fixed=fixed, dirty=[(g, len(rows)) for g, rows, _ in dirty],
                     total=total, n_rows=len(slots), n_decode=len(decode), n_chunk=len(chunk), in_order=total == n,
                     max_decode_len=int(lens[decode].max()) if len(decode) else 0,
                     max_chunk_query=int(counts[chunk].max()) if len(chunk) else 0,
                     max_chunk_len=int(lens[chunk].max()) if len(chunk) else 0)
        return arrays, facts

    def _to_device(self, arrays: list[np.ndarray], arena: torch.Tensor | None = None, first: int = 0
                   ) -> list[torch.Tensor]:
        """Several int32 arrays to the device in one copy (into `arena`, a buffer of fixed address, when given).
        Returns views of arrays `first` onwards. The host side is one of two pinned buffers used in turn; a buffer
        is written again only after its last copy ran."""
        sizes = [a.size for a in arrays]
        total = sum(sizes)
        if self.pinned:
            stage = self._stages[self._turn]
            self._turn ^= 1
            if stage is None or stage[0].numel() < total:
                stage = (torch.empty(max(total, 4096) * 2, dtype=torch.int32).pin_memory(), torch.cuda.Event())
                self._stages[self._turn ^ 1] = stage
            else:
                stage[1].synchronize()
            host = stage[0][:total]
        else:
            host = torch.empty(total, dtype=torch.int32)
        np.concatenate([a.ravel() for a in arrays], out=host.numpy(), casting="unsafe")
        if arena is None:
            dev = host.to(self.device, non_blocking=True)
        else:
            dev = arena[:total]
            dev.copy_(host, non_blocking=True)
        if self.pinned:
            stage[1].record()
        out, at = [], 0
        for i, n in enumerate(sizes):
            if i >= first:
                out.append(dev[at: at + n])
            at += n
        return out

    def _table_rows(self, dev: list[torch.Tensor], facts: dict) -> None:
        """Put the changed block-table rows, now on the device, into the tables. `dev`: views from `facts["fixed"]` on."""
        for i, (g, n) in enumerate(facts["dirty"]):
            self.kernels.scatter_rows(g.table_dev, dev[2 * i], dev[2 * i + 1])

    def _step(self, dev: list[torch.Tensor], facts: dict, slots, starts, counts) -> Step:
        cache = self.cache
        paged = {g.gid: PagedView(cache.page_size, g.table_dev, dev[10 + 2 * i], dev[11 + 2 * i])
                 for i, g in enumerate(cache.groups)}
        attn = AttnRows(slots=dev[3], lens=dev[5], query_start=dev[6], decode_rows=dev[7], chunk_rows=dev[8],
                        n_decode=facts["n_decode"], n_chunk=facts["n_chunk"], max_decode_len=facts["max_decode_len"],
                        max_chunk_query=facts["max_chunk_query"], max_chunk_len=facts["max_chunk_len"],
                        in_order=facts["in_order"])
        return Step(kernels=self.kernels, n_tokens=facts["total"], n_rows=facts["n_rows"], token_ids=dev[0],
                    positions=dev[1], token_row=dev[2], slots=dev[3], starts=dev[4], rows=attn, paged=paged,
                    h_slots=slots, h_starts=starts, h_counts=counts, token_take=(dev[9], self.last_token))

    def _check(self, rows: list[StepRow]
               ) -> tuple[np.ndarray, np.ndarray, np.ndarray, np.ndarray, np.ndarray, np.ndarray]:
        if not rows:
            raise ValueError("a step needs at least one row")
        cache = self.cache
        computed, paged = cache.computed, bool(cache.groups)
        slots, starts, counts, wanted, flat, take = [], [], [], [], [], []
        at = 0
        for b, r in enumerate(rows):
            n = len(r.tokens)
            if n < 1:
                raise ValueError("every row of a step brings at least one token")
            if r.start != computed[r.slot]:
                raise ValueError(f"slot {r.slot}: the row starts at {r.start}, the cache holds {computed[r.slot]}")
            if paged and r.start + n > cache.capacity(r.slot):
                raise RuntimeError(f"slot {r.slot}: no pages reserved for tokens up to {r.start + n}")
            for w in r.want:
                if not 0 <= w < n:
                    raise ValueError(f"row {b}: wanted place {w} is not among its {n} tokens")
                wanted.append(at + w)
            if r.on_device:
                if n != 1:
                    raise ValueError(f"row {b}: only a row of one token can take it from the device")
                take.append(r.slot)
            else:
                take.extend([-1] * n) if n > 1 else take.append(-1)
            slots.append(r.slot)
            starts.append(r.start)
            counts.append(n)
            flat.extend(r.tokens)
            at += n
        if at > self.max_step_tokens:
            raise ValueError(f"the step has {at} tokens; max_step_tokens is {self.max_step_tokens}")
        if len(set(slots)) != len(slots):
            raise ValueError("a request appears twice in one step")
        tokens = np.array(flat, dtype=np.int64)
        if tokens.min() < 0 or tokens.max() >= self.vocab:
            raise ValueError(f"token ids must lie in [0, {self.vocab})")
        return (np.array(slots, dtype=np.int64), np.array(starts, dtype=np.int64), np.array(counts, dtype=np.int64),
                tokens, np.array(wanted, dtype=np.int64), np.array(take, dtype=np.int64))

    def prepare(self, rows: list[StepRow]) -> tuple[Step, np.ndarray]:
        """Device inputs of a step, and the flat indices of the tokens whose logits are wanted (in row order, then in
        the order of each row's `want`)."""
        step, wanted, _ = self._prepare(self._check(rows))
        return step, wanted

    def _prepare(self, checked: tuple) -> tuple[Step, np.ndarray, torch.Tensor | None]:
        """The same from rows already checked; the last value is the wanted places on the device when only some of
        the step's tokens are wanted (they ride in the inputs' copy)."""
        slots, starts, counts, tokens, wanted, take = checked
        some = 0 < len(wanted) and not _all_in_order(wanted, len(tokens))
        arrays, facts = self._arrays(slots, starts, counts, tokens, take, wanted if some else None)
        dev = self._to_device(arrays)
        self._table_rows(dev[facts["fixed"]:], facts)
        return self._step(dev, facts, slots, starts, counts), wanted, dev[facts["fixed"] - 1] if some else None

    # -- the step -------------------------------------------------------------------------------------------------
    def _forward(self, step: Step, wanted: np.ndarray | None, wanted_dev: torch.Tensor | None = None
                 ) -> torch.Tensor | None:
        """The model on a step; `wanted` None: logits of every token. `wanted_dev`: the same places on the device."""
        h, delta = self.model.trunk(step)
        if wanted is not None and not len(wanted):
            return None
        if wanted is None or _all_in_order(wanted, step.n_tokens):
            return self.model.head(h, delta)
        idx = wanted_dev if wanted_dev is not None else torch.from_numpy(wanted).to(self.device)
        return self.model.head(h.index_select(0, idx), delta.index_select(0, idx) if delta is not None else None)

    @torch.no_grad()
    def run(self, rows: list[StepRow]) -> torch.Tensor | None:
        """Run the rows' tokens through the model; returns float32 logits [wanted, vocab] (None when nothing is
        wanted: then the head does not run). Afterwards the cache holds the rows' tokens."""
        checked = self._check(rows)
        if self.use_graphs and len(rows) <= BUCKETS[-1] and all(len(r.tokens) == 1 and r.want == [0] for r in rows):
            logits = self._run_graphed(checked)
        else:
            step, wanted, wanted_dev = self._prepare(checked)
            self.last_slots, self.last_lens = step.slots, step.lens
            logits = self._forward(step, wanted, wanted_dev)
        for r in rows:
            self.cache.advance(r.slot, r.start + len(r.tokens))
        self.steps += 1
        return logits

    # -- graphs ---------------------------------------------------------------------------------------------------
    def _padded(self, checked: tuple, pad: int) -> tuple:
        """The step with `pad` more rows on the padding slot behind its own: one token at position 0 of the null page."""
        slots, starts, counts, tokens, wanted, take = checked
        if not pad:
            return checked
        return (np.concatenate((slots, np.full(pad, self.cache.padding_slot, dtype=np.int64))),
                np.concatenate((starts, np.zeros(pad, dtype=np.int64))),
                np.concatenate((counts, np.ones(pad, dtype=np.int64))),
                np.concatenate((tokens, np.zeros(pad, dtype=np.int64))), wanted,
                np.concatenate((take, np.full(pad, -1, dtype=np.int64))))

    def _arena(self, arrays: list[np.ndarray], facts: dict) -> torch.Tensor:
        """Room at a fixed address for a step's inputs and, behind them, for every block-table row."""
        size = sum(a.size for a in arrays[: facts["fixed"]])
        size += sum(gr.table.size + gr.table.shape[0] for gr in self.cache.groups)
        return torch.zeros(size, dtype=torch.int32, device=self.device)

    def _run_graphed(self, checked: tuple) -> torch.Tensor:
        n = len(checked[0])
        bucket = next(b for b in BUCKETS if b >= n)
        slots, starts, counts, tokens, _, take = self._padded(checked, bucket - n)
        len_bucket = _len_bucket(int((starts + counts).max()))
        arrays, facts = self._arrays(slots, starts, counts, tokens, take)
        facts["max_decode_len"] = len_bucket       # launch shapes are the bucket's, whatever the rows' lengths
        key = (bucket, len_bucket)
        g = self.graphs.get(key)
        if g is None:
            arena = self._arena(arrays, facts)
            dev = self._to_device(arrays, arena)
            g = _Graph(arena=arena, step=self._step(dev, facts, slots, starts, counts))
            self.graphs[key] = g
        else:
            dev = self._to_device(arrays, g.arena)
            g.step.h_slots, g.step.h_starts, g.step.h_counts = slots, starts, counts
        self._table_rows(dev[facts["fixed"]:], facts)
        g.runs += 1
        self.last_slots, self.last_lens = g.step.slots[:n], g.step.lens[:n]
        if g.graph is None and g.runs == 1:        # the first step of a bucket: eagerly, on the fixed buffers
            return self._forward(g.step, None)[:n]
        if g.graph is None:
            torch.cuda.synchronize(self.device)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                g.logits = self._forward(g.step, None)
            g.graph = graph
        g.graph.replay()
        self.graph_replays += 1
        return g.logits[:n]


def _len_bucket(longest: int) -> int:
    return max(LEN_BUCKET_MIN, 1 << (max(longest, 1) - 1).bit_length())


def _all_in_order(wanted: np.ndarray, n_tokens: int) -> bool:
    return len(wanted) == n_tokens and bool((wanted == np.arange(n_tokens)).all())
