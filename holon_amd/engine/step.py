"""The step function: a batch of (request, its next tokens) in, logits at the wanted places out.

It runs only the tokens it is given, as one flat batch, against the cache that earlier steps left: portions of
prompts beside single decoded tokens, cut anywhere. core/holon/core/executor.py:357-430 (`Executor.launch`), :497-564
(host half of the inputs), :460-470 (logits only where wanted).
"""
from __future__ import annotations

import numpy as np
import torch

from ..cache.manager import CacheManager
from ..kernels.api import AttnRows
from ..model import Model
from .batch import PagedView, Step, StepRow


class StepRunner:
    def __init__(self, model: Model, cache: CacheManager, kernels, device: torch.device, *, max_step_tokens: int,
                 max_seqs: int) -> None:
        self.model, self.cache, self.kernels, self.device = model, cache, kernels, device
        self.max_step_tokens, self.max_seqs = max_step_tokens, max_seqs
        self.vocab = model.spec.vocab
        self.steps = 0
        self.pinned = device.type == "cuda"

    # -- inputs ---------------------------------------------------------------------------------------------------
    def _upload(self, arrays: list[np.ndarray]) -> list[torch.Tensor]:
        """Several int32 arrays to the device in one copy."""
        sizes = [a.size for a in arrays]
        flat = np.concatenate([a.astype(np.int32, copy=False).ravel() for a in arrays]) if arrays else np.zeros(0, np.int32)
        host = torch.from_numpy(flat)
        if self.pinned:
            host = host.pin_memory()
        dev = host.to(self.device, non_blocking=True)
        out, at = [], 0
        for n in sizes:
            out.append(dev[at: at + n])
            at += n
        return out

    def prepare(self, rows: list[StepRow]) -> tuple[Step, np.ndarray]:
        """Device inputs of a step, and the flat indices of the tokens whose logits are wanted (in row order, then in
        the order of each row's `want`)."""
        if not rows:
            raise ValueError("a step needs at least one row")
        cache = self.cache
        counts = np.array([len(r.tokens) for r in rows], dtype=np.int64)
        if (counts < 1).any():
            raise ValueError("every row of a step brings at least one token")
        total = int(counts.sum())
        if total > self.max_step_tokens:
            raise ValueError(f"the step has {total} tokens; max_step_tokens is {self.max_step_tokens}")
        if len({r.slot for r in rows}) != len(rows):
            raise ValueError("a request appears twice in one step")
        slots = np.array([r.slot for r in rows], dtype=np.int64)
        starts = np.array([r.start for r in rows], dtype=np.int64)
        for r, n in zip(rows, counts):
            if r.start != cache.computed[r.slot]:
                raise ValueError(f"slot {r.slot}: the row starts at {r.start}, the cache holds {cache.computed[r.slot]}")
            if r.start + n > cache.capacity(r.slot):
                raise RuntimeError(f"slot {r.slot}: no pages reserved for tokens up to {r.start + n}")
        qstart = np.concatenate(([0], np.cumsum(counts)))
        token_row = np.repeat(np.arange(len(rows)), counts)
        positions = np.repeat(starts, counts) + (np.arange(total) - np.repeat(qstart[:-1], counts))
        tokens = np.concatenate([np.asarray(r.tokens, dtype=np.int64) for r in rows])
        if tokens.min() < 0 or tokens.max() >= self.vocab:
            raise ValueError(f"token ids must lie in [0, {self.vocab})")
        lens = starts + counts
        decode = np.flatnonzero(counts == 1)
        chunk = np.flatnonzero(counts > 1)
        wanted = []
        for b, r in enumerate(rows):
            for w in r.want:
                if not 0 <= w < counts[b]:
                    raise ValueError(f"row {b}: wanted place {w} is not among its {counts[b]} tokens")
                wanted.append(qstart[b] + w)
        cache.upload()
        arrays = [tokens, positions, token_row, slots, starts, lens, qstart, decode, chunk]
        for g in cache.groups:
            page, off = cache.write_targets(g.gid, slots[token_row], positions)
            arrays += [page, off]
        dev = self._upload(arrays)
        paged = {g.gid: PagedView(cache.page_size, g.table_dev, dev[9 + 2 * i], dev[10 + 2 * i])
                 for i, g in enumerate(cache.groups)}
        attn = AttnRows(slots=dev[3], lens=dev[5], query_start=dev[6], decode_rows=dev[7], chunk_rows=dev[8],
                        n_decode=len(decode), n_chunk=len(chunk),
                        max_decode_len=int(lens[decode].max()) if len(decode) else 0,
                        max_chunk_query=int(counts[chunk].max()) if len(chunk) else 0,
                        max_chunk_len=int(lens[chunk].max()) if len(chunk) else 0)
        step = Step(kernels=self.kernels, n_tokens=total, n_rows=len(rows), token_ids=dev[0], positions=dev[1],
                    token_row=dev[2], slots=dev[3], starts=dev[4], rows=attn, paged=paged,
                    h_slots=slots, h_starts=starts, h_counts=counts)
        return step, np.asarray(wanted, dtype=np.int64)

    # -- the step -------------------------------------------------------------------------------------------------
    @torch.no_grad()
    def run(self, rows: list[StepRow]) -> torch.Tensor | None:
        """Run the rows' tokens through the model; returns float32 logits [wanted, vocab] (None when nothing is
        wanted: then the head does not run). Afterwards the cache holds the rows' tokens."""
        step, wanted = self.prepare(rows)
        h, delta = self.model.trunk(step)
        logits = None
        if len(wanted):
            if len(wanted) == step.n_tokens and (wanted == np.arange(step.n_tokens)).all():
                rows_h, rows_d = h, delta
            else:
                idx = torch.from_numpy(wanted).to(self.device)
                rows_h = h.index_select(0, idx)
                rows_d = delta.index_select(0, idx) if delta is not None else None
            logits = self.model.head(rows_h, rows_d)
        for r, n in zip(rows, step.h_counts):
            self.cache.advance(r.slot, r.start + int(n))
        self.steps += 1
        return logits
