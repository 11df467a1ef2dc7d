"""The engine: requests in, tokens out. core/holon/core/engine.py:143-282 (start), :332-376 (`add`), :474-524
(`generate`, `step`), :603-709 (commit and finishing).

    engine = Engine(EngineConfig(model=folder))
    rid = engine.add(token_ids, SamplingParams(temperature=0, max_tokens=16))
    while engine.has_work():
        for delta in engine.step(): ...
    engine.generate([ids, ids], params) -> [[token, ...], [token, ...]]

Token ids in, token ids out. One step: the scheduler picks rows, the step function runs them as one batch, the
sampler draws a token for every row that ended its prompt or decoded, the commit appends tokens and finishes requests.
"""
from __future__ import annotations

import dataclasses
import hashlib
import itertools
import secrets
import sys

import numpy as np
import torch

from ..cache.pool import OutOfPages
from ..config.engine import EngineConfig, SamplingParams
from ..sampling.sampler import Sampler, sequence_seed
from .batch import StepRow
from .loading import assemble, attach_cache
from .request import Logprobs, Seq, Status, TokenDelta
from .scheduler import Scheduler

CACHED_PREFIX_TOKENS = 1 << 22      # with a prefix cache the pools grow to this many tokens, if memory allows
PROMPT_LOGPROB_PORTION = 256        # core/holon/core/executor.py:645-666 takes the prompt's logits in pieces as small


@dataclasses.dataclass
class _Launched:
    """A step on the device: its rows, and where its results will be on the host once `done` has passed."""

    rows: list
    sync: bool = False                          # it read the host while it was launched: commit it at once
    tokens: torch.Tensor | None = None          # [sampled rows] int32
    logprobs: list[torch.Tensor] | None = None
    done: "torch.cuda.Event | None" = None


class Engine:
    def __init__(self, cfg: EngineConfig, kernels=None, *, random_config: dict | None = None, seed: int = 0) -> None:
        self.cfg = cfg
        self._assembled = assemble(cfg, kernels, random_config=random_config, seed=seed)
        a = self._assembled
        self.device, self.dtype, self.kernels = a.device, a.dtype, a.kernels
        self.model_config, self.spec, self.model = a.config, a.spec, a.model
        self.eos = set(self.spec.eos_token_ids)
        tokens = self._cache_tokens()
        self.cache, self.runner = attach_cache(self.model, cache_tokens=tokens, graphs=cfg.graphs, **a.shape(cfg))
        if not self.cache.fits_alone(cfg.max_model_len):
            raise OutOfPages(f"the cache holds {tokens} tokens, fewer than one request of max_model_len "
                             f"{cfg.max_model_len}; lower max_model_len or give the cache more memory")
        if cfg.prefix_cache:
            identity = repr((self.spec, cfg.dtype, cfg.page_size)).encode()
            if not self.cache.enable_prefix(hashlib.blake2b(identity, digest_size=16).digest()):
                print("holon_amd: this model keeps state that pages do not hold whole; prompts share nothing",
                      file=sys.stderr)
        self.sampler = Sampler(self.kernels, cfg.max_seqs, self.device)
        budget = min(cfg.max_step_tokens, cfg.chunk_with_decode or cfg.max_step_tokens)
        if self.model.cut(0, budget) < 1:
            raise ValueError(f"no prompt portion of {budget} tokens (max_step_tokens, chunk_with_decode) ends where this "
                             "model's parts allow a portion to end; raise them")
        self.sched = Scheduler(self.cache, cfg.max_step_tokens, cfg.max_model_len, cfg.chunk_with_decode,
                               on_admit=self._on_admit, cut=self.model.cut)
        self._ids = itertools.count()
        self._live: dict[str, list[Seq]] = {}
        self._siblings: dict[Seq, list[Seq]] = {}         # n > 1: waiting until the first sequence's prompt is cached
        self._prompt_lp: dict[Seq, Logprobs] = {}         # sequences still gathering prompt log-probabilities
        self._inflight: _Launched | None = None           # the step that runs while the next one is scheduled
        self._token_bufs = [torch.empty(cfg.max_seqs, dtype=torch.int32, pin_memory=self.device.type == "cuda")
                            for _ in range(2)]
        self._turn = 0
        self.steps = 0

    def _on_admit(self, seq: Seq) -> None:
        self.sampler.admit(seq.slot, seq.params)
        if seq.cached_tokens is None:                     # the first admission's hit; later ones are recomputation
            seq.cached_tokens = seq.num_computed

    @classmethod
    def from_random(cls, config_json: dict, seed: int, cfg: EngineConfig, kernels=None) -> "Engine":
        """An engine over random weights drawn on the device from a config.json dict (no folder is read)."""
        return cls(cfg, kernels, random_config=config_json, seed=seed)

    # -- memory accounting ----------------------------------------------------------------------------------------
    def token_bytes(self) -> int:
        """Bytes of paged state one token takes over all runs of the model."""
        item = torch.empty((), dtype=self.dtype).element_size()
        return sum(d.elems * (torch.empty((), dtype=d.dtype).element_size() if d.dtype else item)
                   for decls in self.model.state_decls() for d in decls if hasattr(d, "elems"))

    def _cache_tokens(self) -> int:
        cfg = self.cfg
        if cfg.cache_tokens is not None:
            return cfg.cache_tokens
        per_token = max(1, self.token_bytes())
        if cfg.state_memory is not None:
            budget = cfg.state_memory
        elif self.device.type == "cuda":
            peak = self._profile_step()
            free, _ = torch.cuda.mem_get_info(self.device)
            budget = int(free * cfg.memory_fraction) - peak
            print(f"holon_amd: weights {self.model.nbytes() / 2**30:.2f} GiB, {free / 2**30:.1f} GiB free, a step takes "
                  f"up to {peak / 2**30:.2f} GiB, {max(budget, 0) / 2**30:.1f} GiB for the cache ({per_token} B a token)",
                  file=sys.stderr)
        else:
            budget = cfg.max_seqs * cfg.max_model_len * per_token
        live = cfg.max_seqs * cfg.max_model_len          # live requests never hold more; what is beyond keeps prompts
        shared = CACHED_PREFIX_TOKENS if cfg.prefix_cache and self.device.type == "cuda" else 0    # others may start with
        tokens = min(budget // per_token, max(live, shared))
        return max(int(tokens), 0) // cfg.page_size * cfg.page_size or cfg.page_size

    def _profile_step(self) -> int:
        """Bytes the largest steps allocate beside weights and cache, measured on a cache just large enough for them
        (core/holon/core/executor.py:208-234): a step of `max_step_tokens` prompt tokens over as many rows as fit,
        every row sampled, and a step of `max_seqs` decode rows, sampled with filters and log-probabilities."""
        cfg, device = self.cfg, self.device
        longest = cfg.max_model_len - 1
        rows = min(cfg.max_seqs, max(1, -(-cfg.max_step_tokens // longest)))
        per_row = min(longest, cfg.max_step_tokens // rows)
        pages = rows * -(-(per_row + 1) // cfg.page_size) + cfg.max_seqs
        cache, runner = attach_cache(self.model, cache_tokens=pages * cfg.page_size, graphs=False,
                                     **self._assembled.shape(cfg))
        sampler = Sampler(self.kernels, cfg.max_seqs, device)
        torch.cuda.synchronize(device)
        torch.cuda.reset_peak_memory_stats(device)
        base = torch.cuda.memory_allocated(device)
        slots = [cache.admit() for _ in range(min(cfg.max_seqs, cfg.max_step_tokens))]
        params = SamplingParams(temperature=1.0, top_k=50, top_p=0.9, min_p=0.01, seed=0)
        for slot in slots:
            sampler.admit(slot, params)
        for slot in slots[:rows]:
            cache.reserve(slot, per_row)
        runner.run([StepRow(slot, 0, [0] * per_row, [per_row - 1]) for slot in slots[:rows]])
        for slot in slots:
            cache.reserve(slot, cache.computed[slot] + 1)
        logits = runner.run([StepRow(slot, cache.computed[slot], [0], [0]) for slot in slots])
        where = np.array(slots, dtype=np.int64)
        drawn = sampler.sample(logits, where, np.array([cache.computed[s] for s in slots], dtype=np.int64))
        self.kernels.logprobs(logits, drawn, 32)
        torch.cuda.synchronize(device)
        peak = torch.cuda.max_memory_allocated(device) - base
        del logits, drawn, runner, cache, sampler
        for site in self.model.sites:
            site.detach()
        torch.cuda.empty_cache()
        return int(peak * 1.1) + (64 << 20)           # the allocator's rounding and fragmentation

    # -- requests -------------------------------------------------------------------------------------------------
    def _check_prompt(self, token_ids: list[int]) -> None:
        room = self.cfg.max_model_len - len(token_ids)
        if not token_ids or room < 1:
            raise ValueError(f"a prompt has 1 to {self.cfg.max_model_len - 1} tokens (max_model_len "
                             f"{self.cfg.max_model_len} less one to generate); this one has {len(token_ids)}")
        bad = [t for t in token_ids if not 0 <= t < self.spec.vocab]
        if bad:
            raise ValueError(f"token id {bad[0]} is outside the vocabulary of {self.spec.vocab}")

    def add(self, token_ids: list[int], params: SamplingParams | None = None, rid: str | None = None) -> str:
        """Queue a prompt; returns the request's id. `params.n` sequences are drawn for it, each with a seed of its
        own derived from the request's (core/holon/core/engine.py:332-376): what a sequence draws depends on its
        seed and positions alone. With shared prefixes only the first sequence is queued now; the others follow when
        its prompt is in the cache, and start from there."""
        params = params if params is not None else SamplingParams()
        params.check()
        self._check_prompt(token_ids)
        if rid is None:
            rid = str(next(self._ids))
        if rid in self._live:
            raise ValueError(f"there is a live request with the id {rid!r} already")
        seed = secrets.randbits(63) if params.seed is None else params.seed
        seqs = [Seq(rid=rid, tokens=list(token_ids), index=i,
                    params=dataclasses.replace(params, seed=sequence_seed(seed, i),
                                               prompt_logprobs=params.prompt_logprobs if i == 0 else None))
                for i in range(params.n)]
        self._live[rid] = seqs
        head = seqs[0]
        if head.params.prompt_logprobs is not None:      # every position computed, in portions whose logits stay small
            head.share_prefix, head.portion_cap = False, PROMPT_LOGPROB_PORTION
            self._prompt_lp[head] = Logprobs([], [], [])
        self.sched.add(head)
        if self.cache.prefix is not None and len(seqs) > 1:
            self._siblings[head] = seqs[1:]
        else:
            for seq in seqs[1:]:
                self.sched.add(seq)
        return rid

    def has_work(self) -> bool:
        return len(self.sched) > 0 or self._inflight is not None

    def idle_for(self) -> float | None:
        """How long a serving loop may wait for new requests before its next `step`: 0 while a request can run, None
        (as long as it likes) when there is no work."""
        return 0.0 if self.has_work() else None

    def abort(self, rid: str, reason: str = "abort") -> list[TokenDelta]:
        """End request `rid` now. One closing delta for each of its sequences that had not finished, whether it ran,
        waited in line or had not been queued yet."""
        seqs = self._live.pop(rid, [])
        held_back = [s for seq in seqs for s in self._siblings.pop(seq, [])]
        closing = []
        for seq in seqs:
            if seq.status is Status.FINISHED:
                continue
            if seq in held_back:
                seq.status, seq.finish_reason = Status.FINISHED, reason
            else:
                self.sched.retire(seq, reason)
            self._prompt_lp.pop(seq, None)
            closing.append(TokenDelta(rid, [], reason, index=seq.index))
        closing.sort(key=lambda d: d.index)
        return closing + self._settle()

    def stats(self) -> dict:
        return {"waiting": len(self.sched) - self.sched.n_running, "running": self.sched.n_running,
                "preemptions": self.sched.preemptions, "mixed_steps": self.sched.mixed_steps, "steps": self.steps,
                "free_pages": min((g.pool.free for g in self.cache.groups), default=0),
                "graphs": len(getattr(self.runner, "graphs", {})),
                "prefix_tokens_saved": self.cache.tokens_saved,
                "cached_pages": len(self.cache.prefix.entries) if self.cache.prefix is not None else 0,
                "products": self.products()}

    def products(self) -> dict[str, str]:
        """What every matrix product with a choice took so far, as `kind:NxK:rows` -> form: the syntax
        `EngineConfig.product_pins` accepts, so a timed run's choices can be pinned for the next."""
        plan = getattr(self.kernels, "plan", None)
        return plan.report() if plan is not None else {}

    def flush_prefix(self) -> list[TokenDelta]:
        """Drop the cached prompt blocks (core/holon/core/engine.py:418-420); the step in flight is committed first."""
        deltas = self.drain()
        self.cache.flush_prefix()
        return deltas

    def close(self) -> None:
        self.drain()
        self._live.clear()

    def generate(self, prompts: list[list[int]], params: SamplingParams | None = None) -> list[list[int]]:
        """Run the prompts to their end; the generated token ids of each, in the prompts' order."""
        if params is not None and params.n != 1:
            raise ValueError("generate() gives back one list of tokens a prompt: for n > 1 add the prompts and read step()'s deltas")
        streams: dict[str, list[int]] = {self.add(p, params): [] for p in prompts}
        unfinished = len(streams)
        while unfinished:
            for delta in self.step():
                stream = streams.get(delta.rid)
                if stream is not None:
                    stream.extend(delta.token_ids)
                    unfinished -= delta.finish_reason is not None
        self._settle()
        return list(streams.values())

    def _settle(self) -> list[TokenDelta]:
        """When the line is empty, what is still in flight are rows of requests that have ended since: commit them now
        (they are dropped), so that nothing is left to wait for."""
        return self.drain() if not len(self.sched) else []

    # -- one step -------------------------------------------------------------------------------------------------
    @torch.no_grad()
    def step(self) -> list[TokenDelta]:
        """Schedule and launch one step, then commit the one before it while this one runs (`overlap`), or this one at
        once. The deltas are those of the step committed. core/holon/core/engine.py:494-524."""
        deltas: list[TokenDelta] = []
        rows = self.sched.schedule()
        if rows is None and self._inflight is not None:      # what is in flight may bring tokens or finish requests
            deltas += self.drain()
            rows = self.sched.schedule()
        if rows is None:
            if self.has_work():
                raise RuntimeError("requests are waiting but the scheduler found nothing to run")
            return deltas
        launched = self._launch(rows)
        deltas += self.drain()
        if self.cfg.overlap and not launched.sync:
            self._inflight = launched
        else:
            deltas += self._commit(launched)
        return deltas

    def _launch(self, rows: list) -> "_Launched":
        """Run the rows and draw their tokens, all on the device; nothing here waits for it."""
        step_rows, owed, places, at = [], [], [], 0
        for seq, n, m in rows:
            want = list(range(*self._prompt_places(seq, n))) if seq in self._prompt_lp else []
            if want:
                owed.append((seq, at, len(want), seq.tokens[seq.num_computed + want[0] + 1:
                                                            seq.num_computed + want[-1] + 2]))
            at += len(want)
            if m:
                places.append(at)
                want.append(n - 1)
                at += 1
            if seq.pending:                          # its token is the one the step in flight draws: still on the device
                step_rows.append(StepRow(seq.slot, seq.num_computed, [0], want, on_device=True))
            else:
                step_rows.append(StepRow(seq.slot, seq.num_computed,
                                         seq.tokens[seq.num_computed: seq.num_computed + n], want))
        logits = self.runner.run(step_rows)
        self.steps += 1
        out = _Launched(rows=rows, sync=bool(owed))
        for seq, lo, count, targets in owed:         # (these read the host: such a step is committed at once)
            self._gather_prompt_logprobs(seq, logits[lo: lo + count], targets)
        if owed and places:
            logits = logits.index_select(0, torch.tensor(places, device=logits.device))
        sampled = [(seq, n) for seq, n, m in rows if m]
        if sampled:
            slots = np.array([seq.slot for seq, _ in sampled], dtype=np.int64)
            positions = np.array([seq.num_computed + n for seq, n in sampled], dtype=np.int64)
            if len(sampled) == len(rows) and not owed:       # every row draws: slots and positions are on the device
                where = self.runner.last_slots[: len(rows)]
                drawn = self.sampler.sample(logits, slots, positions, (where, self.runner.last_lens[: len(rows)]))
            else:
                where = torch.from_numpy(slots.astype(np.int32)).to(self.device, non_blocking=True)
                drawn = self.sampler.sample(logits, slots, positions)
            self.kernels.store_tokens(self.runner.last_token, where, drawn)
            k = max((seq.params.logprobs if seq.params.logprobs is not None else -1) for seq, _ in sampled)
            out.tokens = self._to_host(drawn)
            if k >= 0:
                out.logprobs = [self._to_host(t, fresh=True) for t in self.kernels.logprobs(logits, drawn, k)]
        if self.device.type == "cuda":
            out.done = torch.cuda.Event()
            out.done.record()
        for seq, n, m in rows:
            seq.num_computed += n
            if m:
                seq.pending += 1
                if seq.status is not Status.RUNNING:
                    self.sched.prompt_done(seq)
        return out

    def _to_host(self, t: torch.Tensor, fresh: bool = False) -> torch.Tensor:
        """A copy of `t` on its way to pinned host memory (valid once the step's event has passed). The drawn tokens
        use two buffers in turn: at most one step is in flight while the next is launched."""
        if self.device.type != "cuda":
            return t
        if fresh:
            host = torch.empty(t.shape, dtype=t.dtype, pin_memory=True)
        else:
            self._turn ^= 1
            host = self._token_bufs[self._turn][: t.shape[0]]
        host.copy_(t, non_blocking=True)
        return host

    def drain(self) -> list[TokenDelta]:
        """Commit the step in flight, if any: nothing runs on the device afterwards."""
        prev, self._inflight = self._inflight, None
        return self._commit(prev) if prev is not None else []

    def _commit(self, step: "_Launched") -> list[TokenDelta]:
        """The host's books once a step's tokens are on the host: tokens appended, requests finished, pages published,
        deltas made. A row of a request that finished (or was aborted) after the row was launched is dropped."""
        if step.done is not None:
            step.done.synchronize()
        tokens = step.tokens.tolist() if step.tokens is not None else []
        lps = [t.tolist() for t in step.logprobs] if step.logprobs is not None else None
        deltas, at = [], 0
        chains, page = self.cache.chain, self.cache.page_size
        for seq, n, m in step.rows:
            if m:
                at += 1
            if seq.status is Status.FINISHED:
                continue
            if seq.slot >= 0:
                chain = chains[seq.slot]              # (the check `publish` starts with, without the call: per row, per step)
                if chain is not None and min(seq.num_computed, len(seq.tokens)) // page > len(chain):
                    self.cache.publish(seq.slot, seq.tokens)
            if not m:
                continue
            token = tokens[at - 1]
            seq.pending -= 1
            seq.tokens.append(token)
            self._release_siblings(seq)
            reason = seq.verdict(token, self.eos, self.cfg.max_model_len)
            if reason is not None:
                self._close(seq, reason)
            delta = TokenDelta(seq.rid, [token], reason, index=seq.index)
            if seq.params.logprobs is not None:
                k, row = seq.params.logprobs, at - 1
                delta.logprobs = Logprobs([lps[0][row]], [lps[1][row][:k]], [lps[2][row][:k]])
            if not seq.reported:                       # the first delta also carries what belongs to the prompt
                seq.reported = True
                delta.prompt_logprobs = self._prompt_lp.pop(seq, None)
                delta.cached_tokens = seq.cached_tokens
            deltas.append(delta)
        return deltas

    def _release_siblings(self, seq: Seq) -> None:
        """The first sequence of a request has drawn a token, so its prompt is in the cache: the request's other
        sequences join the head of the line, in their order."""
        for sibling in reversed(self._siblings.pop(seq, ())):
            self.sched.add(sibling, front=True)

    def _close(self, seq: Seq, reason: str) -> None:
        self.sched.retire(seq, reason)
        rest = [s for s in self._live.get(seq.rid, ()) if s is not seq]
        if rest:
            self._live[seq.rid] = rest
        else:
            self._live.pop(seq.rid, None)

    def _prompt_places(self, seq: Seq, n: int) -> tuple[int, int]:
        """The places among the next `n` tokens of `seq` whose logits predict a prompt token not yet recorded (a
        request preempted in its prompt computes some again). core/holon/core/engine.py:588-602."""
        start, have = seq.num_computed, len(self._prompt_lp[seq].token)
        lo, hi = max(start, have), min(start + n, seq.prompt_len - 1)
        return (lo - start, hi - start) if lo < hi else (0, 0)

    def _gather_prompt_logprobs(self, seq: Seq, logits: torch.Tensor, targets: list[int]) -> None:
        acc, k = self._prompt_lp[seq], seq.params.prompt_logprobs
        tokens = torch.tensor(targets, dtype=torch.int32, device=logits.device)
        lp, ids, top = (t.tolist() for t in self.kernels.logprobs(logits.contiguous(), tokens, k))
        acc.token += lp
        acc.top_ids += [row[:k] for row in ids]
        acc.top += [row[:k] for row in top]
