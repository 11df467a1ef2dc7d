"""Shared by the tests: tiny configurations, model folders, trace builders, error budgets."""
from __future__ import annotations

import json
import math
import pathlib
import random

import torch
from safetensors import safe_open
from safetensors.torch import save_file

# Two tiny Qwen3 configurations that differ in every size and option.
CONFIG_A = {"architectures": ["Qwen3ForCausalLM"], "num_hidden_layers": 2, "hidden_size": 64,
            "num_attention_heads": 4, "num_key_value_heads": 1, "head_dim": 16, "intermediate_size": 128,
            "vocab_size": 256, "rope_theta": 10000.0, "rms_norm_eps": 1e-6, "tie_word_embeddings": True,
            "max_position_embeddings": 512}
CONFIG_B = {"architectures": ["Qwen3ForCausalLM"], "num_hidden_layers": 3, "hidden_size": 96,
            "num_attention_heads": 6, "num_key_value_heads": 3, "head_dim": 32, "intermediate_size": 160,
            "vocab_size": 384, "rope_theta": 1e6, "rms_norm_eps": 1e-5, "tie_word_embeddings": False,
            "max_position_embeddings": 512}
# A third with head_dim 64 (the matrix-core attention kernels' smallest) and widths that are no power of two.
CONFIG_C = {"architectures": ["Qwen3ForCausalLM"], "num_hidden_layers": 2, "hidden_size": 120,
            "num_attention_heads": 6, "num_key_value_heads": 2, "head_dim": 64, "intermediate_size": 200,
            "vocab_size": 1000, "rope_parameters": {"rope_theta": 50000.0, "rope_type": "default"},
            "rms_norm_eps": 1e-6, "tie_word_embeddings": False, "max_position_embeddings": 1024}


def make_folder(path: pathlib.Path, cfg: dict, seed: int, qk_gain: float = 1.0, scale: float = 1.0) -> pathlib.Path:
    """A model folder with random weights. `qk_gain` multiplies the q/k norm weights, which makes attention scores
    peaked, so that a wrong or missing key changes the result visibly; `scale` multiplies projections."""
    from holon_amd.weights import write_random_model
    write_random_model(cfg, seed, path)
    if qk_gain != 1.0 or scale != 1.0:
        tensors = {}
        with safe_open(str(path / "model.safetensors"), "pt") as f:
            for name in f.keys():
                t = f.get_tensor(name)
                if name.endswith(("q_norm.weight", "k_norm.weight")):
                    t = (t.float() * qk_gain).to(t.dtype)
                elif scale != 1.0 and "proj" in name:
                    t = (t.float() * scale).to(t.dtype)
                tensors[name] = t
        save_file(tensors, str(path / "model.safetensors"))
    return path


def random_ids(n: int, vocab: int, seed: int) -> list[int]:
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


# -- budgets ------------------------------------------------------------------------------------------------------
U32 = torch.finfo(torch.float32).eps / 2


def op_budget_usage(cand: torch.Tensor, ref: torch.Tensor, dtype: torch.dtype, reduction_len: int) -> float:
    """How much of the error budget of one operation `cand` uses against `ref` (<= 1 passes): per element
    |c - r| <= 3u|r| + 6s rms(r), on average <= s rms(r), with u the roundoff of `dtype` and s = u + u32 sqrt(K)
    for sums of K terms (the reference judge's model, judge/holon_judge/l0.py:1-21)."""
    u = torch.finfo(dtype).eps / 2
    s = u + U32 * math.sqrt(reduction_len)
    c, r = cand.detach().double().cpu().flatten(), ref.detach().double().cpu().flatten()
    assert c.shape == r.shape, (c.shape, r.shape)
    assert torch.isfinite(c).all(), "non-finite values"
    err = (c - r).abs()
    rms = r.square().mean().sqrt().item()
    if rms == 0:
        return 0.0 if not err.any() else math.inf
    per = (err / (3 * u * r.abs() + 6 * s * rms)).max().item()
    mean = (err.mean() / (s * rms)).item()
    return max(per, mean)


def rel_rms(cand: torch.Tensor, ref: torch.Tensor) -> float:
    c, r = cand.double().cpu(), ref.double().cpu()
    return ((c - r).square().mean().sqrt() / r.square().mean().sqrt()).item()


def max_over_rms(cand: torch.Tensor, ref: torch.Tensor) -> float:
    c, r = cand.double().cpu(), ref.double().cpu()
    return ((c - r).abs().max() / r.square().mean().sqrt()).item()


FP32_RMS, FP32_MAX = 2e-5, 2e-4     # float32 engine against the plain float32 model, relative to the logits' rms


def assert_fp32_close(got: torch.Tensor, want: torch.Tensor, what: str = "") -> None:
    assert got.shape == want.shape, (got.shape, want.shape)
    assert torch.isfinite(got).all(), f"{what}: non-finite logits"
    r, m = rel_rms(got, want), max_over_rms(got, want)
    assert r <= FP32_RMS and m <= FP32_MAX, f"{what}: float32 logits differ: rms {r:.3g} (<= {FP32_RMS}), max {m:.3g} (<= {FP32_MAX})"


def assert_bf16_close(got: torch.Tensor, want32: torch.Tensor, floor16: torch.Tensor, what: str = "") -> None:
    """bfloat16 engine logits against the plain float32 model: no further away than twice the distance of the plain
    model run in bfloat16 (its rounding floor), as rms and as the largest element."""
    assert got.shape == want32.shape, (got.shape, want32.shape)
    assert torch.isfinite(got).all(), f"{what}: non-finite logits"
    r, m = rel_rms(got, want32), max_over_rms(got, want32)
    fr, fm = rel_rms(floor16, want32), max_over_rms(floor16, want32)
    assert r <= 2 * fr + 1e-3 and m <= 2 * fm + 5e-3, \
        f"{what}: bfloat16 logits differ: rms {r:.3g} (floor {fr:.3g}), max {m:.3g} (floor {fm:.3g})"


def assert_greedy_follows(plain, prompt: list[int], got: list[int], margin: float = 0.05) -> int:
    """Every generated token is the plain model's most likely one given the tokens before it, wherever the plain
    model's two best logits are further apart than `margin` of the logits' spread (closer than that, rounding may
    decide). Returns how many tokens were held to the plain model's choice."""
    ids, held = list(prompt), 0
    for token in got:
        logits = plain.logits(ids)[-1].float()
        top = logits.topk(2).values
        if float(top[0] - top[1]) > margin * float(logits.std()):
            assert token == int(logits.argmax()), f"token {len(ids)}: {token}, the plain model says {int(logits.argmax())}"
            held += 1
        ids.append(token)
    return held


# -- traces -------------------------------------------------------------------------------------------------------
class Trace:
    """Steps for the replayer, and for each step the (request, position) of every wanted logit row."""

    def __init__(self) -> None:
        self.steps: list[dict] = []
        self.expect: list[list[tuple[str, int]]] = []

    def add(self, entries: list[tuple[str, int, list[int], list[int]]], end: list[str] = ()) -> None:
        """entries: (id, position of the first token, tokens, want)."""
        self.steps.append({"step": len(self.steps),
                           "entries": [{"id": rid, "tokens": toks, "want": want} for rid, _, toks, want in entries],
                           "end": list(end)})
        self.expect.append([(rid, start + w) for rid, start, _, want in entries for w in want])

    def jsonl(self) -> str:
        return "".join(json.dumps(s) + "\n" for s in self.steps)


def trace_whole(requests: dict[str, list[int]]) -> Trace:
    t = Trace()
    for rid, ids in requests.items():
        t.add([(rid, 0, ids, list(range(len(ids))))], end=[rid])
    return t


def trace_decode_tail(rid: str, ids: list[int], tail: int = 32) -> Trace:
    t = Trace()
    head = len(ids) - tail
    assert head >= 1
    t.add([(rid, 0, ids[:head], list(range(head)))])
    for p in range(head, len(ids)):
        t.add([(rid, p, [ids[p]], [0])], end=[rid] if p == len(ids) - 1 else [])
    return t


def trace_chunks(rid: str, ids: list[int], sizes: list[int]) -> Trace:
    t, at, i = Trace(), 0, 0
    while at < len(ids):
        n = min(sizes[i % len(sizes)], len(ids) - at)
        if len(ids) - at - n == 1:                 # never leave a single token for the last portion of this shape
            n += 1
        t.add([(rid, at, ids[at: at + n], list(range(n)))], end=[rid] if at + n == len(ids) else [])
        at += n
        i += 1
    return t


def trace_mixed(requests: dict[str, list[int]], seed: int, max_live: int = 4, decode_tail: int = 8,
                max_chunk: int = 19) -> Trace:
    """Up to `max_live` requests at a time: portions of prompts (2 .. max_chunk tokens) beside single decoded tokens
    (the last `decode_tail` tokens of each request go one by one); a request is sometimes left out of a step; a
    finished request ends and the next one starts, so its pages are used again."""
    rng = random.Random(seed)
    t = Trace()
    waiting = list(requests.items())
    live: dict[str, int] = {}
    while waiting or live:
        while waiting and len(live) < max_live:
            live[waiting.pop(0)[0]] = 0
        entries, end = [], []
        for rid in list(live):
            ids, at = requests[rid], live[rid]
            if len(live) > 1 and rng.random() < 0.2:
                continue                           # left out of this step
            left = len(ids) - at
            if left <= decode_tail:
                n = 1
            else:
                n = min(rng.randint(2, max_chunk), left - decode_tail)
                if n < 2:
                    n = left - decode_tail if left - decode_tail >= 1 else 1
            entries.append((rid, at, ids[at: at + n], list(range(n))))
            live[rid] = at + n
            if live[rid] == len(ids):
                end.append(rid)
                del live[rid]
        if entries:
            t.add(entries, end)
    return t


def peak_live_tokens(trace: Trace, round_to: int = 64) -> int:
    """The most tokens live requests hold at any time, each request's count rounded up to `round_to`."""
    held: dict[str, int] = {}
    peak = 0
    for step in trace.steps:
        for e in step["entries"]:
            held[e["id"]] = held.get(e["id"], 0) + len(e["tokens"])
        peak = max(peak, sum(-(-n // round_to) * round_to for n in held.values()))
        for rid in step["end"]:
            held.pop(rid, None)
    return peak


def run_trace(replayer, trace: Trace) -> dict[tuple[str, int], torch.Tensor]:
    """Replay in process; returns logits by (request, position)."""
    out = {}
    for step, expect in zip(trace.steps, trace.expect):
        logits = replayer.step(step["entries"], step["end"])
        if expect:
            logits = logits.float().cpu()
            assert logits.shape[0] == len(expect)
            for row, key in zip(logits, expect):
                out[key] = row
    return out


def gather(plain_logits: dict[str, torch.Tensor], got: dict[tuple[str, int], torch.Tensor]
           ) -> tuple[torch.Tensor, torch.Tensor]:
    keys = sorted(got)
    return torch.stack([got[k] for k in keys]), torch.stack([plain_logits[r][p] for r, p in keys])
