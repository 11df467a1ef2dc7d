"""A plain, slow Qwen3 dense model: whole sequences, no cache, one function per part.

This file is the yardstick the engine is compared with. It shares no code with `holon_amd`: it reads a model
folder by itself (config.json, model.safetensors, Hugging Face tensor names) and computes every token's logits from
the formulas of the reference engine, cited per function as `file:line` under the reference tree.

`dtype` is the activation and weight dtype. Every part computes in float32 inside and rounds its result to `dtype`
once, where the reference's oracles round; with `dtype=torch.float32` no rounding happens anywhere. The whole model
in float64 (`PlainQwen3(folder, torch.float64)`) computes every part in float64 instead (`computing_in`), rotation
angles included: the same formulas almost free of rounding, which tells how far the float32 evaluation itself is from
them.
"""
from __future__ import annotations

import contextlib
import json
import pathlib

import torch
from safetensors import safe_open


_WORK = [torch.float32]


def wide(x: torch.Tensor) -> torch.Tensor:
    """`x` in the type a part computes in: float32, or what `computing_in` says."""
    return x.to(_WORK[-1])


@contextlib.contextmanager
def computing_in(dtype: torch.dtype):
    """Inside, every part computes in `dtype` instead of float32."""
    _WORK.append(dtype)
    try:
        yield
    finally:
        _WORK.pop()


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) * weight over the last dim, one rounding at the end.
    std/holon_std/ops/reference.py:7-11 (offset 0 for Qwen3)."""
    x32 = wide(x)
    inv = torch.rsqrt((x32 * x32).mean(dim=-1, keepdim=True) + eps)
    return (x32 * inv * wide(weight)).to(x.dtype)


def rope_angles(positions: torch.Tensor, head_dim: int, theta: float) -> tuple[torch.Tensor, torch.Tensor]:
    """cos and sin of position * theta^(-2i/D), i < D/2, all float32.
    std/holon_std/ops/reference.py:24-26."""
    work = _WORK[-1]
    inv_freq = 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=work) / head_dim))
    angles = positions.to(work)[:, None] * inv_freq.to(positions.device)[None, :]
    return angles.cos(), angles.sin()


def rope_neox(x: torch.Tensor, positions: torch.Tensor, theta: float) -> torch.Tensor:
    """Half-split rotation of x [T, heads, D]: pairs are (i, i + D/2).
    std/holon_std/ops/reference.py:21-30."""
    half = x.shape[-1] // 2
    cos, sin = rope_angles(positions, x.shape[-1], theta)
    cos, sin = cos[:, None, :], sin[:, None, :]
    a, b = wide(x[..., :half]), wide(x[..., half:])
    return torch.cat((a * cos - b * sin, b * cos + a * sin), dim=-1).to(x.dtype)


def causal_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, window: int = 0) -> torch.Tensor:
    """One sequence from position 0. q [T, Hq, D], k and v [T, Hkv, D]; query head j reads kv head j // (Hq/Hkv);
    scores / sqrt(D); key j is hidden from query i when j > i (and, with a window W > 0, when i - j >= W).
    std/holon_std/mixers/gqa/reference.py:7-24."""
    t, hq, d = q.shape
    group = hq // k.shape[1]
    k32 = wide(k).repeat_interleave(group, dim=1)
    v32 = wide(v).repeat_interleave(group, dim=1)
    pos = torch.arange(t, device=q.device)
    out = []
    for lo in range(0, t, QUERY_ROWS):     # a query row's result does not depend on the other rows: the rows are taken
        rows = pos[lo: lo + QUERY_ROWS]    # some at a time only so that the [heads, rows, T] scores fit in memory
        scores = torch.einsum("qhd,khd->hqk", wide(q[lo: lo + QUERY_ROWS]), k32) / d ** 0.5
        hidden = pos[None, :] > rows[:, None]
        if window:
            hidden = hidden | (rows[:, None] - pos[None, :] >= window)
        probs = scores.masked_fill(hidden, float("-inf")).softmax(dim=-1)
        out.append(torch.einsum("hqk,khd->qhd", probs, v32).to(q.dtype))
    return torch.cat(out)


QUERY_ROWS = 4096


def linear(x: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """x @ weight.T, no bias, float32 accumulation, rounded to x's dtype.
    std/holon_std/ops/units.py:229 (F.linear); std/holon_std/ops/reference.py:33-34."""
    return (wide(x) @ wide(weight).T).to(x.dtype)


def silu_mul(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """silu(gate) in float32, rounded, times up in the activation dtype.
    std/holon_std/ffn/reference.py:7-12."""
    g = wide(gate)
    return (g * torch.sigmoid(g)).to(gate.dtype) * up


def swiglu(x: torch.Tensor, w_gate: torch.Tensor, w_up: torch.Tensor, w_down: torch.Tensor) -> torch.Tensor:
    """down(silu(gate(x)) * up(x)). std/holon_std/ffn/units.py:12-50."""
    return linear(silu_mul(linear(x, w_gate), linear(x, w_up)), w_down)


def attention_layer(x: torch.Tensor, positions: torch.Tensor, w: dict[str, torch.Tensor], prefix: str, cfg: dict,
                    window: int = 0) -> torch.Tensor:
    """q/k/v projections, per-head RMSNorm on q and k, then RoPE on q and k, causal attention, o projection.
    std/holon_std/mixers/gqa/units.py:254-263 (norm before rope), :282-294 (forward)."""
    t = x.shape[0]
    hq, hkv, d = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    eps = cfg["rms_norm_eps"]
    q = linear(x, w[prefix + "q_proj.weight"]).view(t, hq, d)
    k = linear(x, w[prefix + "k_proj.weight"]).view(t, hkv, d)
    v = linear(x, w[prefix + "v_proj.weight"]).view(t, hkv, d)
    q = rms_norm(q, w[prefix + "q_norm.weight"], eps)
    k = rms_norm(k, w[prefix + "k_norm.weight"], eps)
    theta = rope_theta(cfg)
    q, k = rope_neox(q, positions, theta), rope_neox(k, positions, theta)
    out = causal_attention(q, k, v, window)
    return linear(out.reshape(t, hq * d), w[prefix + "o_proj.weight"])


def block(h: torch.Tensor, positions: torch.Tensor, w: dict[str, torch.Tensor], i: int, cfg: dict) -> torch.Tensor:
    """Pre-norm residual block: h += attn(norm(h)); h += mlp(norm(h)); both adds in the activation dtype.
    std/holon_std/blocks/units.py:23-25; std/holon_std/ops/reference.py:14-18 (the add of add_rmsnorm)."""
    p = f"model.layers.{i}."
    eps = cfg["rms_norm_eps"]
    a = attention_layer(rms_norm(h, w[p + "input_layernorm.weight"], eps), positions, w, p + "self_attn.", cfg)
    h = h + a
    x = rms_norm(h, w[p + "post_attention_layernorm.weight"], eps)
    m = swiglu(x, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
    return h + m


def rope_theta(cfg: dict) -> float:
    """plugins/holon_plugins/models/qwen3/recipe.py:32-38."""
    params = cfg.get("rope_parameters") or {"rope_theta": cfg["rope_theta"]}
    return float(params["rope_theta"])


def logits_of(ids: list[int], w: dict[str, torch.Tensor], cfg: dict) -> torch.Tensor:
    """Float32 logits [T, V] of every token of one sequence (float64 from a float64 model).
    core/holon/core/build.py:296-307 (embed, blocks, final norm, head); std/holon_std/ops/units.py:345-348 (head reads
    the embedding when tied; logits are float32)."""
    table = w["model.embed_tokens.weight"]
    h = table[torch.tensor(ids, dtype=torch.long, device=table.device)]
    positions = torch.arange(len(ids), device=table.device)
    for i in range(cfg["num_hidden_layers"]):
        h = block(h, positions, w, i, cfg)
    h = rms_norm(h, w["model.norm.weight"], cfg["rms_norm_eps"])
    head = w["model.embed_tokens.weight"] if cfg.get("tie_word_embeddings", False) else w["lm_head.weight"]
    return wide(linear(h, head))


def read_folder(folder: str | pathlib.Path, dtype: torch.dtype = torch.float32, device: str = "cpu"
                ) -> tuple[dict, dict[str, torch.Tensor]]:
    """config.json as a dict, and every tensor of model.safetensors by its stored name, cast to `dtype`. `device`:
    where the same plain functions run (a test of a wide model may put them on the GPU to be done in seconds)."""
    folder = pathlib.Path(folder)
    cfg = json.loads((folder / "config.json").read_text())
    weights = {}
    with safe_open(str(folder / "model.safetensors"), "pt", device="cpu") as f:
        for name in f.keys():
            weights[name] = f.get_tensor(name).to(dtype).to(device)
    return cfg, weights


class PlainQwen3:
    """The plain model of one folder: `logits(ids)` for a whole sequence, `greedy(ids, n)` by recomputing it."""

    def __init__(self, folder: str | pathlib.Path, dtype: torch.dtype = torch.float32, device: str = "cpu") -> None:
        self.cfg, self.weights = read_folder(folder, dtype, device)
        self.work = torch.float64 if dtype == torch.float64 else torch.float32

    @classmethod
    def from_tensors(cls, cfg: dict, weights: dict[str, torch.Tensor], dtype: torch.dtype = torch.float32
                     ) -> "PlainQwen3":
        """The plain model over tensors that are already in memory (config.json's keys, Hugging Face tensor names),
        cast to `dtype` where they lie: for models too large to write as a folder in a test."""
        self = cls.__new__(cls)
        self.cfg, self.weights = dict(cfg), {name: t.to(dtype) for name, t in weights.items()}
        self.work = torch.float64 if dtype == torch.float64 else torch.float32
        return self

    @torch.no_grad()
    def logits(self, ids: list[int]) -> torch.Tensor:
        with computing_in(self.work):
            return logits_of(ids, self.weights, self.cfg)

    @torch.no_grad()
    def greedy(self, ids: list[int], n: int) -> list[int]:
        ids, out = list(ids), []
        for _ in range(n):
            token = int(self.logits(ids)[-1].argmax())
            out.append(token)
            ids.append(token)
        return out
