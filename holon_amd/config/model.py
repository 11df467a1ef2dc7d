"""Typed model configuration, read from a checkpoint's config.json.

Every size and constant of the model comes from here; no code below holds one. Required keys have no default, as in
the reference's recipe (plugins/holon_plugins/models/qwen3/recipe.py:41-59: every size is `c["..."]`), and the options
the reference refuses are refused here with the same meaning (recipe.py:32-46).
"""
from __future__ import annotations

import dataclasses
import json
import pathlib
from collections.abc import Mapping
from typing import Any


class ConfigError(ValueError):
    """config.json is missing a key, or asks for something this architecture does not do."""


def _eos_ids(*sources: Mapping[str, Any] | None) -> tuple[int, ...]:
    """The union of `eos_token_id` (an int or a list) over config.json and generation_config.json
    (std/holon_std/weights/hf/source.py:62-66)."""
    out: list[int] = []
    for src in sources:
        value = (src or {}).get("eos_token_id")
        for token in ([] if value is None else value if isinstance(value, list) else [value]):
            if token not in out:
                out.append(int(token))
    return tuple(out)


@dataclasses.dataclass(frozen=True)
class Qwen3Config:
    """Qwen3 dense, as config.json describes it."""

    hidden_size: int
    vocab_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    intermediate_size: int
    rms_norm_eps: float
    rope_theta: float
    tie_word_embeddings: bool = False
    max_position_embeddings: int | None = None
    eos_token_ids: tuple[int, ...] = ()
    architecture: str = "Qwen3ForCausalLM"

    REQUIRED = ("hidden_size", "vocab_size", "num_hidden_layers", "num_attention_heads", "num_key_value_heads",
                "head_dim", "intermediate_size", "rms_norm_eps")

    def __post_init__(self) -> None:
        for name in ("hidden_size", "vocab_size", "num_hidden_layers", "num_attention_heads", "num_key_value_heads",
                     "head_dim", "intermediate_size"):
            value = getattr(self, name)
            if not isinstance(value, int) or isinstance(value, bool) or value < 1:
                raise ConfigError(f"{name} must be a positive integer, got {value!r}")
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError(f"num_attention_heads {self.num_attention_heads} is not a multiple of "
                              f"num_key_value_heads {self.num_key_value_heads}")
        if self.head_dim % 2:
            raise ConfigError(f"head_dim {self.head_dim} must be even (rotary pairs)")
        if not self.rms_norm_eps >= 0 or not self.rope_theta > 0:
            raise ConfigError(f"rms_norm_eps {self.rms_norm_eps} must be >= 0 and rope_theta {self.rope_theta} > 0")

    @classmethod
    def from_dict(cls, c: Mapping[str, Any], generation: Mapping[str, Any] | None = None) -> "Qwen3Config":
        missing = [k for k in cls.REQUIRED if k not in c]
        rope = c.get("rope_parameters") or None
        if rope is None:
            if "rope_theta" not in c:
                missing.append("rope_theta")
            rope = {"rope_theta": c.get("rope_theta"), **(c.get("rope_scaling") or {})}
        elif "rope_theta" not in rope:
            missing.append("rope_parameters.rope_theta")
        if missing:
            raise ConfigError(f"config.json lacks required keys: {', '.join(missing)}")
        kind = rope.get("rope_type", rope.get("type", "default"))
        if kind != "default":
            raise NotImplementedError(f"qwen3: rope type {kind!r} is not supported")
        refused = {k: c[k] for k in ("attention_bias", "use_sliding_window") if c.get(k)}
        if refused:
            raise NotImplementedError(f"qwen3: config options not supported: {refused}")
        archs = c.get("architectures") or ["Qwen3ForCausalLM"]
        return cls(hidden_size=c["hidden_size"], vocab_size=c["vocab_size"],
                   num_hidden_layers=c["num_hidden_layers"], num_attention_heads=c["num_attention_heads"],
                   num_key_value_heads=c["num_key_value_heads"], head_dim=c["head_dim"],
                   intermediate_size=c["intermediate_size"], rms_norm_eps=float(c["rms_norm_eps"]),
                   rope_theta=float(rope["rope_theta"]), tie_word_embeddings=bool(c.get("tie_word_embeddings", False)),
                   max_position_embeddings=c.get("max_position_embeddings"),
                   eos_token_ids=_eos_ids(c, generation), architecture=archs[0])

    def to_dict(self) -> dict[str, Any]:
        """config.json for a folder written from this configuration."""
        out: dict[str, Any] = {
            "architectures": [self.architecture], "model_type": "qwen3",
            "hidden_size": self.hidden_size, "vocab_size": self.vocab_size,
            "num_hidden_layers": self.num_hidden_layers, "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads, "head_dim": self.head_dim,
            "intermediate_size": self.intermediate_size, "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta, "tie_word_embeddings": self.tie_word_embeddings,
            "attention_bias": False, "use_sliding_window": False, "hidden_act": "silu"}
        if self.max_position_embeddings is not None:
            out["max_position_embeddings"] = self.max_position_embeddings
        if self.eos_token_ids:
            out["eos_token_id"] = list(self.eos_token_ids) if len(self.eos_token_ids) > 1 else self.eos_token_ids[0]
        return out


def read_config_json(folder: str | pathlib.Path) -> tuple[dict[str, Any], dict[str, Any] | None]:
    """config.json (required) and generation_config.json (optional) of a model folder, as dicts."""
    folder = pathlib.Path(folder)
    path = folder / "config.json"
    if not path.is_file():
        raise FileNotFoundError(f"{folder}: no config.json")
    gen = folder / "generation_config.json"
    return json.loads(path.read_text()), (json.loads(gen.read_text()) if gen.is_file() else None)
