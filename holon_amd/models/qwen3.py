"""Qwen3 dense: its typed configuration, and configuration to spec. plugins/holon_plugins/models/qwen3/recipe.py:10-59.

Pre-norm decoder; grouped-query attention with an RMSNorm over head_dim on q and k before the rotary embedding;
SwiGLU feed-forward; the head may be tied to the embedding.

Required config.json keys have no default, as in the reference's recipe (recipe.py:41-59: every size is `c["..."]`),
and the options the reference refuses are refused here with the same meaning (recipe.py:32-46)."""
from __future__ import annotations

import dataclasses
from collections.abc import Mapping
from typing import Any

from ..config.model import ConfigError, eos_ids
from ..registry import register_architecture
from ..spec import LayerSpec, ModelSpec, PartRef, WeightRule, in_order

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
                   eos_token_ids=eos_ids(c, generation), architecture=archs[0])

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


HF_RULES = (
    WeightRule("model.embed_tokens.weight", "embed.weight"),
    WeightRule("model.norm.weight", "norm.weight"),
    WeightRule("lm_head.weight", "lm_head.weight"),
    WeightRule("model.layers.{i}.input_layernorm.{rest}", "layers.{i}.input_norm.{rest}"),
    WeightRule("model.layers.{i}.post_attention_layernorm.{rest}", "layers.{i}.post_norm.{rest}"),
    WeightRule("model.layers.{i}.self_attn.{rest}", "layers.{i}.mixer.{rest}"),
    WeightRule("model.layers.{i}.mlp.{rest}", "layers.{i}.ffn.{rest}"),
)


def recipe(c: Qwen3Config) -> ModelSpec:
    norm = PartRef("norm", "rmsnorm", eps=c.rms_norm_eps)
    mixer = PartRef("mixer", "gqa", heads=c.num_attention_heads, kv_heads=c.num_key_value_heads,
                    head_dim=c.head_dim, qk_norm=norm, position=PartRef("position", "rope", theta=c.rope_theta))
    ffn = PartRef("ffn", "swiglu", inter=c.intermediate_size)
    layer = LayerSpec(block=PartRef("block", "prenorm"), mixer=mixer, ffn=ffn, norm=norm)
    return ModelSpec(
        hidden=c.hidden_size, vocab=c.vocab_size, layers=(layer,) * c.num_hidden_layers,
        order=in_order(c.num_hidden_layers), embed=PartRef("embed", "table"), norm=norm,
        head=PartRef("head", "linear", tied=c.tie_word_embeddings), rules=HF_RULES,
        skip=("lm_head.",) if c.tie_word_embeddings else (),
        trained_context=c.max_position_embeddings, eos_token_ids=c.eos_token_ids)


register_architecture("Qwen3ForCausalLM", Qwen3Config, recipe)
