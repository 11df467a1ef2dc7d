"""Qwen3 dense: configuration to spec. plugins/holon_plugins/models/qwen3/recipe.py:10-59.

Pre-norm decoder; grouped-query attention with an RMSNorm over head_dim on q and k before the rotary embedding;
SwiGLU feed-forward; the head may be tied to the embedding."""
from __future__ import annotations

from ..config.model import Qwen3Config
from ..registry import register_architecture
from ..spec import LayerSpec, ModelSpec, PartRef, WeightRule, in_order

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
