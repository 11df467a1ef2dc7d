"""Engine settings and per-request sampling parameters: plain dataclasses, no torch.

Field names, defaults and meanings follow the reference's `EngineConfig` (core/holon/core/engine.py:61-100) and
`SamplingParams` (core/holon/api/batch.py:45-61) where this engine has the feature; the command line makes one flag
per field from the help lines, as the reference's does (core/holon/core/cli.py:52-80).
"""
from __future__ import annotations

import dataclasses
from typing import Any

DTYPES = ("bfloat16", "float32")


def _setting(default: object, text: str) -> Any:
    """A field with the line the command line shows for it."""
    return dataclasses.field(default=default, metadata={"help": text})


@dataclasses.dataclass
class EngineConfig:
    model: str = dataclasses.field(metadata={"help": "model folder (config.json and *.safetensors)"})
    device: str = _setting("cuda", "the GPU the engine runs on, as torch names it")
    dtype: str = _setting("bfloat16", "activation, weight and cache dtype: bfloat16, or float32 (every product, sum "
                                      "and stored value in true 32-bit)")
    page_size: int = _setting(16, "how many tokens one cache page holds")
    max_seqs: int = _setting(64, "the most requests that run side by side (slots)")
    max_model_len: int = _setting(8192, "the longest a request may grow, prompt and generated tokens together; the cache is never smaller than one such request")
    max_step_tokens: int = _setting(4096, "the token budget of one step (prompt portions and decode rows together)")
    chunk_with_decode: int = _setting(0, "how many prompt tokens may ride along in a step that also decodes (0: such steps decode only)")
    memory_fraction: float = _setting(0.9, "the share of the GPU memory still free once the weights are loaded that steps and the cache may use")
    state_memory: int | None = _setting(None, "the cache's size in bytes, instead of deriving it from memory_fraction")
    cache_tokens: int | None = _setting(None, "tokens of paged state per pool (overrides state_memory)")
    prefix_cache: bool = _setting(True, "let a request start from the pages of an earlier request with the same first tokens")
    overlap: bool = _setting(True, "schedule and launch the next step while the last one runs")
    graphs: bool = _setting(True, "replay decode steps from HIP graphs, per batch-size bucket")
    decode_weight_copy: bool = _setting(True, "keep a second copy of every projection in the tile layout that steps of "
                                              "few rows stream fastest (doubles the weights' memory)")
    products: str = _setting("own", "which kernel a matrix product of 17 to 1,024 rows takes where several serve it: "
                                    "own (this package's wherever one serves), vendor (the vendor library's plain "
                                    "product), timed (candidates are timed once while the engine starts)")
    product_pins: dict | None = _setting(None, "single products pinned whatever the mode, as kind:NxK:rows=form,... "
                                               "(what stats()['products'] lists; on the command line a comma-"
                                               "separated list)")

    def __post_init__(self) -> None:
        too_small = [name for name, least in (("page_size", 1), ("max_seqs", 1), ("max_model_len", 1),
                                              ("max_step_tokens", 1), ("chunk_with_decode", 0))
                     if getattr(self, name) < least]
        if too_small:
            raise ValueError(f"EngineConfig: {', '.join(too_small)} below the least value allowed (0 for "
                             "chunk_with_decode, 1 for the others)")
        if self.dtype not in DTYPES:
            raise ValueError(f"EngineConfig.dtype must be one of {DTYPES}, got {self.dtype!r}")
        if self.chunk_with_decode and self.max_step_tokens < self.max_seqs + self.chunk_with_decode:
            raise ValueError("mixed steps need max_step_tokens >= max_seqs + chunk_with_decode")
        from .products import MODES, check_pins
        if self.products not in MODES:
            raise ValueError(f"EngineConfig.products must be one of {MODES}, got {self.products!r}")
        self.product_pins = check_pins(self.product_pins) or None


@dataclasses.dataclass
class SamplingParams:
    temperature: float = 1.0
    top_p: float = 1.0
    top_k: int = 0                       # 0: off
    min_p: float = 0.0
    presence_penalty: float = 0.0        # penalties are refused when set, as the reference refuses them
    frequency_penalty: float = 0.0
    repetition_penalty: float = 1.0
    n: int = 1                           # sequences drawn for the prompt; sequence i uses `sequence_seed(seed, i)`
    max_tokens: int | None = None
    ignore_eos: bool = False
    stop_token_ids: tuple[int, ...] = ()
    seed: int | None = None
    logprobs: int | None = None          # with every generated token: its log-probability and the k most likely (k <= 32)
    prompt_logprobs: int | None = None   # the same for the prompt's own tokens, each given the tokens before it
    ext: dict[str, Any] = dataclasses.field(default_factory=dict)   # a caller's own values; the engine reads none (core/holon/api/batch.py:61)

    def check(self) -> None:
        for name in ("logprobs", "prompt_logprobs"):
            if getattr(self, name) is not None and not 0 <= getattr(self, name) <= 32:
                raise ValueError(f"{name} must be between 0 and 32")
        if self.n < 1:
            raise ValueError(f"n must be >= 1, got {self.n}")
        if self.presence_penalty or self.frequency_penalty or self.repetition_penalty != 1:
            raise NotImplementedError("sampling penalties are not supported")
        if self.temperature < 0 or not 0 < self.top_p <= 1 or self.top_k < 0 or not 0 <= self.min_p <= 1:
            raise ValueError(f"sampling parameters out of range: {self}")
        if self.max_tokens is not None and self.max_tokens < 1:
            raise ValueError("max_tokens must be >= 1")

    @property
    def greedy(self) -> bool:
        return self.temperature == 0

    @property
    def filtered(self) -> bool:
        return self.top_k > 0 or self.top_p < 1 or self.min_p > 0
