"""Engine settings and per-request sampling parameters: plain dataclasses, no torch.

Field names, defaults and meanings follow the reference's `EngineConfig` (core/holon/core/engine.py:61-100) and
`SamplingParams` (core/holon/api/batch.py:45-61) where this engine has the feature; the command line makes one flag
per field from the help lines, as the reference's does (core/holon/core/cli.py:52-80).
"""
from __future__ import annotations

import dataclasses
from typing import Any

DTYPES = ("bfloat16", "float32")


def _setting(default: object, help: str) -> Any:
    return dataclasses.field(default=default, metadata={"help": help})


@dataclasses.dataclass
class EngineConfig:
    model: str = dataclasses.field(metadata={"help": "model folder (config.json and *.safetensors)"})
    device: str = _setting("cuda", "torch device to serve on")
    dtype: str = _setting("bfloat16", "activation, weight and cache dtype: bfloat16, or float32 (every product, sum "
                                      "and stored value in true 32-bit)")
    page_size: int = _setting(16, "tokens per page of paged state")
    max_seqs: int = _setting(64, "sequences served at once")
    max_model_len: int = _setting(8192, "prompt + generated tokens per request; pools always hold one")
    max_step_tokens: int = _setting(4096, "tokens one step computes at most")
    chunk_with_decode: int = _setting(0, "prefill tokens a step with decode rows may also carry (0: none)")
    memory_fraction: float = _setting(0.9, "of the memory left after weights, for activations and state")
    state_memory: int | None = _setting(None, "bytes for state pools; default: from memory_fraction")
    cache_tokens: int | None = _setting(None, "tokens of paged state per pool (overrides state_memory)")
    prefix_cache: bool = _setting(True, "reuse cached prompt blocks across requests")
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
        for name in ("page_size", "max_seqs", "max_model_len", "max_step_tokens"):
            if getattr(self, name) < 1:
                raise ValueError(f"EngineConfig.{name} must be >= 1")
        if self.chunk_with_decode < 0:
            raise ValueError("EngineConfig.chunk_with_decode must be >= 0")
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
