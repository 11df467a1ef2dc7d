"""From a model folder to a model on the device, with its cache and step function."""
from __future__ import annotations

import dataclasses
import pathlib

import torch

from ..cache.manager import CacheManager
from ..config.engine import EngineConfig
from ..config.model import read_config_json
from ..model import Model, build_model
from ..parts.base import Build
from ..registry import resolve
from ..spec import ModelSpec
from ..weights.loader import load_weights
from ..weights.random_init import fill_random
from .step import StepRunner

TORCH_DTYPES = {"bfloat16": torch.bfloat16, "float32": torch.float32}


def torch_dtype(name: str | torch.dtype) -> torch.dtype:
    if isinstance(name, torch.dtype):
        if name not in TORCH_DTYPES.values():
            raise ValueError(f"dtype must be bfloat16 or float32, got {name}")
        return name
    if name not in TORCH_DTYPES:
        raise ValueError(f"dtype must be one of {sorted(TORCH_DTYPES)}, got {name!r}")
    return TORCH_DTYPES[name]


def default_kernels(device: torch.device):
    """The HIP kernels. There is no other implementation to fall back to: a device that is not a GPU, or a missing
    library that cannot be built, is an error."""
    if device.type != "cuda":
        raise RuntimeError(f"holon_amd runs on an AMD GPU ('cuda' device of PyTorch-ROCm), not on {device}; "
                           "there is no CPU path")
    from ..kernels import load_hip
    return load_hip()


@dataclasses.dataclass
class Loaded:
    config: object
    spec: ModelSpec
    model: Model
    cache: CacheManager
    runner: StepRunner
    kernels: object
    device: torch.device
    dtype: torch.dtype


def build_from_spec(spec: ModelSpec, *, device: torch.device, dtype: torch.dtype, kernels, page_size: int,
                    max_seqs: int, max_model_len: int, max_step_tokens: int, decode_copy: bool = True
                    ) -> tuple[Model, Build]:
    build = Build(kernels=kernels, device=device, dtype=dtype, page_size=page_size, max_model_len=max_model_len,
                  max_seqs=max_seqs, max_step_tokens=max_step_tokens, decode_copy=decode_copy)
    return build_model(spec, build), build


def attach_cache(model: Model, *, device: torch.device, dtype: torch.dtype, kernels, page_size: int, max_seqs: int,
                 max_model_len: int, max_step_tokens: int, cache_tokens: int, graphs: bool = False
                 ) -> tuple[CacheManager, StepRunner]:
    cache = CacheManager(model.sites, model.state_decls(), page_size=page_size, max_seqs=max_seqs,
                         max_model_len=max_model_len, tokens=cache_tokens, device=device, dtype=dtype)
    runner = StepRunner(model, cache, kernels, device, max_step_tokens=max_step_tokens, max_seqs=max_seqs,
                        graphs=graphs)
    return cache, runner


@dataclasses.dataclass
class Assembled:
    """A model with its weights on the device and its kernels configured; no cache yet."""

    config: object
    spec: ModelSpec
    model: Model
    kernels: object
    device: torch.device
    dtype: torch.dtype

    def shape(self, cfg: EngineConfig) -> dict:
        return dict(device=self.device, dtype=self.dtype, kernels=self.kernels, page_size=cfg.page_size,
                    max_seqs=cfg.max_seqs, max_model_len=cfg.max_model_len, max_step_tokens=cfg.max_step_tokens)


def assemble(cfg: EngineConfig, kernels=None, *, random_config: dict | None = None, seed: int = 0) -> Assembled:
    """From the engine's settings to a model ready to step: the kernels with this engine's product choices, the
    architecture by config.json's name, the parts, the weights (from the folder, or random ones drawn on the device
    from `random_config`), and, in mode `timed`, the product choices timed now. The one place a model is put together:
    `Engine` and `load_model` both call it."""
    device, dtype = torch.device(cfg.device), torch_dtype(cfg.dtype)
    kernels = kernels if kernels is not None else default_kernels(device)
    configured = getattr(kernels, "configured", None)      # a kernel set with one form a product has nothing to choose
    if configured is not None:
        kernels = configured(cfg.products, cfg.product_pins)
    config_json, generation = (random_config, None) if random_config is not None else read_config_json(cfg.model)
    model_config, spec = resolve(config_json, generation)
    model, _ = build_from_spec(spec, device=device, dtype=dtype, kernels=kernels, page_size=cfg.page_size,
                               max_seqs=cfg.max_seqs, max_model_len=cfg.max_model_len,
                               max_step_tokens=cfg.max_step_tokens, decode_copy=cfg.decode_weight_copy)
    if random_config is not None:
        fill_random(model, spec, seed, device, dtype)
    else:
        load_weights(model, spec, cfg.model, device, dtype)
    out = Assembled(model_config, spec, model, kernels, device, dtype)
    time_products(out, cfg)
    return out


TIMED_ROWS = (32, 64, 128, 256, 512, 768, 1024)       # one step in each row bucket a product choice is kept for


def time_products(a: Assembled, cfg: EngineConfig) -> None:
    """Mode `timed`: run one step in every row bucket this engine can reach, on a cache just large enough, with the
    kernels allowed to time their candidates; afterwards every choice is fixed and no request ever pays for one."""
    plan = getattr(a.kernels, "plan", None)
    if plan is None or plan.mode != "timed" or a.device.type != "cuda" or a.dtype != torch.bfloat16:
        return
    import sys
    import time

    from .batch import StepRow
    t0 = time.perf_counter()
    longest = max(1, cfg.max_model_len - 1)
    plan.resolving = True
    try:
        for bucket in TIMED_ROWS:
            if bucket > cfg.max_step_tokens:
                break
            per_row = min(bucket, longest)
            rows = bucket // per_row
            if rows > cfg.max_seqs:
                continue
            pages = rows * -(-(per_row + 1) // cfg.page_size) + 1
            cache, runner = attach_cache(a.model, cache_tokens=pages * cfg.page_size, graphs=False, **a.shape(cfg))
            slots = [cache.admit() for _ in range(rows)]
            for slot in slots:
                cache.reserve(slot, per_row)
            want = list(range(per_row)) if rows * per_row <= 64 else [per_row - 1]
            runner.run([StepRow(slot, 0, [0] * per_row, want) for slot in slots])
            torch.cuda.synchronize(a.device)
            del cache, runner
    finally:
        plan.resolving = False
        for site in a.model.sites:
            site.detach()
        torch.cuda.empty_cache()
    print(f"holon_amd: product choices timed in {time.perf_counter() - t0:.1f} s: "
          + (", ".join(f"{k}={v}" for k, v in plan.report().items()) or "nothing to choose"), file=sys.stderr)


def load_model(folder: str | pathlib.Path, *, device: str | torch.device = "cuda", dtype: str | torch.dtype = "bfloat16",
               kernels=None, page_size: int = 16, max_seqs: int = 64, max_model_len: int = 8192,
               max_step_tokens: int = 4096, cache_tokens: int | None = None, graphs: bool = False,
               products: str = "own", product_pins: dict | None = None, decode_weight_copy: bool = True,
               random_config: dict | None = None, seed: int = 0) -> Loaded:
    """Read config.json, pick the model by its architecture name, load the weights, allocate the cache. With
    `random_config` (a config.json as a dict) no folder is read: the weights are drawn on the device from `seed`."""
    dtype_name = dtype if isinstance(dtype, str) else {v: k for k, v in TORCH_DTYPES.items()}[torch_dtype(dtype)]
    cfg = EngineConfig(model=str(folder), device=str(device), dtype=dtype_name, page_size=page_size, max_seqs=max_seqs,
                       max_model_len=max_model_len, max_step_tokens=max_step_tokens, graphs=graphs, products=products,
                       product_pins=product_pins, decode_weight_copy=decode_weight_copy)
    a = assemble(cfg, kernels, random_config=random_config, seed=seed)
    tokens = cache_tokens if cache_tokens is not None else max_model_len
    cache, runner = attach_cache(a.model, cache_tokens=tokens, graphs=graphs, **a.shape(cfg))
    return Loaded(a.config, a.spec, a.model, cache, runner, a.kernels, a.device, a.dtype)
