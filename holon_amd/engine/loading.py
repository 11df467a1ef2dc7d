"""From a model folder to a model on the device, with its cache and step function."""
from __future__ import annotations

import dataclasses
import pathlib

import torch

from ..cache.manager import CacheManager
from ..config.model import read_config_json
from ..model import Model, build_model
from ..parts.base import Build
from ..registry import resolve
from ..spec import ModelSpec
from ..weights.loader import load_weights
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


def load_model(folder: str | pathlib.Path, *, device: str | torch.device = "cuda", dtype: str | torch.dtype = "bfloat16",
               kernels=None, page_size: int = 16, max_seqs: int = 64, max_model_len: int = 8192,
               max_step_tokens: int = 4096, cache_tokens: int | None = None, graphs: bool = False) -> Loaded:
    """Read config.json, pick the model by its architecture name, load the weights, allocate the cache."""
    device, dtype = torch.device(device), torch_dtype(dtype)
    kernels = kernels if kernels is not None else default_kernels(device)
    config_json, generation = read_config_json(folder)
    cfg, spec = resolve(config_json, generation)
    model, _ = build_from_spec(spec, device=device, dtype=dtype, kernels=kernels, page_size=page_size,
                               max_seqs=max_seqs, max_model_len=max_model_len, max_step_tokens=max_step_tokens)
    load_weights(model, spec, folder, device, dtype)
    tokens = cache_tokens if cache_tokens is not None else max_model_len
    cache, runner = attach_cache(model, device=device, dtype=dtype, kernels=kernels, page_size=page_size,
                                 max_seqs=max_seqs, max_model_len=max_model_len, max_step_tokens=max_step_tokens,
                                 cache_tokens=tokens, graphs=graphs)
    return Loaded(cfg, spec, model, cache, runner, kernels, device, dtype)
