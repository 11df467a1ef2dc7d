"""Random weights from a configuration and a seed: written as a model folder, or put straight into a built model.

Each tensor is drawn from its own generator, seeded by (seed, checkpoint tensor name), so the values do not depend on
the order of creation. Projections and the embedding are N(0, 0.02); norm weights are 1 + N(0, 0.1). Values are
rounded to bfloat16 before they are stored, so the 32-bit and the bfloat16 model of one folder hold the same numbers.
"""
from __future__ import annotations

import dataclasses
import hashlib
import json
import pathlib
from typing import Any

import torch
from safetensors.torch import save_file

from ..parts.base import INT32, Build, ParamDecl
from ..registry import resolve
from .loader import checkpoint_names, finalize, param_dtype

LINEAR_STD, NORM_STD = 0.02, 0.1


def tensor_seed(seed: int, name: str) -> int:
    return int.from_bytes(hashlib.sha256(f"{seed}:{name}".encode()).digest()[:8], "little") & (2 ** 63 - 1)


def random_tensor(name: str, decl: ParamDecl, seed: int, device: torch.device | str = "cpu") -> torch.Tensor:
    """float32 values (bfloat16-representable) of tensor `name`."""
    if decl.kind == INT32:
        raise NotImplementedError(f"{name}: no rule to draw an integer table")
    g = torch.Generator(device=device).manual_seed(tensor_seed(seed, name))
    x = torch.randn(decl.shape, generator=g, device=device, dtype=torch.float32)
    x = 1 + NORM_STD * x if decl.init == "norm" else LINEAR_STD * x
    return x.bfloat16().float()


def meta_model(config_json: dict[str, Any]):
    """(typed configuration, spec, the model built without storage): what tensors a configuration has."""
    from ..model import build_model
    cfg, spec = resolve(config_json)
    build = Build(kernels=None, device=torch.device("meta"), dtype=torch.float32, max_model_len=2)
    return cfg, spec, build_model(spec, build)


def write_random_model(config_json: dict[str, Any], seed: int, folder: str | pathlib.Path,
                       store_dtype: torch.dtype = torch.bfloat16) -> pathlib.Path:
    """A model folder (config.json, model.safetensors) for `config_json`, every tensor under its checkpoint name."""
    cfg, spec, model = meta_model(config_json)
    folder = pathlib.Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    tensors = {}
    for path, _, _, decl in model.named_params():
        names = checkpoint_names(spec.rules, path, decl.shape)
        if not names:
            raise ValueError(f"no weight rule names parameter {path}")
        for name, index in names:                 # a stacked parameter is stored as one tensor per slice
            one = decl if index is None else dataclasses.replace(decl, shape=decl.shape[1:])
            tensors[name] = random_tensor(name, one, seed).to(torch.int32 if decl.kind == INT32 else store_dtype)
    (folder / "config.json").write_text(json.dumps(cfg.to_dict(), indent=1) + "\n")
    save_file(tensors, str(folder / "model.safetensors"), metadata={"format": "pt", "seed": str(seed)})
    return folder


def fill_random(model, spec, seed: int, device: torch.device, dtype: torch.dtype) -> None:
    """Random weights drawn on the device into a built model (no folder): for measurements at sizes whose folder would
    take minutes to write. The values differ from `write_random_model`'s (another generator), the law is the same."""
    for path, owner, attr, decl in model.named_params():
        names = checkpoint_names(spec.rules, path, decl.shape) or [(path, None)]
        if names[0][1] is None:
            value = random_tensor(names[0][0], decl, seed, device)
        else:
            one = dataclasses.replace(decl, shape=decl.shape[1:])
            value = torch.stack([random_tensor(name, one, seed, device) for name, _ in names])
        setattr(owner, attr, value.to(param_dtype(decl, dtype)))
    finalize(model)
