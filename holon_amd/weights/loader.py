"""Weights from safetensors files, by tensor name.

Every `*.safetensors` of the folder is read, in file-name order; a name in two files is an error
(std/holon_std/weights/hf/source.py:84-99). Names are mapped to parameter paths by the spec's rules, tried in order
(core/holon/core/build.py:317-337). Before any tensor is read, names and shapes are checked against what the model
declares, and one error lists every missing tensor, every unexpected one and every wrong shape. Then each tensor is
read, moved to the device in its parameter's dtype and handed to its part; parts then finalise (merge projections),
children first (core/holon/core/build.py:372-424).
"""
from __future__ import annotations

import pathlib
import re

import torch
from safetensors import safe_open

from ..parts.base import FLOAT32, INT32, MODEL, ParamDecl, Part
from ..spec import ModelSpec, WeightRule


class WeightError(ValueError):
    """The checkpoint does not fit the model; `missing`, `unexpected` and `wrong_shape` say how."""

    def __init__(self, missing: list[str], unexpected: list[str], wrong_shape: list[tuple[str, tuple, tuple]],
                 other: list[str] = ()) -> None:
        self.missing, self.unexpected, self.wrong_shape, self.other = missing, unexpected, wrong_shape, list(other)
        lines = ["the checkpoint does not fit the model:"]
        if missing:
            lines.append(f"  missing tensors ({len(missing)}): " + ", ".join(missing))
        if unexpected:
            lines.append(f"  unexpected tensors ({len(unexpected)}): " + ", ".join(unexpected))
        if wrong_shape:
            lines.append(f"  wrong shapes ({len(wrong_shape)}): " + ", ".join(
                f"{n} is {list(got)}, the model needs {list(want)}" for n, got, want in wrong_shape))
        lines += [f"  {o}" for o in self.other]
        super().__init__("\n".join(lines))


def map_name(rules: tuple[WeightRule, ...], name: str, compiled: list[re.Pattern] | None = None) -> str | None:
    """The parameter path of checkpoint tensor `name`, or None when no rule matches."""
    for rule, pattern in zip(rules, compiled or [r.compile() for r in rules]):
        m = pattern.match(name)
        if m:
            return rule.target.format(**m.groupdict())
    return None


def unmap_name(rules: tuple[WeightRule, ...], path: str) -> str | None:
    """The checkpoint name that maps to parameter path `path` (the rules run backwards)."""
    for rule in rules:
        m = WeightRule(rule.target, rule.pattern).compile().match(path)
        if m:
            name = rule.pattern.format(**m.groupdict())
            if map_name(rules, name) == path:
                return name
    return None


def param_dtype(decl: ParamDecl, dtype: torch.dtype) -> torch.dtype:
    return {MODEL: dtype, FLOAT32: torch.float32, INT32: torch.int32}[decl.kind]


def tensor_files(folder: str | pathlib.Path) -> list[pathlib.Path]:
    files = sorted(pathlib.Path(folder).glob("*.safetensors"))
    if not files:
        raise FileNotFoundError(f"{folder}: no *.safetensors file")
    return files


def load_weights(model: Part, spec: ModelSpec, folder: str | pathlib.Path, device: torch.device,
                 dtype: torch.dtype) -> None:
    params = {path: (owner, attr, decl) for path, owner, attr, decl in model.named_params()}
    compiled = [r.compile() for r in spec.rules]
    where: dict[str, tuple[pathlib.Path, str]] = {}          # parameter path -> (file, tensor name)
    seen: dict[str, pathlib.Path] = {}
    missing, unexpected, wrong, other = [], [], [], []
    files = tensor_files(folder)
    for file in files:
        with safe_open(str(file), "pt", device="cpu") as f:
            for name in f.keys():
                if name in seen:
                    other.append(f"tensor {name} is in both {seen[name].name} and {file.name}")
                    continue
                seen[name] = file
                if any(name.startswith(p) for p in spec.skip):
                    continue
                path = map_name(spec.rules, name, compiled)
                if path is None or path not in params:
                    unexpected.append(name)
                    continue
                if path in where:
                    other.append(f"tensors {where[path][1]} and {name} both fill {path}")
                    continue
                got, want = tuple(f.get_slice(name).get_shape()), params[path][2].shape
                if got != want:
                    wrong.append((name, got, want))
                where[path] = (file, name)
    for path in params:
        if path not in where:
            missing.append(unmap_name(spec.rules, path) or path)
    if missing or unexpected or wrong or other:
        raise WeightError(sorted(missing), sorted(unexpected), sorted(wrong), other)
    by_file: dict[pathlib.Path, list[str]] = {}
    for path, (file, _) in where.items():
        by_file.setdefault(file, []).append(path)
    for file in files:
        with safe_open(str(file), "pt", device="cpu") as f:
            for path in by_file.get(file, []):
                owner, attr, decl = params[path]
                tensor = f.get_tensor(where[path][1])
                setattr(owner, attr, tensor.to(device=device, dtype=param_dtype(decl, dtype)).contiguous())
    finalize(model)


def finalize(model: Part) -> None:
    for part in model.walk():
        part.finalize()
