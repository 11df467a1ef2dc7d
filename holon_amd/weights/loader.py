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


def locate(rules: tuple[WeightRule, ...], name: str, compiled: list[re.Pattern] | None = None
           ) -> tuple[str, int | None] | None:
    """Where checkpoint tensor `name` goes: (parameter path, slice of its first dimension or None for the whole
    parameter); None when no rule matches."""
    for rule, pattern in zip(rules, compiled or [r.compile() for r in rules]):
        m = pattern.match(name)
        if m:
            groups = m.groupdict()
            index = int(groups.pop(rule.stack)) if rule.stack is not None else None
            return rule.target.format(**groups), index
    return None


def map_name(rules: tuple[WeightRule, ...], name: str, compiled: list[re.Pattern] | None = None) -> str | None:
    """The parameter path of checkpoint tensor `name`, or None when no rule matches."""
    found = locate(rules, name, compiled)
    return found[0] if found is not None else None


def checkpoint_names(rules: tuple[WeightRule, ...], path: str, shape: tuple[int, ...]) -> list[tuple[str, int | None]]:
    """The checkpoint tensors that fill parameter `path` of `shape`, as (name, slice or None): the rules run
    backwards. One name for a whole parameter, one per slice for a stacked one; empty when no rule names it."""
    for rule in rules:
        m = WeightRule(rule.target, "").compile().match(path)
        if not m:
            continue
        slices = [None] if rule.stack is None else list(range(shape[0]))
        names = [(rule.pattern.format(**m.groupdict(), **({rule.stack: e} if e is not None else {})), e) for e in slices]
        if all(locate(rules, name) == (path, e) for name, e in names):
            return names
    return []


def unmap_name(rules: tuple[WeightRule, ...], path: str) -> str | None:
    """The checkpoint name that maps to the whole of parameter `path`, if one rule gives one."""
    for rule in rules:
        if rule.stack is None:
            names = checkpoint_names((rule,), path, ())
            if names and map_name(rules, names[0][0]) == path:
                return names[0][0]
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
    where: dict[tuple[str, int | None], tuple[pathlib.Path, str]] = {}      # (parameter path, slice) -> (file, name)
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
                found = locate(spec.rules, name, compiled)
                if found is None or found[0] not in params:
                    unexpected.append(name)
                    continue
                path, index = found
                want = params[path][2].shape
                if index is not None:             # one slice of a stacked parameter
                    if not want or index >= want[0]:
                        unexpected.append(name)
                        continue
                    want = want[1:]
                if found in where:
                    other.append(f"tensors {where[found][1]} and {name} both fill {path}")
                    continue
                got = tuple(f.get_slice(name).get_shape())
                if got != want:
                    wrong.append((name, got, want))
                where[found] = (file, name)
    stacked = {path for path, index in where if index is not None}
    for path, (_, _, decl) in params.items():
        if path in stacked:
            if (path, None) in where:
                other.append(f"{where[(path, None)][1]} fills {path} whole and other tensors fill slices of it")
            names = dict((e, n) for n, e in checkpoint_names(spec.rules, path, decl.shape))
            missing += [names.get(e, f"{path}[{e}]") for e in range(decl.shape[0]) if (path, e) not in where]
        elif (path, None) not in where:
            names = checkpoint_names(spec.rules, path, decl.shape)
            missing += [n for n, _ in names] or [path]
    if missing or unexpected or wrong or other:
        raise WeightError(sorted(missing), sorted(unexpected), sorted(wrong), other)
    by_file: dict[pathlib.Path, list[tuple[str, int | None]]] = {}
    for key, (file, _) in where.items():
        by_file.setdefault(file, []).append(key)
    for path in stacked:
        owner, attr, decl = params[path]
        setattr(owner, attr, torch.empty(decl.shape, dtype=param_dtype(decl, dtype), device=device))
    for file in files:
        with safe_open(str(file), "pt", device="cpu") as f:
            for path, index in by_file.get(file, []):
                owner, attr, decl = params[path]
                tensor = f.get_tensor(where[(path, index)][1]).to(device=device, dtype=param_dtype(decl, dtype))
                if index is None:
                    setattr(owner, attr, tensor.contiguous())
                else:
                    getattr(owner, attr)[index].copy_(tensor)
    finalize(model)


def finalize(model: Part) -> None:
    for part in model.walk():
        part.finalize()
