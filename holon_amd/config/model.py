"""What every architecture's typed configuration shares: reading a model folder's config.json, the error a bad one
raises, and the end-of-sequence ids. The typed configuration of an architecture lives beside its recipe, under
`holon_amd/models/`: every size and constant of a model comes from there, and no code below holds one.
"""
from __future__ import annotations

import json
import pathlib
from collections.abc import Mapping
from typing import Any


class ConfigError(ValueError):
    """config.json is missing a key, or asks for something this architecture does not do."""


def eos_ids(*sources: Mapping[str, Any] | None) -> tuple[int, ...]:
    """The union of `eos_token_id` (an int or a list) over config.json and generation_config.json
    (std/holon_std/weights/hf/source.py:62-66)."""
    out: list[int] = []
    for src in sources:
        value = (src or {}).get("eos_token_id")
        for token in ([] if value is None else value if isinstance(value, list) else [value]):
            if token not in out:
                out.append(int(token))
    return tuple(out)


def read_config_json(folder: str | pathlib.Path) -> tuple[dict[str, Any], dict[str, Any] | None]:
    """config.json (required) and generation_config.json (optional) of a model folder, as dicts."""
    folder = pathlib.Path(folder)
    path = folder / "config.json"
    if not path.is_file():
        raise FileNotFoundError(f"{folder}: no config.json")
    gen = folder / "generation_config.json"
    return json.loads(path.read_text()), (json.loads(gen.read_text()) if gen.is_file() else None)
