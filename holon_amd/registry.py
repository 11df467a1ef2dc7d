"""One registry from names to what builds them: architectures (config.json's `architectures[0]` to a configuration
class and a recipe) and parts by family. A name is registered once; asking for an unknown one lists what exists
(core/holon/core/plugins.py:31-122: duplicates and unknown names are errors)."""
from __future__ import annotations

import dataclasses
from collections.abc import Callable, Mapping
from typing import Any

from .spec import ModelSpec, PartRef

FAMILIES = ("mixer", "ffn", "norm", "position", "block", "embed", "head")     # the built-in parts' families


class RegistryError(KeyError):
    def __str__(self) -> str:                    # KeyError quotes its message
        return str(self.args[0])


@dataclasses.dataclass(frozen=True)
class Architecture:
    name: str
    config: Any                                  # a class with from_dict(config.json, generation_config.json)
    recipe: Callable[[Any], ModelSpec]


_ARCHITECTURES: dict[str, Architecture] = {}
_PARTS: dict[str, dict[str, type]] = {f: {} for f in FAMILIES}


def register_architecture(name: str, config: Any, recipe: Callable[[Any], ModelSpec]) -> None:
    if name in _ARCHITECTURES:
        raise RegistryError(f"architecture {name!r} is registered twice")
    _ARCHITECTURES[name] = Architecture(name, config, recipe)


def unregister_architecture(name: str) -> None:
    _ARCHITECTURES.pop(name, None)


def architecture(name: str) -> Architecture:
    _load_builtin()
    if name not in _ARCHITECTURES:
        raise RegistryError(f"no model for architecture {name!r}; registered: {sorted(_ARCHITECTURES)}")
    return _ARCHITECTURES[name]


def architectures() -> list[str]:
    _load_builtin()
    return sorted(_ARCHITECTURES)


def resolve(config_json: Mapping[str, Any], generation: Mapping[str, Any] | None = None) -> tuple[Any, ModelSpec]:
    """config.json to (typed configuration, model spec), by `architectures[0]`
    (core/holon/core/assembly.py:28-31)."""
    names = config_json.get("architectures")
    if not names:
        raise RegistryError("config.json has no `architectures`")
    arch = architecture(names[0])
    cfg = arch.config.from_dict(config_json, generation)
    return cfg, arch.recipe(cfg)


def register_part(family: str, kind: str) -> Callable[[type], type]:
    """Class decorator: `@register_part("mixer", "gqa")`. A family is any name: the first part of a new one (a
    router, another kind of state) opens it."""
    if not family or not isinstance(family, str):
        raise RegistryError(f"a part family is a name, not {family!r}")

    def add(cls: type) -> type:
        kinds = _PARTS.setdefault(family, {})
        if kind in kinds:
            raise RegistryError(f"{family} {kind!r} is registered twice")
        kinds[kind] = cls
        return cls
    return add


def unregister_part(family: str, kind: str) -> None:
    _PARTS.get(family, {}).pop(kind, None)
    if family not in FAMILIES and not _PARTS.get(family, True):
        del _PARTS[family]


def part_class(ref: PartRef) -> type:
    _load_builtin()
    if ref.family not in _PARTS or ref.kind not in _PARTS[ref.family]:
        raise RegistryError(f"no {ref.family} named {ref.kind!r}; registered: {sorted(_PARTS.get(ref.family, {}))}"
                            + ("" if ref.family in _PARTS else f" (families: {sorted(_PARTS)})"))
    return _PARTS[ref.family][ref.kind]


_loaded = False


def _load_builtin() -> None:
    global _loaded
    if not _loaded:
        _loaded = True
        from . import models, parts               # noqa: F401  (their import registers them)
