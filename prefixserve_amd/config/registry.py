"""One registry from an architecture's name to its configuration class and model builder.

``config.json["architectures"][0]`` picks the entry; the entry's configuration class
parses the architecture's own keys and its builder turns the typed configuration into a
``ModelSpec``. An unknown name is an error that lists what is registered.
"""

from __future__ import annotations

import json
from dataclasses import dataclass
from pathlib import Path
from typing import Any, Callable, Mapping

from prefixserve_amd.parts.spec import ModelSpec


@dataclass(frozen=True)
class Architecture:
    name: str
    config_cls: Any                              # needs from_dicts(raw, gen) -> config
    build_spec: Callable[[Any], ModelSpec]


_ARCHITECTURES: dict[str, Architecture] = {}


class UnknownArchitectureError(ValueError):
    pass


def register_architecture(name: str, config_cls: Any, build_spec: Callable[[Any], ModelSpec]) -> None:
    if name in _ARCHITECTURES:
        raise ValueError(f"architecture {name!r} is already registered")
    _ARCHITECTURES[name] = Architecture(name, config_cls, build_spec)


def registered_architectures() -> list[str]:
    return sorted(_ARCHITECTURES)


def architecture_of(raw: Mapping[str, Any]) -> Architecture:
    archs = raw.get("architectures")
    if not archs or not isinstance(archs, list):
        raise UnknownArchitectureError(
            f"config.json has no 'architectures' entry; registered: {registered_architectures()}")
    name = archs[0]
    if name not in _ARCHITECTURES:
        raise UnknownArchitectureError(
            f"architecture {name!r} is not registered; registered: {registered_architectures()}")
    return _ARCHITECTURES[name]


def read_model_dir(model_dir: str | Path) -> tuple[Architecture, Any, dict[str, Any]]:
    """(architecture entry, typed configuration, raw config.json) of a model folder."""
    model_dir = Path(model_dir)
    cfg_path = model_dir / "config.json"
    if not cfg_path.exists():
        raise FileNotFoundError(f"{cfg_path} not found")
    raw = json.loads(cfg_path.read_text())
    gen_path = model_dir / "generation_config.json"
    gen = json.loads(gen_path.read_text()) if gen_path.exists() else {}
    arch = architecture_of(raw)
    return arch, arch.config_cls.from_dicts(raw, gen), raw
