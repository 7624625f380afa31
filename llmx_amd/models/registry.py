"""One registry from an architecture's name (config.json `architectures[0]`) to its typed configuration and its model.

An entry holds the configuration class (`from_json(dict)`, `to_json()`) and the function that turns a configuration
into a `ModelSpec`.  The lookup follows /root/reference/src/model/arch/registry.hpp:25-60: an unknown name is refused
by name.
"""

from __future__ import annotations

from dataclasses import dataclass
from pathlib import Path
from typing import Any, Callable, Dict

from ..config.reader import ConfigError, read_json
from ..parts.spec import ModelSpec


@dataclass(frozen=True)
class ArchitectureEntry:
    name: str
    config_class: Any
    assemble: Callable[[Any], ModelSpec]


_ARCHITECTURES: Dict[str, ArchitectureEntry] = {}


def register_architecture(name: str, config_class: Any, assemble: Callable[[Any], ModelSpec], replace: bool = False) -> None:
    if name in _ARCHITECTURES and not replace:
        raise ValueError(f"architecture {name!r} is already registered")
    _ARCHITECTURES[name] = ArchitectureEntry(name, config_class, assemble)


def unregister_architecture(name: str) -> None:
    _ARCHITECTURES.pop(name, None)


def architecture_of(name: str) -> ArchitectureEntry:
    if name not in _ARCHITECTURES:
        raise ConfigError(f"config: unsupported architecture {name!r} (this engine runs: {sorted(_ARCHITECTURES)})")
    return _ARCHITECTURES[name]


def architectures() -> list[str]:
    return sorted(_ARCHITECTURES)


def read_config(values: dict):
    """The typed configuration of a parsed config.json, its class chosen by `architectures`."""
    archs = values.get("architectures") if isinstance(values, dict) else None
    if not isinstance(archs, list) or len(archs) != 1 or not isinstance(archs[0], str):
        raise ConfigError("config: missing key architectures" if not archs else f"config: unsupported value for architectures ({archs!r})")
    return architecture_of(archs[0]).config_class.from_json(values)


def read_model_dir(path: str | Path):
    """(configuration, ModelSpec) of the model folder `path` (config.json decides the class)."""
    cfg = read_config(read_json(Path(path) / "config.json"))
    return cfg, assemble(cfg)


def assemble(cfg) -> ModelSpec:
    spec = architecture_of(cfg.architecture).assemble(cfg)
    spec.check()
    return spec
