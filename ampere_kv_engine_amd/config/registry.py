"""The one registry from an architecture's name (config.json `architectures[0]`) to its typed configuration.

An entry is a configuration class with `from_folder(folder)` and `to_model_spec()`.  The model itself is
always assembled from the `ModelSpec` by the part registries, so registering an architecture means
registering how its config.json reads, nothing else.
"""

from __future__ import annotations

import json
import os
from typing import Protocol

from .qwen3 import ConfigError, Qwen3Config
from .specs import ModelSpec


class ArchitectureConfig(Protocol):
    architecture: str

    @classmethod
    def from_folder(cls, folder: str) -> "ArchitectureConfig": ...

    def to_model_spec(self) -> ModelSpec: ...


_ARCHITECTURES: dict[str, type] = {}


def register_architecture(name: str, config_class: type, *, replace: bool = False) -> None:
    if name in _ARCHITECTURES and not replace:
        raise ValueError(f"architecture {name!r} is already registered")
    _ARCHITECTURES[name] = config_class


def known_architectures() -> tuple[str, ...]:
    return tuple(sorted(_ARCHITECTURES))


def architecture_of(folder: str) -> str:
    path = os.path.join(folder, "config.json")
    if not os.path.exists(path):
        raise ConfigError(f"{folder} holds no config.json")
    with open(path) as handle:
        raw = json.load(handle)
    names = raw.get("architectures")
    if not isinstance(names, list) or len(names) != 1 or not isinstance(names[0], str):
        raise ConfigError(f"config.json key architectures must be a list with one name, got {names!r}")
    return names[0]


def load_config(folder: str) -> ArchitectureConfig:
    """Read the folder's config.json with the configuration class its `architectures` entry names."""
    name = architecture_of(folder)
    if name not in _ARCHITECTURES:
        raise ConfigError(f"architecture {name!r} is not registered; known: {', '.join(known_architectures())}")
    return _ARCHITECTURES[name].from_folder(folder)


register_architecture(Qwen3Config.architecture, Qwen3Config)
