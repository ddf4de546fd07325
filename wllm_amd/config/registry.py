"""One registry from an architecture's name to everything that builds it.

The reference keeps a dict from config.json's `architectures` strings to model
classes and takes the first name it knows (src/wllm/models/registry.py:34-53).
Here an entry holds two callables instead of a class: one that reads the
architecture's own config.json keys into a typed configuration, and one that
turns that configuration into a `ModelPlan` (parts chosen layer by layer).  The
generic model in `wllm_amd.parts.model` is assembled from the plan, so adding
an architecture is one `register_architecture` call.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Any, Callable


class ConfigError(ValueError):
    """config.json is missing, malformed or describes a model that cannot be built."""


@dataclass(frozen=True)
class ArchitectureEntry:
    name: str
    parse_config: Callable[[dict], Any]
    build_plan: Callable[[Any], Any]


_REGISTRY: dict[str, ArchitectureEntry] = {}


def register_architecture(name: str, parse_config: Callable[[dict], Any],
                          build_plan: Callable[[Any], Any], *, replace: bool = False) -> ArchitectureEntry:
    if name in _REGISTRY and not replace:
        raise ConfigError(f"architecture {name!r} is already registered")
    entry = ArchitectureEntry(name, parse_config, build_plan)
    _REGISTRY[name] = entry
    return entry


def registered_architectures() -> list[str]:
    return sorted(_REGISTRY)


def resolve_architecture(architectures: list[str] | None) -> ArchitectureEntry:
    """First known name of config.json's `architectures` list wins
    (src/wllm/models/registry.py:41-53); an unknown list is an error that names
    what is supported."""
    for name in architectures or []:
        if name in _REGISTRY:
            return _REGISTRY[name]
    raise ConfigError(
        f"unsupported architecture(s) {list(architectures or [])!r}; "
        f"registered: {', '.join(registered_architectures()) or '(none)'}"
    )


def read_config_json(folder: str) -> dict:
    path = os.path.join(folder, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"no config.json in {folder!r}")
    try:
        with open(path, "r", encoding="utf-8") as f:
            raw = json.load(f)
    except json.JSONDecodeError as e:
        raise ConfigError(f"{path}: not valid JSON: {e}") from e
    if not isinstance(raw, dict):
        raise ConfigError(f"{path}: expected a JSON object")
    return raw
