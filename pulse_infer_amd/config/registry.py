"""One registry from an architecture's name to its configuration class and model.

The name is ``architectures[0]`` of config.json.  An entry holds the class that
reads the configuration and a builder that turns (configuration, weights,
options) into a model.  The default builder makes the generic ``CausalLM``
from the configuration's ``model_spec()``.  (The reference constructs its one
model directly, demo/qwen3_infer.cpp:596-611; the registry is this engine's.)
"""
from __future__ import annotations

import os
from dataclasses import dataclass
from typing import Any, Callable, Dict, Optional

from .base import ConfigError, architecture_name, read_json_file, resolve_model_dir


@dataclass
class ArchitectureEntry:
    name: str
    config_class: Any
    build_model: Optional[Callable[..., Any]] = None  # (config, weights, **options) -> model


_ARCHITECTURES: Dict[str, ArchitectureEntry] = {}


def register_architecture(name: str, config_class: Any, build_model: Optional[Callable[..., Any]] = None,
                          replace: bool = False) -> ArchitectureEntry:
    if name in _ARCHITECTURES and not replace:
        raise ValueError(f"architecture '{name}' is already registered")
    entry = ArchitectureEntry(name, config_class, build_model)
    _ARCHITECTURES[name] = entry
    return entry


def unregister_architecture(name: str) -> None:
    _ARCHITECTURES.pop(name, None)


def registered_architectures() -> list:
    return sorted(_ARCHITECTURES)


def lookup_architecture(name: str) -> ArchitectureEntry:
    try:
        return _ARCHITECTURES[name]
    except KeyError:
        known = ", ".join(registered_architectures()) or "<none>"
        raise ConfigError(f"unknown architecture '{name}'; registered: {known}") from None


def load_config(path: str):
    """Read config.json of a model folder with the class its architecture registered."""
    model_dir = resolve_model_dir(path)
    config_path = os.path.join(model_dir, "config.json")
    data = read_json_file(config_path)
    entry = lookup_architecture(architecture_name(data, config_path))
    return entry.config_class.load(model_dir)


def config_from_dict(data: Dict[str, Any], origin: str = "<dict>"):
    entry = lookup_architecture(architecture_name(data, origin))
    return entry.config_class.from_dict(data, origin)
