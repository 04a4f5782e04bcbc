"""From a model folder (or a configuration and a weight source) to a model, by way of the registry."""
from __future__ import annotations

from typing import Any, Dict, Optional

from ..config.registry import load_config, lookup_architecture
from ..weights.store import SafetensorsSource
from .causal_lm import CausalLM


def build_model(config: Any, source: Any, mode: str = "bfloat16", device: Any = "cuda:0", strict: bool = False,
                options: Optional[Dict[str, Any]] = None):
    """The model that ``config``'s architecture registered, with weights from ``source``."""
    entry = lookup_architecture(config.architecture)
    if entry.build_model is not None:
        return entry.build_model(config, source, mode=mode, device=device, strict=strict, options=options)
    return CausalLM(config.model_spec(), source, mode=mode, device=device, strict=strict, options=options)


def load_model(model_dir: str, mode: str = "bfloat16", device: Any = "cuda:0", strict: bool = False,
               options: Optional[Dict[str, Any]] = None, config_overrides: Optional[Dict[str, Any]] = None):
    """config.json chooses the class; every *.safetensors file of the folder supplies the weights.

    ``config_overrides`` sets fields of the configuration that are options of the engine rather than keys of
    config.json (such as Qwen3's ``rope_pairing``); the configuration is validated again afterwards.  ``strict``:
    a tensor in the folder that no part of the model asked for is an error instead of a warning."""
    config = load_config(model_dir)
    config.apply_overrides(config_overrides, model_dir)
    return config, build_model(config, SafetensorsSource(model_dir), mode=mode, device=device, strict=strict,
                               options=options)
