"""Typed reading of a model folder's JSON configuration, and what the engine asks of a configuration.

``JsonReader`` fetches each key with a type check and produces errors that name the
file, the key and what was found, in the manner of the reference's ``read_required_*``
helpers (reference: src/model/qwen3/config.cpp:70-138).

``ModelConfig`` is the base of every architecture's configuration class.  The engine,
the command line and the loaders use nothing of a configuration beyond it:

* fields: ``architecture``, ``vocab_size``, ``eos_token_ids``, and the sampling defaults
  ``temperature``, ``top_k``, ``top_p``;
* ``from_dict(data, origin, generation, generation_origin)`` / ``load(folder)``: read and
  validate; ``to_dict()``: what ``config.json`` of a written model folder holds;
* ``validate(origin)``; ``apply_overrides({field: value})``: options of the engine that are
  no keys of config.json (the command line's ``--set field=value``);
* ``model_spec()``: the architecture as data (a ``ModelSpec``), which the generic model
  is built from.

An architecture brings a subclass with its own keys and registers it by name.
"""
from __future__ import annotations

import json
import os
from typing import Any, Dict, List, Mapping, Optional, Sequence


class ConfigError(ValueError):
    """A configuration file is missing, malformed, or describes something unsupported."""


_MISSING = object()


def resolve_model_dir(path: str) -> str:
    """A file path stands for its parent folder (reference: src/model/qwen3/config.cpp:38-44)."""
    path = os.fspath(path)
    if os.path.isfile(path):
        return os.path.dirname(os.path.abspath(path))
    return path


def strip_json_comments(text: str) -> str:
    """``text`` without // line comments and /* block comments */ outside strings (a comment becomes a blank)."""
    out: List[str] = []
    i, n = 0, len(text)
    in_string = False
    while i < n:
        c = text[i]
        if in_string:
            out.append(c)
            if c == "\\" and i + 1 < n:
                out.append(text[i + 1])
                i += 1
            elif c == '"':
                in_string = False
        elif c == '"':
            in_string = True
            out.append(c)
        elif c == "/" and text[i:i + 2] == "//":
            while i < n and text[i] != "\n":
                i += 1
            continue
        elif c == "/" and text[i:i + 2] == "/*":
            end = text.find("*/", i + 2)
            i = n if end < 0 else end + 2
            out.append(" ")
            continue
        else:
            out.append(c)
        i += 1
    return "".join(out)


def read_json_file(path: str) -> Dict[str, Any]:
    """A JSON object from a file; comments are allowed, as in the reference's reader
    (reference: src/model/qwen3/config.cpp:52 parses with ignore_comments)."""
    if not os.path.exists(path):
        raise ConfigError(f"there is no file '{path}'")
    try:
        with open(path, "r", encoding="utf-8") as fh:
            text = fh.read()
        try:
            data = json.loads(text)
        except json.JSONDecodeError:
            data = json.loads(strip_json_comments(text))
    except json.JSONDecodeError as exc:
        raise ConfigError(f"'{path}' is not valid JSON: {exc}") from exc
    if not isinstance(data, dict):
        raise ConfigError(f"'{path}' must hold a JSON object, found {type(data).__name__}")
    return data


class JsonReader:
    """Typed access to one JSON object; every error names the key and the file."""

    def __init__(self, data: Dict[str, Any], origin: str):
        self.data = data
        self.origin = origin

    def _fail(self, kind: str, key: str) -> ConfigError:
        if self.data.get(key) is None:
            return ConfigError(f"'{self.origin}': key '{key}' ({kind}) is required and missing")
        return ConfigError(f"'{self.origin}': key '{key}' must be {kind}, found {self.data[key]!r}")

    def has(self, key: str) -> bool:
        return key in self.data and self.data[key] is not None

    def raw(self, key: str, default: Any = None) -> Any:
        return self.data.get(key, default)

    def integer(self, key: str, default: Any = _MISSING) -> int:
        value = self.data.get(key, None)
        if value is None:
            if default is _MISSING:
                raise self._fail("an integer", key)
            return default
        if isinstance(value, bool) or not isinstance(value, int):
            if isinstance(value, float) and value.is_integer():
                return int(value)
            raise self._fail("an integer", key)
        return int(value)

    def number(self, key: str, default: Any = _MISSING) -> float:
        value = self.data.get(key, None)
        if value is None:
            if default is _MISSING:
                raise self._fail("a number", key)
            return default
        if isinstance(value, bool) or not isinstance(value, (int, float)):
            raise self._fail("a number", key)
        return float(value)

    def boolean(self, key: str, default: Any = _MISSING) -> bool:
        value = self.data.get(key, None)
        if value is None:
            if default is _MISSING:
                raise self._fail("true or false", key)
            return default
        if not isinstance(value, bool):
            raise self._fail("true or false", key)
        return value

    def string(self, key: str, default: Any = _MISSING) -> str:
        value = self.data.get(key, None)
        if value is None:
            if default is _MISSING:
                raise self._fail("a string", key)
            return default
        if not isinstance(value, str):
            raise self._fail("a string", key)
        return value

    def int_or_int_list(self, key: str) -> List[int]:
        """An integer or a list of integers; absent gives an empty list
        (reference: src/model/qwen3/config.cpp:160-206)."""
        value = self.data.get(key, None)
        if value is None:
            return []
        if isinstance(value, int) and not isinstance(value, bool):
            return [int(value)]
        if isinstance(value, list) and all(isinstance(v, int) and not isinstance(v, bool) for v in value):
            return [int(v) for v in value]
        raise self._fail("an integer or a list of integers", key)

    def string_list(self, key: str) -> Optional[List[str]]:
        value = self.data.get(key, None)
        if value is None:
            return None
        if isinstance(value, list) and all(isinstance(v, str) for v in value):
            return list(value)
        raise self._fail("a list of strings", key)


def require_positive(origin: str, **named: int) -> None:
    bad = [name for name, value in named.items() if value <= 0]
    if bad:
        raise ConfigError(f"'{origin}': these sizes must be positive: " + ", ".join(f"{name} = {named[name]}" for name in bad))


def architecture_name(data: Dict[str, Any], origin: str) -> str:
    archs = data.get("architectures")
    if not isinstance(archs, Sequence) or isinstance(archs, str) or len(archs) == 0 or not isinstance(archs[0], str):
        raise ConfigError(f"'{origin}': key 'architectures' must be a list that starts with the model's class name")
    return archs[0]


class ModelConfig:
    """Base of an architecture's configuration (see the module's text for what the engine uses of it).

    Subclasses are dataclasses with their own fields, among them ``vocab_size``, and set ``architecture``.  The
    sampling defaults and the end-of-sequence ids have defaults here, so an architecture that has no use for
    generation_config.json need not mention them."""

    architecture: str = ""
    # Fields that are options of the engine rather than keys of config.json, by field name: each becomes an option
    # of the command line (``--field-name``) with these argparse keywords (choices, type, help).  Every field can
    # also be set with ``--set field=value``.
    engine_options: Dict[str, Dict[str, Any]] = {}
    eos_token_ids: Sequence[int] = ()
    temperature: float = 0.0
    top_k: int = 0
    top_p: float = 0.0

    # ------------------------------------------------------------------ reading
    @classmethod
    def from_dict(cls, data: Dict[str, Any], origin: str = "<dict>", generation: Optional[Dict[str, Any]] = None,
                  generation_origin: str = "<dict>") -> "ModelConfig":
        raise NotImplementedError(f"{cls.__name__} must read its own keys in from_dict")

    @classmethod
    def load(cls, path: str) -> "ModelConfig":
        """config.json of the folder, and generation_config.json beside it if there is one."""
        model_dir = resolve_model_dir(path)
        config_path = os.path.join(model_dir, "config.json")
        data = read_json_file(config_path)
        gen_path = os.path.join(model_dir, "generation_config.json")
        generation = read_json_file(gen_path) if os.path.exists(gen_path) else None
        return cls.from_dict(data, config_path, generation, gen_path)

    def read_generation_defaults(self, generation: Optional[Dict[str, Any]], origin: str = "<dict>") -> None:
        """Sampling defaults and end-of-sequence ids from generation_config.json; its ids replace config.json's
        (reference: src/model/qwen3/config.cpp:333-365)."""
        if generation is None:
            return
        g = JsonReader(generation, origin)
        eos = g.int_or_int_list("eos_token_id")
        if eos:
            self.eos_token_ids = eos
        self.temperature = g.number("temperature", self.temperature)
        self.top_k = g.integer("top_k", self.top_k)
        self.top_p = g.number("top_p", self.top_p)

    # --------------------------------------------------------------- validation
    def validate(self, origin: str = "<config>") -> None:
        """Raise ``ConfigError`` for values the architecture cannot run with."""

    def apply_overrides(self, overrides: Optional[Mapping[str, Any]], origin: str = "<overrides>") -> None:
        """Set fields by name (options of the engine rather than keys of config.json) and validate again.  A name
        the configuration does not have, or a value of another type than the field's, is refused."""
        if not overrides:
            return
        for key, value in overrides.items():
            if key.startswith("_") or key == "engine_options" or not hasattr(self, key) or callable(getattr(self, key)):
                fields = sorted(k for k in vars(self) if not k.startswith("_"))
                raise ConfigError(f"the configuration of '{self.architecture}' has no field '{key}' "
                                  f"(it has: {', '.join(fields)})")
            current = getattr(self, key)
            if isinstance(current, float) and isinstance(value, int) and not isinstance(value, bool):
                value = float(value)
            if current is not None and value is not None and type(current) is not type(value):
                raise ConfigError(f"field '{key}' of '{self.architecture}' is {type(current).__name__}, "
                                  f"got {type(value).__name__} {value!r}")
            setattr(self, key, value)
        self.validate(origin)

    # ------------------------------------------------------------------ writing
    def to_dict(self) -> Dict[str, Any]:
        raise NotImplementedError(f"{type(self).__name__} must say what its config.json holds in to_dict")

    def model_spec(self) -> Any:
        raise NotImplementedError(f"{type(self).__name__} must describe its model in model_spec")
