"""Typed reading of a model folder's JSON configuration.

A configuration class declares its fields once; ``JsonReader`` fetches each
key with a type check and produces errors that name the key and the file, in
the manner of the reference's ``read_required_*`` helpers
(reference: src/model/qwen3/config.cpp:70-138).
"""
from __future__ import annotations

import json
import os
from typing import Any, Dict, List, Optional, Sequence


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
        raise ConfigError(f"Config file '{path}' does not exist")
    try:
        with open(path, "r", encoding="utf-8") as fh:
            text = fh.read()
        try:
            data = json.loads(text)
        except json.JSONDecodeError:
            data = json.loads(strip_json_comments(text))
    except json.JSONDecodeError as exc:
        raise ConfigError(f"Config file '{path}' is not valid JSON: {exc}") from exc
    if not isinstance(data, dict):
        raise ConfigError(f"Config file '{path}' must hold a JSON object")
    return data


class JsonReader:
    """Typed access to one JSON object; every error names the key and the file."""

    def __init__(self, data: Dict[str, Any], origin: str):
        self.data = data
        self.origin = origin

    def _fail(self, kind: str, key: str) -> ConfigError:
        return ConfigError(f"Missing or invalid {kind} key '{key}' in '{self.origin}'")

    def has(self, key: str) -> bool:
        return key in self.data and self.data[key] is not None

    def raw(self, key: str, default: Any = None) -> Any:
        return self.data.get(key, default)

    def integer(self, key: str, default: Any = _MISSING) -> int:
        value = self.data.get(key, None)
        if value is None:
            if default is _MISSING:
                raise self._fail("integer", key)
            return default
        if isinstance(value, bool) or not isinstance(value, int):
            if isinstance(value, float) and value.is_integer():
                return int(value)
            raise self._fail("integer", key)
        return int(value)

    def number(self, key: str, default: Any = _MISSING) -> float:
        value = self.data.get(key, None)
        if value is None:
            if default is _MISSING:
                raise self._fail("number", key)
            return default
        if isinstance(value, bool) or not isinstance(value, (int, float)):
            raise self._fail("number", key)
        return float(value)

    def boolean(self, key: str, default: Any = _MISSING) -> bool:
        value = self.data.get(key, None)
        if value is None:
            if default is _MISSING:
                raise self._fail("boolean", key)
            return default
        if not isinstance(value, bool):
            raise self._fail("boolean", key)
        return value

    def string(self, key: str, default: Any = _MISSING) -> str:
        value = self.data.get(key, None)
        if value is None:
            if default is _MISSING:
                raise self._fail("string", key)
            return default
        if not isinstance(value, str):
            raise self._fail("string", key)
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
        raise ConfigError(f"Invalid int list key '{key}' in '{self.origin}'")

    def string_list(self, key: str) -> Optional[List[str]]:
        value = self.data.get(key, None)
        if value is None:
            return None
        if isinstance(value, list) and all(isinstance(v, str) for v in value):
            return list(value)
        raise self._fail("string list", key)


def require_positive(origin: str, **named: int) -> None:
    bad = [name for name, value in named.items() if value <= 0]
    if bad:
        raise ConfigError(f"Invalid model dimensions in '{origin}': {', '.join(bad)} must be positive")


def architecture_name(data: Dict[str, Any], origin: str) -> str:
    archs = data.get("architectures")
    if not isinstance(archs, Sequence) or isinstance(archs, str) or len(archs) == 0 or not isinstance(archs[0], str):
        raise ConfigError(f"Missing or invalid string list key 'architectures' in '{origin}'")
    return archs[0]
