"""Strict JSON for configuration files: a duplicate key is an error, not a silent overwrite.

The reference reads ``config.json`` the same way (``src/Inference/llama_import.jl:43-57``).
"""
from __future__ import annotations

import json

from ..errors import ConfigError


def _no_duplicates(pairs):
    out = {}
    for key, value in pairs:
        if key in out:
            raise ConfigError(f"duplicate key {key!r} in JSON object", key=key)
        out[key] = value
    return out


def loads_strict(text: str, what: str = "JSON") -> dict:
    try:
        value = json.loads(text, object_pairs_hook=_no_duplicates)
    except json.JSONDecodeError as err:
        raise ConfigError(f"{what} is not valid JSON: {err}") from err
    if not isinstance(value, dict):
        raise ConfigError(f"{what} must hold a JSON object, found {type(value).__name__}")
    return value


def load_strict(path: str) -> dict:
    try:
        with open(path, "r", encoding="utf-8") as f:
            text = f.read()
    except OSError as err:
        raise ConfigError(f"cannot read {path}: {err}", path=path) from err
    return loads_strict(text, what=path)
