"""Registries of part kinds: mixers, feed-forwards, norms, position encodings, blocks.

A spec's ``kind`` picks the class.  Registering a new kind (from a test, from another
architecture's file) needs no change here: ``register("mixer", "my_kind", MyMixer)``.
"""
from __future__ import annotations

from typing import Dict

from ..errors import ConfigError

CATEGORIES = ("mixer", "ffn", "norm", "position", "block")
_PARTS: Dict[str, Dict[str, type]] = {c: {} for c in CATEGORIES}


def register(category: str, kind: str, cls: type, replace: bool = False) -> type:
    if category not in _PARTS:
        raise ConfigError(f"unknown part category {category!r}", known=CATEGORIES)
    if kind in _PARTS[category] and not replace and _PARTS[category][kind] is not cls:
        raise ConfigError(f"{category} kind {kind!r} is already registered")
    _PARTS[category][kind] = cls
    return cls


def unregister(category: str, kind: str) -> None:
    _PARTS[category].pop(kind, None)


def part_class(category: str, spec) -> type:
    kind = getattr(spec, "kind", None)
    cls = _PARTS[category].get(kind)
    if cls is None:
        raise ConfigError(f"no {category} of kind {kind!r} is registered", known=sorted(_PARTS[category]))
    return cls


def build(category: str, spec, rt):
    return part_class(category, spec)(spec, rt)
