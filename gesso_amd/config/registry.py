"""One registry from an architecture's name to its configuration type and model factory.

``config.json`` names the architecture in ``architectures[0]``; the entry registered under
that name parses the file's keys into a typed configuration and turns the configuration
into a :class:`~gesso_amd.config.spec.ModelSpec`.  The reference's counterpart is the
adapter table ``_ADAPTERS`` with ``adapter_for`` (``src/Inference/arch_adapters.jl:1075-1109``),
whose error lists the known names; so does ours.
"""
from __future__ import annotations

import os
from dataclasses import dataclass
from typing import Callable, Dict

from ..errors import ConfigError
from .jsonio import load_strict
from .spec import ModelSpec


@dataclass(frozen=True)
class Architecture:
    name: str
    parse: Callable[[dict], object]          # config.json keys -> typed configuration
    to_spec: Callable[[object], ModelSpec]   # typed configuration -> model as data
    to_json: Callable[[object], dict]        # typed configuration -> config.json keys


_ARCHITECTURES: Dict[str, Architecture] = {}


def register_architecture(name: str, parse, to_spec, to_json) -> None:
    if name in _ARCHITECTURES:
        raise ConfigError(f"architecture {name!r} is already registered")
    _ARCHITECTURES[name] = Architecture(name, parse, to_spec, to_json)


def unregister_architecture(name: str) -> None:
    _ARCHITECTURES.pop(name, None)


def registered_architectures():
    return sorted(_ARCHITECTURES)


def architecture_of(raw: dict) -> Architecture:
    names = raw.get("architectures")
    if not (isinstance(names, list) and len(names) >= 1 and isinstance(names[0], str)):
        raise ConfigError("config.json must name its model in architectures[0]",
                          known=registered_architectures())
    arch = _ARCHITECTURES.get(names[0])
    if arch is None:
        raise ConfigError(f"unknown architecture {names[0]!r}", known=registered_architectures())
    return arch


def load_config(model_dir: str):
    """``(architecture entry, typed configuration)`` of a model folder."""
    raw = load_strict(os.path.join(model_dir, "config.json"))
    arch = architecture_of(raw)
    return arch, arch.parse(raw)
