"""Binding tensors by name: from a model folder to the device, or from a seed.

The loader walks the model's tensor table (``file name -> shape, role``) and the files'
headers and reports **all** faults in one :class:`~gesso_amd.errors.WeightError`: missing
tensors, unexpected ones, wrong shapes, unusable types; as the reference's binder does one by
one (``src/Inference/materialize_architecture.jl:217-222``, ``:344-349``, ``:369-384``).

Storage widths: in ``bfloat16`` mode a matrix stored in bfloat16 stays bfloat16 and a matrix
stored in 32-bit stays 32-bit (its products then run in float32); half precision and float64
become float32.  Small vectors (norm weights, taps, biases) are held in float32, an exact
widening of bfloat16.  In ``float32`` mode everything is widened to float32.  Integer tables
would be kept as int32.  A tied head may be present in the file if it equals the embedding
table (``materialize_architecture.jl:268-289``).
"""
from __future__ import annotations

import os
from typing import Dict, Iterable

import torch

from ..errors import WeightError
from ..parts.base import VECTOR, TensorSpec
from .safetensors_io import open_model_files, write_safetensors

_FLOATS = (torch.float64, torch.float32, torch.float16, torch.bfloat16)
_INTS = (torch.int64, torch.int32, torch.int16, torch.int8, torch.uint8)


def held_dtype(stored: torch.dtype, role: str, mode: torch.dtype) -> torch.dtype:
    """The type a tensor of ``role`` stored as ``stored`` is held in when the engine runs in ``mode``."""
    if stored in _INTS:
        return torch.int32
    if mode == torch.float32 or role == VECTOR:
        return torch.float32
    return torch.bfloat16 if stored == torch.bfloat16 else torch.float32


def load_tensors(model_dir: str, table: Dict[str, TensorSpec], mode: torch.dtype, device,
                 aliases: Dict[str, str] = None, ignored_suffixes: Iterable[str] = ()) -> Dict[str, torch.Tensor]:
    files = open_model_files(model_dir)
    aliases = aliases or {}
    where = {}
    duplicates = []
    for f in files:
        for name in f.names():
            if name in where:
                duplicates.append(name)
            where[name] = f
    missing = [n for n in table if n not in where]
    unexpected = [n for n in where if n not in table and n not in aliases
                  and not any(n.endswith(s) for s in ignored_suffixes)]
    wrong_shape, wrong_type = [], []
    for name, ts in table.items():
        if name in where:
            f = where[name]
            if _core(f.shape(name)) != _core(ts.shape):
                wrong_shape.append(f"{name}: file has {tuple(f.shape(name))}, the configuration needs {tuple(ts.shape)}")
            if f.dtype(name) not in _FLOATS:
                wrong_type.append(f"{name}: {f.dtype(name)}")
    if missing or unexpected or wrong_shape or wrong_type or duplicates:
        parts = []
        if missing:
            parts.append(f"{len(missing)} missing: " + ", ".join(sorted(missing)))
        if unexpected:
            parts.append(f"{len(unexpected)} unexpected: " + ", ".join(sorted(unexpected)))
        if wrong_shape:
            parts.append(f"{len(wrong_shape)} with wrong shape: " + "; ".join(wrong_shape))
        if wrong_type:
            parts.append(f"{len(wrong_type)} with unusable type: " + "; ".join(wrong_type))
        if duplicates:
            parts.append(f"{len(duplicates)} stored twice: " + ", ".join(sorted(duplicates)))
        raise WeightError(f"weights of {model_dir} do not fit the configuration: " + " | ".join(parts),
                          missing=sorted(missing), unexpected=sorted(unexpected), wrong_shape=wrong_shape,
                          wrong_type=wrong_type, duplicates=sorted(duplicates))
    out = {}
    for name, ts in table.items():
        t = where[name].tensor(name).reshape(ts.shape)      # axes of length one may be stored or left out
        out[name] = t.to(device=device, dtype=held_dtype(t.dtype, ts.role, mode)).contiguous()
    for alias, target in aliases.items():
        if alias in where:
            a, b = where[alias].tensor(alias), where[target].tensor(target)
            if a.shape != b.shape or a.dtype != b.dtype or not torch.equal(a, b):
                raise WeightError(f"{alias} is present though tied to {target}, and differs from it",
                                  unexpected=[alias])
    for f in files:
        f.close()
    return out


def _core(shape) -> tuple:
    """A shape without its axes of length one: a depthwise convolution's taps are (H, 1, W) in some files, (H, W) in
    others, and mean the same."""
    return tuple(int(n) for n in shape if int(n) != 1)


def random_tensors(table: Dict[str, TensorSpec], seed: int, dtype: torch.dtype, device="cpu",
                   std: float = 0.02) -> Dict[str, torch.Tensor]:
    """Seeded random weights, tensor by tensor in the table's order from one generator.

    ``normal``: N(0, std); ``one_plus_normal`` (norm weights): 1 + N(0, std).  Drawn in float32
    and rounded to ``dtype``, so the same seed gives the float32 file and its bfloat16 rounding.
    """
    gen = torch.Generator(device=device)
    gen.manual_seed(int(seed))
    out = {}
    for name, ts in table.items():
        t = torch.empty(ts.shape, dtype=torch.float32, device=device).normal_(0.0, std, generator=gen)
        if ts.init == "one_plus_normal":
            t += 1.0
        elif ts.init != "normal":
            raise WeightError(f"unknown initialisation {ts.init!r} for {name}")
        out[name] = t.to(dtype)
    return out


def write_model_folder(out_dir: str, config, seed: int, dtype: torch.dtype = torch.bfloat16, std: float = 0.02) -> str:
    """Write ``config.json`` and ``model.safetensors`` with seeded random weights for a typed configuration."""
    import json

    from ..config.registry import architecture_of
    from ..models.model import tensor_table

    raw = config.to_json()
    arch = architecture_of(raw)
    spec = arch.to_spec(config)
    os.makedirs(out_dir, exist_ok=True)
    with open(os.path.join(out_dir, "config.json"), "w", encoding="utf-8") as f:
        json.dump(raw, f, indent=1)
    tensors = random_tensors(tensor_table(spec), seed, dtype, std=std)
    write_safetensors(os.path.join(out_dir, "model.safetensors"), tensors,
                      metadata={"format": "pt", "seed": str(seed)})
    return out_dir
