"""What every part is: a spec, the tensors it needs, and a forward over flattened tokens.

A part never learns which model holds it.  It is built from its spec (every size and
constant a field) and a :class:`Runtime` (device, dtype, kernels); it names the tensors it
needs by local names (``q_proj.weight``); the block's name table maps those to the names
in the weight file.

Interfaces (duck-typed; the classes below are convenient bases):

* norm            ``tensor_specs(spec)``, ``bind(tensors)``,
                  ``add_norm(residual, delta, out=None, rows=None) -> normed``
* position        ``tensor_specs(spec)`` (usually none), ``bind``, attributes
                  ``cos``, ``sin`` (``(max_position, rotary_dim/2)`` float32) and ``rotary_dim``;
                  or ``rotary_dim == 0`` for none
* mixer           ``tensor_specs(spec)``, ``cache_need(spec) -> PagedKV | SlotState | None``,
                  ``bind(tensors)``, ``forward(x, ctx, cache) -> (T, hidden)``
* feed-forward    ``tensor_specs(spec)``, ``bind(tensors)``, ``forward(x, ctx) -> (T, hidden)``
* block           ``tensor_specs(spec)``, ``cache_need(spec)``, ``bind``,
                  ``forward(stream, ctx, cache)`` on a :class:`ResidualStream`
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Optional, Tuple

MATRIX = "matrix"     # operand of a matrix product: keeps the stored width (bfloat16 stays bfloat16)
VECTOR = "vector"     # norm weights, taps, biases: held in float32 (an exact widening)
TABLE = "table"       # embedding table; a matrix that is also gathered from


@dataclass(frozen=True)
class TensorSpec:
    shape: Tuple[int, ...]
    role: str = MATRIX
    init: str = "normal"          # "normal": N(0, std); "one_plus_normal": 1 + N(0, std)


@dataclass(frozen=True)
class PagedKV:
    """Per-token state: keys and values of ``n_kv_heads x head_dim`` per token, kept in pages.

    ``window``: only the last ``window`` tokens are ever read again (None = all of them).
    """

    n_kv_heads: int
    head_dim: int
    window: Optional[int] = None


@dataclass(frozen=True)
class SlotState:
    """Per-request state of fixed size: ``name -> (shape, dtype name)``; zero at a request's start."""

    tensors: Tuple[Tuple[str, Tuple[int, ...], str], ...]


class Part:
    """Base of parts: keeps spec and runtime; subclasses fill the rest."""

    def __init__(self, spec, rt):
        self.spec = spec
        self.rt = rt

    @staticmethod
    def tensor_specs(spec) -> Dict[str, TensorSpec]:
        return {}

    def bind(self, tensors: Dict[str, "object"]) -> None:
        if tensors:
            raise ValueError(f"{type(self).__name__} takes no tensors, got {sorted(tensors)}")


def sub_tensors(tensors: Dict[str, object], prefix: str) -> Dict[str, object]:
    """The entries of ``tensors`` under ``prefix.``, with the prefix removed."""
    p = prefix + "."
    return {k[len(p):]: v for k, v in tensors.items() if k.startswith(p)}
