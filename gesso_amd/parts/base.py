"""What every part is: a spec, the tensors it needs, and a forward over flattened tokens.

A part never learns which model holds it.  It is built from its spec (every size and
constant a field) and a :class:`Runtime` (device, dtype, kernels); it names the tensors it
needs by local names (``q_proj.weight``); the block's name table maps those to the names
in the weight file.

Interfaces (duck-typed; the classes below are convenient bases):

* norm            ``tensor_specs(spec)``, ``bind(tensors)``, ``add_norm(stream, rows=None, out=None) -> normed``;
                  optional hint ``row_weight``: a float32 vector ``w`` with ``norm(x) = inv_rms(x) * (x * w)``, which
                  lets whatever writes the stream before the norm leave the rows pre-weighted (None: no such form)
* position        ``tensor_specs(spec)`` (usually none), ``bind``, attributes
                  ``cos``, ``sin`` (``(max_position, rotary_dim/2)`` float32), ``rotary_dim`` and ``layout``
                  (``"half"``: pairs ``(i, i + rotary_dim/2)``, ``"interleaved"``: ``(2i, 2i + 1)``);
                  or ``rotary_dim == 0`` for none
* mixer           ``tensor_specs(spec)``, ``cache_need(spec) -> PagedKV | SlotState | None``,
                  ``bind(tensors)``, ``forward(x, ctx, cache) -> (T, hidden)``
* feed-forward    ``tensor_specs(spec)``, ``bind(tensors)``, ``forward(x, ctx) -> (T, hidden)``
* block           ``tensor_specs(spec)``, ``cache_need(spec)``, ``bind``,
                  ``forward(stream, ctx, cache)`` on a :class:`ResidualStream`; optional hint ``first_norm``: the
                  norm that reads the stream first when the block runs (None: unknown)

``Part`` below carries the optional hints with their defaults, so a part derived from it need not mention them.
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
    """Per-token state kept in pages: per token and key head a key row of ``head_dim`` and a value row of
    ``value_dim`` numbers (None: as wide as the key; 0: no value rows at all, for a mixer that caches one row per
    token and derives both from it).

    ``window``: only the last ``window`` tokens are ever read again (None = all of them).
    """

    n_kv_heads: int
    head_dim: int
    window: Optional[int] = None
    value_dim: Optional[int] = None

    @property
    def value_width(self) -> int:
        return self.head_dim if self.value_dim is None else int(self.value_dim)


@dataclass(frozen=True)
class SlotState:
    """Per-request state of fixed size.  ``tensors``: ``(name, shape, dtype name)`` or ``(name, shape, dtype name,
    initial value)`` each; ``dtype name`` is ``"float32"`` or ``"bfloat16"``; a slot handed to a request is filled
    with the initial value (0 unless given)."""

    tensors: Tuple[tuple, ...]

    def entries(self):
        """``(name, shape, dtype name, initial value)`` of every tensor."""
        out = []
        for t in self.tensors:
            if len(t) not in (3, 4):
                raise ValueError(f"a state tensor is (name, shape, dtype[, initial value]), not {t!r}")
            name, shape, dtype = t[:3]
            out.append((name, tuple(int(n) for n in shape), dtype, float(t[3]) if len(t) == 4 else 0.0))
        return out


class Part:
    """Base of parts: keeps spec and runtime; subclasses fill the rest."""

    graph_safe = False      # True: forward makes no host round trip, so a decode step through it may be recorded
    row_weight = None       # norms: see the module's text
    first_norm = None       # blocks: see the module's text

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
