"""Choosing the next token: greedy, temperature, nucleus; in the reference's manner.

Greedy is the default: the first maximum of the row (ties go to the lowest id), and a row with
a NaN or an infinity yields no token but :class:`~gesso_amd.errors.NumericalInstability`
(``src/Inference/session.jl:444-458``).  ``Sampler(temperature=, top_p=1.0, seed=)`` is the
reference's opt-in sampler (``src/Inference/sampling.jl:13-29``): weights
``exp((x - max) / temperature)`` in float64, exactly one draw of a fixed splitmix64 generator per
token (``:32-39``), an inverse-CDF walk in id order, or, with ``top_p < 1``, in descending-weight
order over the shortest prefix whose mass reaches ``top_p`` (``:43-74``).  The draw is made on
the host (it is a few integer operations); the rows never leave the GPU.
"""
from __future__ import annotations

from typing import List, Optional, Sequence, Union

import torch

from ..errors import InvalidPlan, NumericalInstability

_M64 = (1 << 64) - 1


class Sampler:
    """Temperature and nucleus sampling state of one request; one draw per token."""

    def __init__(self, temperature: float, top_p: float = 1.0, seed: int = 0):
        if not temperature > 0:
            raise InvalidPlan(f"sampler temperature must be > 0, got {temperature}")
        if not 0 < top_p <= 1:
            raise InvalidPlan(f"sampler top_p must be in (0, 1], got {top_p}")
        if seed < 0:
            raise InvalidPlan(f"sampler seed must be >= 0, got {seed}")
        self.temperature = float(temperature)
        self.top_p = float(top_p)
        self.state = int(seed) & _M64

    def unit(self) -> float:
        """One splitmix64 step; a float in [0, 1) from the top 53 bits."""
        self.state = (self.state + 0x9E3779B97F4A7C15) & _M64
        z = self.state
        z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _M64
        z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _M64
        z ^= z >> 31
        return float(z >> 11) * 2.0 ** -53

    def clone(self) -> "Sampler":
        s = Sampler(self.temperature, self.top_p, 0)
        s.state = self.state
        return s


def choose(ops, logits: torch.Tensor, samplers: Sequence[Optional[Sampler]]) -> List[Union[int, Exception]]:
    """One token id per row of ``logits (rows, V)``; ``samplers[i] is None`` means greedy.

    A row with a non-finite logit gives a :class:`NumericalInstability` in its place (and its
    sampler makes no draw), so that one request's fault does not stop the others.
    """
    rows = logits.shape[0]
    if rows != len(samplers):
        raise InvalidPlan("one sampler entry per row of logits")
    dev = logits.device
    if all(s is None for s in samplers):
        ids, bad = ops.argmax_rows(logits)
    else:
        # every row in one pass, each in its own manner.  The draws are made before the rows are known to be finite; a
        # row that is not emits no token and makes no draw, so its sampler goes back to where it stood
        before = [None if s is None else s.state for s in samplers]
        facts = torch.tensor([[0.0 if s is None else s.temperature for s in samplers],
                              [1.0 if s is None else s.top_p for s in samplers],
                              [0.0 if s is None else s.unit() for s in samplers]], dtype=torch.float64).to(dev)
        ids, bad = ops.choose_rows(logits, facts[0], facts[1], facts[2])
    ids, bad = ids.tolist(), bad.tolist()
    out: List[Union[int, Exception]] = []
    for i, (tok, b) in enumerate(zip(ids, bad)):
        if b:
            if samplers[i] is not None:
                samplers[i].state = before[i]
            out.append(NumericalInstability("non-finite logits: no token is emitted", row=i))
        else:
            out.append(int(tok))
    return out
