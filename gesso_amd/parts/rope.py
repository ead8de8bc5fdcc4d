"""Position encodings as tables: what the attention kernels need is ``cos``, ``sin``, ``rotary_dim`` and ``layout``.

Rotary; pair ``i`` is ``(i, i + rotary_dim/2)`` (``layout = "half"``) or ``(2i, 2i + 1)`` (``"interleaved"``), its
angle ``pos * theta^(-2i/rotary_dim)`` (reference ``src/Operators/cpu.jl:357-371``; LFM2 has ``interleaved=false``,
``src/Inference/architecture_spec.jl:66``).  A kernel that is written for one layout is not used for the other: the
mixer asks ``layout`` before it takes a fused route.  Angles, cosines and
sines are computed on the host in float64 and stored as float32, one table per distinct spec.
Another encoding (scaled frequencies, another theta per layer) is another class that fills
the same three attributes; ``rotary_dim = 0`` means none.
"""
from __future__ import annotations

import torch

from .base import Part
from .registry import register


def rope_tables(rotary_dim: int, theta: float, max_position: int):
    i = torch.arange(rotary_dim // 2, dtype=torch.float64)
    inv_freq = torch.tensor(float(theta), dtype=torch.float64) ** (-2.0 * i / rotary_dim)
    ang = torch.arange(max_position, dtype=torch.float64)[:, None] * inv_freq[None, :]
    return torch.cos(ang).to(torch.float32), torch.sin(ang).to(torch.float32)


class Rope(Part):
    graph_safe = True

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        if spec.rotary_dim % 2 or not 0 < spec.rotary_dim <= spec.head_dim:
            raise ValueError(f"rotary_dim {spec.rotary_dim} must be even and within the head width {spec.head_dim}")
        self.rotary_dim = spec.rotary_dim
        self.layout = getattr(spec, "layout", "half")
        if self.layout not in rt.ops.ROPE_LAYOUTS:
            raise ValueError(f"rotation pairs are laid out 'half' or 'interleaved', not {self.layout!r}")

        def make():
            cos, sin = rope_tables(spec.rotary_dim, spec.theta, spec.max_position)
            return cos.to(rt.device), sin.to(rt.device)

        self.cos, self.sin = rt.shared(("rope", spec.rotary_dim, float(spec.theta), spec.max_position), make)


class NoPosition(Part):
    graph_safe = True
    rotary_dim = 0
    layout = "half"
    cos = None
    sin = None


register("position", "rope", Rope)
register("position", "none", NoPosition)
