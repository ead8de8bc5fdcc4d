"""RMSNorm: ``y = x / sqrt(mean(x^2) + eps) * w`` over the last axis, eps inside the root, no +1.

Reference: ``src/Operators/cpu.jl:293-312``.  The kernel folds the residual add that precedes
the norm into the same pass, as the reference's seam does (``src/Inference/Inference.jl:1936-1939``).
"""
from __future__ import annotations

from .base import VECTOR, Part, TensorSpec
from .registry import register


class ResidualStream:
    """The float32 hidden state ``res (T, H)`` and a sub-layer output not yet added to it."""

    __slots__ = ("res", "pending")

    def __init__(self, res, pending=None):
        self.res = res
        self.pending = pending


class RMSNorm(Part):
    @staticmethod
    def tensor_specs(spec):
        return {"weight": TensorSpec((spec.size,), VECTOR, "one_plus_normal")}

    def bind(self, tensors):
        self.weight = tensors["weight"]

    def add_norm(self, stream: ResidualStream, rows=None, out=None):
        """Add what is pending to the stream, then norm it (only ``rows`` of it when given)."""
        y = self.rt.ops.add_rmsnorm(stream.res, stream.pending, self.weight, self.spec.eps, self.rt.dtype,
                                    rows=rows, out=out)
        if rows is None:
            stream.pending = None
        return y


register("norm", "rmsnorm", RMSNorm)
