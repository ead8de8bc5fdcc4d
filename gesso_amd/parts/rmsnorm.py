"""RMSNorm: ``y = x / sqrt(mean(x^2) + eps) * w`` over the last axis, eps inside the root, no +1.

Reference: ``src/Operators/cpu.jl:293-312``.  The kernel folds the residual add that precedes
the norm into the same pass, as the reference's seam does (``src/Inference/Inference.jl:1936-1939``).
"""
from __future__ import annotations

from .base import VECTOR, Part, TensorSpec
from .registry import register


class ResidualStream:
    """The float32 hidden state ``res (T, H)`` and a sub-layer output not yet added to it.

    ``push`` takes a sub-layer's output: a tensor becomes ``pending`` (the next norm adds it), a
    deferred product (:class:`~gesso_amd.parts.runtime.DeferredLinear`) is computed straight into
    ``res``, which leaves the new rows' sums of squares in ``ssq`` for a lazy norm.
    """

    __slots__ = ("res", "pending", "ssq")

    def __init__(self, res, pending=None, ssq=None):
        self.res = res
        self.pending = pending
        self.ssq = ssq

    def push(self, out, rt) -> None:
        from .runtime import DeferredLinear
        if isinstance(out, DeferredLinear):
            self.flush(rt)
            self.ssq = rt.ops.gemm_skinny_residual(out.x, out.w, self.res, wt=rt._wt(out.w))
        else:
            self.flush(rt)
            self.pending, self.ssq = out, None

    def flush(self, rt) -> None:
        """Add what is pending, if a norm has not done so."""
        if self.pending is not None:
            rt.ops.residual_add(self.res, self.pending)
            self.pending, self.ssq = None, None


class RMSNorm(Part):
    graph_safe = True

    @staticmethod
    def tensor_specs(spec):
        return {"weight": TensorSpec((spec.size,), VECTOR, "one_plus_normal")}

    def bind(self, tensors):
        self.weight = tensors["weight"]

    def add_norm(self, stream: ResidualStream, rows=None, out=None):
        """Add what is pending to the stream, then norm it (only ``rows`` of it when given).

        While a decode step is recorded with fused kernels, and the stream's sums of squares are at
        hand, the norm is not run: a :class:`~gesso_amd.kernels.ops.LazyNorm` goes to the product that
        follows, which norms on the fly.
        """
        if self.rt.fused and rows is None and stream.pending is None and stream.ssq is not None:
            return self.rt.ops.LazyNorm(stream.res, stream.ssq, self.weight, self.spec.eps, self.rt.dtype)
        y = self.rt.ops.add_rmsnorm(stream.res, stream.pending, self.weight, self.spec.eps, self.rt.dtype,
                                    rows=rows, out=out)
        if rows is None:
            stream.pending = None
            stream.ssq = None
        return y


register("norm", "rmsnorm", RMSNorm)
