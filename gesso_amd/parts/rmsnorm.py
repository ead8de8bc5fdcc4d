"""RMSNorm: ``y = x / sqrt(mean(x^2) + eps) * w`` over the last axis, eps inside the root, no +1.

Reference: ``src/Operators/cpu.jl:293-312``.  The kernel folds the residual add that precedes
the norm into the same pass, as the reference's seam does (``src/Inference/Inference.jl:1936-1939``).
"""
from __future__ import annotations

import torch

from .base import VECTOR, Part, TensorSpec
from .registry import register


class ResidualStream:
    """The float32 hidden state ``res (T, H)`` and a sub-layer output not yet added to it.

    ``push`` takes a sub-layer's output: a tensor becomes ``pending`` (the next norm adds it), a
    deferred product (:class:`~gesso_amd.parts.runtime.DeferredLinear`) is computed straight into
    ``res``, which leaves the new rows' sums of squares in ``ssq`` for a lazy norm.

    Whoever knows which norm reads the stream next may say so (``next_norm`` of ``push``; ``following``, set
    by the model, names the norm after the current block).  If that norm offers ``row_weight`` (a float32
    vector ``w`` with ``norm(x) = inv_rms(x) * (x * w)``), the deferred product also leaves ``xs = res * w``
    in bfloat16, and the norm's consumer needs no norm pass at all.  ``xs_for`` is the norm ``xs`` was made for.
    """

    __slots__ = ("res", "pending", "ssq", "xs", "xs_for", "following", "normed")

    def __init__(self, res, pending=None, ssq=None, xs=None, xs_for=None):
        self.res = res
        self.pending = pending
        self.ssq = ssq
        self.xs, self.xs_for = xs, xs_for
        self.following = None
        self.normed = None            # the rows normed for ``xs_for``, where the last push made them

    def push(self, out, rt, next_norm=None) -> None:
        from .runtime import DeferredLinear
        self.flush(rt)
        self.xs = self.xs_for = self.normed = None
        if isinstance(out, DeferredLinear) and self.res.shape[0] > rt.weighted_rows_max:
            # many rows: K is shared out over many blocks, and the pass that adds their partial sums to the stream
            # norms the rows for the next norm on its way (it sees whole rows)
            w = getattr(next_norm, "row_weight", None)
            eps = getattr(getattr(next_norm, "spec", None), "eps", None)
            if w is not None and (w.shape != (self.res.shape[1],) or eps is None):
                w = None
            eps = eps if w is not None else 0.0
            self.ssq, self.normed = rt.ops.gemm_skinny_residual_parts(
                out.x, out.w, self.res, rt.split_parts(out.w), wt=rt.tiles_of(out.w), next_weight=w, eps=eps, out_dtype=rt.dtype,
                tiled=w is not None and rt.rows_tiled(self.res.shape[1]))
            self.xs_for = next_norm if self.normed is not None else None
        elif isinstance(out, DeferredLinear):
            w = row_weight_of(next_norm, self.res, rt)
            if w is not None:
                self.xs = rt.new_rows(*self.res.shape)
                self.xs_for = next_norm
            self.ssq = rt.ops.gemm_skinny_residual(out.x, out.w, self.res, wt=rt.tiles_of(out.w), next_weight=w, xs=self.xs)
        else:
            self.pending, self.ssq = out, None

    def flush(self, rt) -> None:
        """Add what is pending, if a norm has not done so."""
        if self.pending is not None:
            rt.ops.residual_add(self.res, self.pending)
            self.pending, self.ssq = None, None
            self.xs = self.xs_for = self.normed = None


def row_weight_of(norm, res, rt):
    """``norm.row_weight`` if the norm offers one that fits the stream's width and the rows are few enough, else None."""
    w = getattr(norm, "row_weight", None)
    if w is None or w.dtype != res.dtype or w.shape != (res.shape[1],) or res.shape[0] > rt.weighted_rows_max:
        return None
    return w


class RMSNorm(Part):
    graph_safe = True
    portions_recordable = True

    @staticmethod
    def tensor_specs(spec):
        return {"weight": TensorSpec((spec.size,), VECTOR, "one_plus_normal")}

    def bind(self, tensors):
        self.weight = tensors["weight"]

    @property
    def row_weight(self):
        """``norm(x) = inv_rms(x) * (x * row_weight)``: what lets a producer pre-weight the rows for this norm."""
        return self.weight if self.rt.dtype == torch.bfloat16 else None

    def add_norm(self, stream: ResidualStream, rows=None, out=None):
        """Add what is pending to the stream, then norm it (only ``rows`` of it when given).

        While a decode step is recorded with fused kernels, and the stream's sums of squares are at
        hand, the norm is not run: a :class:`~gesso_amd.kernels.ops.LazyNorm` goes to the product that
        follows, which norms on the fly.
        """
        if self.rt.fused and rows is None and stream.pending is None and stream.ssq is not None:
            mine = stream.xs_for is self
            return self.rt.ops.LazyNorm(stream.res, stream.ssq, self.weight, self.spec.eps, self.rt.dtype,
                                        xs=stream.xs if mine else None, ready=stream.normed if mine else None)
        y = self.rt.ops.add_rmsnorm(stream.res, stream.pending, self.weight, self.spec.eps, self.rt.dtype,
                                    rows=rows, out=out)
        if rows is None:
            stream.pending = None
            stream.ssq = None
        return y


register("norm", "rmsnorm", RMSNorm)
