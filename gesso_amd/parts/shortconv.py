"""Gated short convolution mixer.

``bcx = x W_in^T`` gives B, C, X side by side; ``u = B * X``; a causal depthwise convolution of
``width`` taps over time (taps oldest to newest, the current input on the last tap); the gate
``C`` multiplies the sum; ``W_out`` projects back.  Reference: ``src/Inference/lfm2.jl:192-204``
and ``:253-271``.  The last ``width - 1`` values of ``u`` are the request's state, a slot of
fixed size, float32 in both precisions, zero at a request's start (``lfm2.jl:195``).
The convolution weight has the depthwise layout ``(hidden, 1, width)``.
"""
from __future__ import annotations

from .base import MATRIX, VECTOR, Part, SlotState, TensorSpec
from .registry import register


class ShortConv(Part):
    graph_safe = True
    portions_recordable = True
    stage, out_stage = "conv_mixer", "conv_out"       # the decode profiler's names

    @staticmethod
    def tensor_specs(spec):
        H, W = spec.hidden, spec.width
        out = {"in_proj.weight": TensorSpec((3 * H, H), MATRIX), "conv.weight": TensorSpec((H, 1, W), VECTOR),
               "out_proj.weight": TensorSpec((H, H), MATRIX)}
        if spec.bias:
            out.update({"in_proj.bias": TensorSpec((3 * H,), VECTOR), "conv.bias": TensorSpec((H,), VECTOR),
                        "out_proj.bias": TensorSpec((H,), VECTOR)})
        return out

    @staticmethod
    def cache_need(spec):
        return SlotState((("history", (spec.hidden, spec.width - 1), "float32"),))

    def bind(self, tensors):
        H, W = self.spec.hidden, self.spec.width
        self.w_in = self.rt.prepare(tensors["in_proj.weight"], unit=H)
        self.w_out = self.rt.prepare(tensors["out_proj.weight"])
        self.taps = tensors["conv.weight"].reshape(H, W).contiguous()
        self.b_in = tensors.get("in_proj.bias")
        self.b_conv = tensors.get("conv.bias")
        self.b_out = tensors.get("out_proj.bias")

    def forward(self, x, ctx, cache):
        mixed = self.mix(x, ctx, cache.state["history"])
        return self.rt.project(mixed, self.w_out, self.b_out)

    def mix(self, x, ctx, state):
        """Input product and gated short convolution: ``(T, H)`` mixed rows; ``state`` is advanced.

        While a decode step is recorded the convolution runs as the epilogue of its input product
        (one token per sequence, taps in registers); otherwise the product, then the kernel over segments."""
        rt, ops = self.rt, self.rt.ops
        if rt.fused and self.b_in is None and ctx.all_single and self.taps.shape[1] <= 16:
            x = rt.lazy_rows(x)
            if rt.streams(x, self.w_in):
                with rt.stage("conv_in"):          # product and convolution are one kernel here
                    return ops.gemm_skinny_conv(x, self.w_in, self.taps, self.b_conv, state, ctx.slots,
                                                wt=rt.tiles_of(self.w_in), tiled=rt.rows_tiled(self.taps.shape[0]))
        with rt.stage("conv_in"):
            bcx = rt.linear(rt.dense(x), self.w_in, self.b_in)
        with rt.stage("conv_mix"):
            return ops.short_conv(bcx, self.taps, self.b_conv, state, ctx.seq_of_token, ctx.q_start, ctx.slots,
                                  ctx.nseq, ctx.all_single)


register("mixer", "short_conv", ShortConv)
