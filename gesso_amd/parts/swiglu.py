"""SwiGLU feed-forward: ``w2( silu(w1 x) * (w3 x) )``, ``silu(g) = g / (1 + exp(-g))``.

Reference: ``src/Inference/Inference.jl:843-884`` and ``src/Operators/cpu.jl:482-488``.
w1 (gate) and w3 (up) are laid side by side at load so that one product feeds both, as the
reference groups projections that share an input (``src/Inference/cpu_decode.jl:195-211``).
"""
from __future__ import annotations

import torch

from .base import MATRIX, Part, TensorSpec
from .registry import register


class SwiGLU(Part):
    graph_safe = True
    portions_recordable = True
    stage, out_stage = "dense_ffn", "ffn_down"        # the decode profiler's names

    @staticmethod
    def tensor_specs(spec):
        H, F = spec.hidden, spec.intermediate
        return {"w1.weight": TensorSpec((F, H), MATRIX), "w3.weight": TensorSpec((F, H), MATRIX),
                "w2.weight": TensorSpec((H, F), MATRIX)}

    def bind(self, tensors):
        w1, w3 = tensors["w1.weight"], tensors["w3.weight"]
        if w1.dtype != w3.dtype:
            w1, w3 = w1.float(), w3.float()
        self.w13 = self.rt.prepare(torch.cat([w1, w3], 0).contiguous(), unit=w1.shape[0])
        self.w2 = self.rt.prepare(tensors["w2.weight"])

    def forward(self, x, ctx):
        with self.rt.stage("ffn_gateup"):                # with its activation where the kernel fuses them
            a = self.rt.linear_swiglu(x, self.w13)
        return self.rt.project(a, self.w2)


register("ffn", "swiglu", SwiGLU)
