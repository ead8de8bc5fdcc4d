"""Grouped-query causal attention over the paged cache.

``q, k, v = x Wq^T, x Wk^T, x Wv^T``; per-head RMSNorm of q and k (when the spec has one),
then the position encoding, both before the cache write; keys and values of this step go
into the request's pages and the queries read all keys they may see from there.
Reference: ``src/Inference/Inference.jl:296-357`` (order of norm and rotation ``:307-323``),
causal rule ``:1206-1207``, grouping ``:1852-1870``.  The cache holds post-norm, post-rotation
keys and raw values (``:2417-2422``).  Wq, Wk, Wv are laid side by side at load.
"""
from __future__ import annotations

import math

import torch

from .base import MATRIX, VECTOR, PagedKV, Part, TensorSpec
from .registry import build, register


class Attention(Part):
    graph_safe = True

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        if spec.n_heads % spec.n_kv_heads:
            raise ValueError("query heads must be a multiple of key heads")
        self.position = build("position", spec.position, rt)
        self.scale = spec.scale if spec.scale is not None else 1.0 / math.sqrt(spec.head_dim)

    @staticmethod
    def tensor_specs(spec):
        H, nh, nkv, d = spec.hidden, spec.n_heads, spec.n_kv_heads, spec.head_dim
        out = {"q_proj.weight": TensorSpec((nh * d, H), MATRIX), "k_proj.weight": TensorSpec((nkv * d, H), MATRIX),
               "v_proj.weight": TensorSpec((nkv * d, H), MATRIX), "out_proj.weight": TensorSpec((H, nh * d), MATRIX)}
        if spec.bias:
            out.update({"q_proj.bias": TensorSpec((nh * d,), VECTOR), "k_proj.bias": TensorSpec((nkv * d,), VECTOR),
                        "v_proj.bias": TensorSpec((nkv * d,), VECTOR), "out_proj.bias": TensorSpec((H,), VECTOR)})
        if spec.qk_norm is not None:
            out.update({"q_norm.weight": TensorSpec((d,), VECTOR, "one_plus_normal"),
                        "k_norm.weight": TensorSpec((d,), VECTOR, "one_plus_normal")})
        return out

    @staticmethod
    def cache_need(spec):
        return PagedKV(spec.n_kv_heads, spec.head_dim, spec.window)

    def bind(self, tensors):
        ws = [tensors["q_proj.weight"], tensors["k_proj.weight"], tensors["v_proj.weight"]]
        if len({w.dtype for w in ws}) > 1:
            ws = [w.float() for w in ws]
        self.wqkv = self.rt.prepare(torch.cat(ws, 0).contiguous())
        self.wo = self.rt.prepare(tensors["out_proj.weight"])
        self.bqkv = self.bo = None
        if self.spec.bias:
            self.bqkv = torch.cat([tensors["q_proj.bias"], tensors["k_proj.bias"], tensors["v_proj.bias"]], 0).contiguous()
            self.bo = tensors["out_proj.bias"]
        self.q_norm = tensors.get("q_norm.weight")
        self.k_norm = tensors.get("k_norm.weight")

    def forward(self, x, ctx, cache):
        s = self.spec
        nh, nkv, d = s.n_heads, s.n_kv_heads, s.head_dim
        q, q_stride = self.rt.attention_in(x, self.wqkv, self.bqkv, self.q_norm, self.k_norm,
                                           s.qk_norm.eps if s.qk_norm is not None else 1.0, self.position, ctx,
                                           cache, nh, nkv, d)
        o = self.rt.attention(q, q_stride, cache, ctx, s.window, self.scale, nh, nkv, d)
        return self.rt.project(o, self.wo, self.bo)


register("mixer", "attention", Attention)
