"""A block: how a mixer, a feed-forward and their norms are arranged around the residual stream.

``prenorm``: ``h += mixer(norm_a(h)); h += ffn(norm_b(h))`` (reference
``src/Inference/Inference.jl:270-363``).  Each add is folded into the norm that follows it;
the model adds what is still pending after the last block.  A sub-layer may return a tensor or a
deferred product (its last projection, computed straight into the stream).  Another arrangement (post-norms on
sub-layer outputs, a parallel block) is another class registered under another kind.
"""
from __future__ import annotations

from .base import Part, sub_tensors
from .registry import build, part_class, register


class PreNormBlock(Part):
    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        self.mixer_norm = build("norm", spec.mixer_norm, rt)
        self.mixer = build("mixer", spec.mixer, rt)
        self.ffn = self.ffn_norm = None
        if spec.ffn is not None:
            self.ffn_norm = build("norm", spec.ffn_norm, rt)
            self.ffn = build("ffn", spec.ffn, rt)

    @staticmethod
    def tensor_specs(spec):
        out = {}
        roles = [("mixer_norm", "norm", spec.mixer_norm), ("mixer", "mixer", spec.mixer)]
        if spec.ffn is not None:
            roles += [("ffn_norm", "norm", spec.ffn_norm), ("ffn", "ffn", spec.ffn)]
        for role, category, sub in roles:
            for name, ts in part_class(category, sub).tensor_specs(sub).items():
                out[f"{role}.{name}"] = ts
        return out

    @staticmethod
    def cache_need(spec):
        cls = part_class("mixer", spec.mixer)
        return cls.cache_need(spec.mixer) if hasattr(cls, "cache_need") else None

    def bind(self, tensors):
        self.mixer_norm.bind(sub_tensors(tensors, "mixer_norm"))
        self.mixer.bind(sub_tensors(tensors, "mixer"))
        if self.ffn is not None:
            self.ffn_norm.bind(sub_tensors(tensors, "ffn_norm"))
            self.ffn.bind(sub_tensors(tensors, "ffn"))

    @property
    def first_norm(self):
        """The norm that reads the stream first when this block runs (a hint for whoever writes the stream before)."""
        return self.mixer_norm

    def forward(self, stream, ctx, cache):
        after, rt = stream.following, self.rt
        with rt.stage("norm"):
            x = self.mixer_norm.add_norm(stream)
        # a stage per kind of mixer (the profiler's names: conv_mixer, attn_mixer, ...); a sub-layer's last product
        # runs inside push, straight into the stream, and belongs to its stage
        with rt.stage(getattr(self.mixer, "stage", "mixer")):
            out = self.mixer.forward(x, ctx, cache)
            with rt.stage(getattr(self.mixer, "out_stage", "mixer_out")):
                stream.push(out, rt, next_norm=self.ffn_norm if self.ffn is not None else after)
        if self.ffn is not None:
            with rt.stage("norm"):
                x = self.ffn_norm.add_norm(stream)
            with rt.stage(getattr(self.ffn, "stage", "ffn")):
                out = self.ffn.forward(x, ctx)
                with rt.stage(getattr(self.ffn, "out_stage", "ffn_out")):
                    stream.push(out, rt, next_norm=after)

    @property
    def portions_recordable(self) -> bool:
        """Whether a step of prompt portions through this block may be recorded for replay (see ``Model``)."""
        parts = [self.mixer_norm, self.mixer] + ([self.ffn_norm, self.ffn] if self.ffn is not None else [])
        return all(getattr(p, "portions_recordable", False) for p in parts)

    def replay_key(self, q_lens, max_kv_len):
        f = getattr(self.mixer, "replay_key", None)
        return f(q_lens, max_kv_len) if f is not None else None

    @property
    def graph_safe(self) -> bool:
        """Whether a step through this block may be recorded into a HIP graph (no host round trips inside)."""
        parts = [self.mixer_norm, self.mixer] + ([self.ffn_norm, self.ffn] if self.ffn is not None else [])
        return all(getattr(p, "graph_safe", False) for p in parts)


register("block", "prenorm", PreNormBlock)
