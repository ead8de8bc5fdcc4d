"""The model: an embedding table, blocks run in the order the schedule gives, a final norm, a head.

Built from a :class:`~gesso_amd.config.spec.ModelSpec` alone; which architecture the spec came
from plays no part here.  ``tensor_table`` lists every tensor the model reads, by its name in
the weight file, with the shape the spec implies (the reference's shape law,
``src/Inference/materialize_architecture.jl:31-121``).
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..config.spec import ModelSpec
from ..errors import ConfigError
from ..parts.base import MATRIX, TABLE, TensorSpec
from ..parts.registry import build, part_class
from ..parts.rmsnorm import ResidualStream, row_weight_of


def tensor_table(spec: ModelSpec) -> Dict[str, TensorSpec]:
    """``file name -> TensorSpec`` of every tensor the model must find."""
    out: Dict[str, TensorSpec] = {}

    def put(name, ts):
        if name in out and out[name] != ts:
            raise ConfigError(f"tensor {name!r} is claimed twice with different shapes")
        out[name] = ts

    put(spec.names["embed"], TensorSpec((spec.vocab, spec.hidden), TABLE))
    for local, ts in part_class("norm", spec.final_norm).tensor_specs(spec.final_norm).items():
        put(spec.names["final_norm." + local], ts)
    if not spec.tie_embeddings:
        put(spec.names["head"], TensorSpec((spec.vocab, spec.hidden), MATRIX))
    for i, b in enumerate(spec.blocks):
        for local, ts in part_class("block", b).tensor_specs(b).items():
            if local not in b.names:
                raise ConfigError(f"block {i} has no file name for its tensor {local!r}")
            put(b.names[local], ts)
    return out


def tied_aliases(spec: ModelSpec) -> Dict[str, str]:
    """Tensors a file may hold though nobody reads them, if they equal another: a tied head."""
    if spec.tie_embeddings and "head" in spec.names:
        return {spec.names["head"]: spec.names["embed"]}
    return {}


class Model:
    def __init__(self, spec: ModelSpec, rt):
        self.spec = spec
        self.rt = rt
        self.blocks = [build("block", b, rt) for b in spec.blocks]
        self.final_norm = build("norm", spec.final_norm, rt)
        self.embed = None
        self.head = None

    def cache_needs(self) -> List[Optional[object]]:
        """For each entry of the schedule: what its own cache must hold (None: none, or it reads another's)."""
        out = []
        for call in self.spec.schedule:
            b = self.spec.blocks[call.layer]
            need = part_class("block", b).cache_need(b)
            out.append(None if call.cache is not None else need)
        return out

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        s = self.spec
        self.embed = tensors[s.names["embed"]]
        self.head = self.rt.prepare(self.embed if s.tie_embeddings else tensors[s.names["head"]])
        self.final_norm.bind({k: tensors[s.names["final_norm." + k]]
                              for k in part_class("norm", s.final_norm).tensor_specs(s.final_norm)})
        for b, block in zip(s.blocks, self.blocks):
            local = {k: tensors[b.names[k]] for k in part_class("block", b).tensor_specs(b)}
            block.bind(local)

    @property
    def graph_safe(self) -> bool:
        return all(getattr(b, "graph_safe", False) for b in self.blocks) and getattr(self.final_norm, "graph_safe", False)

    def forward(self, ctx) -> Optional[torch.Tensor]:
        """Run the tokens of ``ctx`` through every scheduled block; float32 logits at ``ctx.want_rows``."""
        stream = self.run_blocks(ctx)
        if ctx.n_want == 0:
            return None
        # every row wanted, in order (a decode step): no gather, and the norm may stay lazy
        return self.logits(stream, None if ctx.decode_only else ctx.want_rows)

    def run_blocks(self, ctx) -> ResidualStream:
        """The embedding and every scheduled block: the residual stream as the last block leaves it (what is still
        pending is added by the norm that follows)."""
        rt = self.rt
        # the norm that reads the stream after the i-th scheduled block: the next block's first, then the final one
        # (``first_norm`` and ``row_weight`` are the optional hints of blocks and norms, see parts/base.py)
        order = [self.blocks[call.layer] for call in self.spec.schedule]
        readers = [getattr(b, "first_norm", None) for b in order[1:]] + [self.final_norm if ctx.decode_only else None]
        scale = 1.0 if self.spec.embed_scale is None else float(self.spec.embed_scale)
        with rt.stage("embed"):
            stream = self._embed(ctx, order, scale)
        for i, call in enumerate(self.spec.schedule):
            stream.following = readers[i]
            order[i].forward(stream, ctx, ctx.cache_view(i))
        return stream

    def logits(self, stream: ResidualStream, rows) -> torch.Tensor:
        """The final norm of the stream's ``rows`` (int32 on the device; None: all, in order) and the head: float32."""
        ops, rt = self.rt.ops, self.rt
        with rt.stage("norm"):
            normed = self.final_norm.add_norm(stream, rows=rows)
        with rt.stage("lm_head"):
            logits = self.rt.linear(normed, self.head, out_dtype=torch.float32)
            if self.spec.logit_softcap is not None:
                ops.softcap(logits, float(self.spec.logit_softcap))
        return logits

    @property
    def portions_recordable(self) -> bool:
        """Whether steps of prompt portions through this model may be recorded for replay (every part says so: what it
        launches then depends on the step's token count and on device buffers alone, or it tells the recorder)."""
        return all(getattr(b, "portions_recordable", False) for b in self.blocks) and \
            getattr(self.final_norm, "portions_recordable", False)

    def replay_key(self, q_lens, max_kv_len):
        """What a recording of a step of prompt portions must share with the step that replays it, beside the token
        count: each block's own answer (None: nothing; False from any block: such a step is not to be recorded, and
        the answer is None)."""
        key = tuple(b.replay_key(q_lens, max_kv_len) if hasattr(b, "replay_key") else None for b in self.blocks)
        return None if any(k is False for k in key) else key

    def _embed(self, ctx, order, scale):
        ops, rt = self.rt.ops, self.rt
        if rt.fused:
            ssq = torch.empty((ctx.T, 1), dtype=torch.float32, device=rt.device)
            first = getattr(order[0], "first_norm", None) if order else None
            res = torch.empty((ctx.T, self.embed.shape[1]), dtype=torch.float32, device=rt.device)
            w = row_weight_of(first, res, rt)
            xs = rt.new_rows(*res.shape) if w is not None else None
            ops.embed(ctx.token_ids, self.embed, out=res, ssq=ssq, next_weight=w, xs=xs, scale=scale)
            stream = ResidualStream(res, ssq=ssq, xs=xs, xs_for=first if xs is not None else None)
        else:
            stream = ResidualStream(ops.embed(ctx.token_ids, self.embed, scale=scale))
        return stream

