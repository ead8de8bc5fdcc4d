"""A model as data: the specs that parts are built from.

A :class:`ModelSpec` is what an architecture's factory makes of its typed configuration.
It lists blocks (each a mixer, a feed-forward and their norms, every size a field), the
order in which blocks run (:class:`LayerCall`, a list that may name a block twice or let a
call read the cache of an earlier call) and the names of the tensors that fill them.
Nothing below this file knows which architecture it serves.

The reference keeps the same facts in ``ArchitectureSpec``
(``src/Inference/architecture_spec.jl:218-364``), per-layer mixer kinds in
``ShortConvSpec`` (``:169-178``) and position policy in ``RoPEPolicy`` (``:47-103``).

A spec of a new part is any frozen dataclass with a ``kind`` string; the part class
registered under that kind (``gesso_amd.parts.registry``) receives it unchanged.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Mapping, Optional, Tuple


@dataclass(frozen=True)
class RMSNormSpec:
    size: int
    eps: float
    kind: str = "rmsnorm"


@dataclass(frozen=True)
class RopeSpec:
    """Rotary encoding over the first ``rotary_dim`` features of a head; ``layout``: pairs ``(i, i + rotary_dim/2)``
    (``"half"``) or ``(2i, 2i + 1)`` (``"interleaved"``)."""

    head_dim: int
    rotary_dim: int
    theta: float
    max_position: int
    layout: str = "half"
    kind: str = "rope"


@dataclass(frozen=True)
class NoPositionSpec:
    kind: str = "none"


@dataclass(frozen=True)
class AttentionSpec:
    hidden: int
    n_heads: int
    n_kv_heads: int
    head_dim: int
    position: Any                      # a position-encoding spec
    qk_norm: Optional[RMSNormSpec]     # per-head norm of q and k before the rotation
    window: Optional[int] = None       # keys a query sees, itself included; None = all
    bias: bool = False
    scale: Optional[float] = None      # None = 1/sqrt(head_dim)
    kind: str = "attention"


@dataclass(frozen=True)
class ShortConvSpec:
    hidden: int
    width: int                         # taps, the current input included (conv_L_cache)
    bias: bool = False
    kind: str = "short_conv"


@dataclass(frozen=True)
class SwiGLUSpec:
    hidden: int
    intermediate: int
    kind: str = "swiglu"


@dataclass(frozen=True)
class BlockSpec:
    """One block: ``h += mixer(norm(h)); h += ffn(norm(h))`` for ``arrangement="prenorm"``.

    ``names`` maps a part-local tensor name, prefixed by the part's role
    (``mixer.``, ``mixer_norm.``, ``ffn.``, ``ffn_norm.``), to the tensor's name in the
    weight file.
    """

    mixer: Any
    mixer_norm: Any
    ffn: Any                           # None = no feed-forward in this block
    ffn_norm: Any
    names: Mapping[str, str] = field(compare=False, hash=False, default_factory=dict)
    kind: str = "prenorm"


@dataclass(frozen=True)
class LayerCall:
    """One entry of the run order: block ``layer`` runs here.

    ``cache`` is the position in the schedule of an earlier call whose cache this call
    reads instead of keeping its own (None = its own).
    """

    layer: int
    cache: Optional[int] = None


@dataclass(frozen=True)
class ModelSpec:
    architecture: str
    hidden: int
    vocab: int
    blocks: Tuple[BlockSpec, ...]
    schedule: Tuple[LayerCall, ...]
    final_norm: Any
    tie_embeddings: bool
    max_position: int
    names: Mapping[str, str] = field(compare=False, hash=False, default_factory=dict)
    # names: "embed" -> table, "final_norm.weight" -> ..., "head" -> untied head
    eos_token_ids: Tuple[int, ...] = ()
    ignored_tensors: Tuple[str, ...] = ()   # suffixes that a file may hold and nobody reads
    embed_scale: Optional[float] = None     # the embedding rows are multiplied by this (None: as they are)
    logit_softcap: Optional[float] = None   # logits = cap * tanh(logits / cap) (None: as they are)

    def __post_init__(self):
        n = len(self.blocks)
        for i, call in enumerate(self.schedule):
            if not 0 <= call.layer < n:
                raise ValueError(f"schedule entry {i} names block {call.layer}, there are {n}")
            if call.cache is not None and not 0 <= call.cache < i:
                raise ValueError(f"schedule entry {i} reads the cache of entry {call.cache}, which does not run before it")
