"""LFM2 (dense) as a composition of parts: configuration -> model as data.

A pre-norm decoder whose blocks hold either a gated short-convolution mixer or a
grouped-query attention mixer (per-head q/k norm, then half-split rotary), each followed
by a SwiGLU feed-forward; a final norm (``embedding_norm``) and a head that may be the
embedding table.  The reference describes the same model in ``src/Inference/lfm2.jl:154-178``
(which tensors a layer of each kind binds) and runs it in ``src/Inference/Inference.jl:270-386``.

This file holds everything that is LFM2's own: the tensor names and the way the typed
configuration fills the parts' sizes.  Another architecture is another file of this shape.
"""
from __future__ import annotations

from ..config.lfm2 import CONV, Lfm2Config
from ..config.registry import register_architecture
from ..config.spec import (AttentionSpec, BlockSpec, LayerCall, ModelSpec, RMSNormSpec, RopeSpec,
                           ShortConvSpec, SwiGLUSpec)

ARCHITECTURE = "Lfm2ForCausalLM"


def lfm2_spec(cfg: Lfm2Config) -> ModelSpec:
    H, d = cfg.hidden_size, cfg.head_dim
    norm = RMSNormSpec(size=H, eps=cfg.norm_eps)
    rope = RopeSpec(head_dim=d, rotary_dim=d, theta=cfg.rope_theta, max_position=cfg.max_position_embeddings)
    attention = AttentionSpec(hidden=H, n_heads=cfg.num_attention_heads, n_kv_heads=cfg.num_key_value_heads,
                              head_dim=d, position=rope, qk_norm=RMSNormSpec(size=d, eps=cfg.norm_eps))
    conv = ShortConvSpec(hidden=H, width=cfg.conv_L_cache, bias=cfg.conv_bias)
    ffn = SwiGLUSpec(hidden=H, intermediate=cfg.intermediate_size)

    blocks = []
    for i, kind in enumerate(cfg.layer_types):
        p = f"model.layers.{i}."
        names = {
            "mixer_norm.weight": p + "operator_norm.weight",
            "ffn_norm.weight": p + "ffn_norm.weight",
            "ffn.w1.weight": p + "feed_forward.w1.weight",
            "ffn.w3.weight": p + "feed_forward.w3.weight",
            "ffn.w2.weight": p + "feed_forward.w2.weight",
        }
        if kind == CONV:
            names.update({
                "mixer.in_proj.weight": p + "conv.in_proj.weight",
                "mixer.conv.weight": p + "conv.conv.weight",
                "mixer.out_proj.weight": p + "conv.out_proj.weight",
            })
            if cfg.conv_bias:
                names.update({
                    "mixer.in_proj.bias": p + "conv.in_proj.bias",
                    "mixer.conv.bias": p + "conv.conv.bias",
                    "mixer.out_proj.bias": p + "conv.out_proj.bias",
                })
            mixer = conv
        else:
            names.update({
                "mixer.q_proj.weight": p + "self_attn.q_proj.weight",
                "mixer.k_proj.weight": p + "self_attn.k_proj.weight",
                "mixer.v_proj.weight": p + "self_attn.v_proj.weight",
                "mixer.out_proj.weight": p + "self_attn.out_proj.weight",
                "mixer.q_norm.weight": p + "self_attn.q_layernorm.weight",
                "mixer.k_norm.weight": p + "self_attn.k_layernorm.weight",
            })
            mixer = attention
        blocks.append(BlockSpec(mixer=mixer, mixer_norm=norm, ffn=ffn, ffn_norm=norm, names=names))

    # "head" is read when the head is untied; a tied file may still hold it, equal to the table
    names = {"embed": "model.embed_tokens.weight", "final_norm.weight": "model.embedding_norm.weight",
             "head": "lm_head.weight"}
    return ModelSpec(
        architecture=ARCHITECTURE, hidden=H, vocab=cfg.vocab_size, blocks=tuple(blocks),
        schedule=tuple(LayerCall(i) for i in range(len(blocks))), final_norm=norm,
        tie_embeddings=cfg.tie_word_embeddings, max_position=cfg.max_position_embeddings, names=names,
        eos_token_ids=() if cfg.eos_token_id is None else (cfg.eos_token_id,),
        ignored_tensors=("rotary_emb.inv_freq",),
    )


register_architecture(ARCHITECTURE, Lfm2Config.from_dict, lfm2_spec, Lfm2Config.to_json)
