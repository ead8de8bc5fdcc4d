"""Typed configuration of LFM2 (dense), read from the architecture's own config.json keys.

The reference reads the same facts from GGUF metadata (``src/Inference/lfm2.jl:32-152``):
an unknown key is an error that names the key (``:43-47``), the head width must satisfy
``heads * head_dim == hidden`` (``:63-65``), partial rotary, sliding windows without a
pattern and per-layer scalars are refused (``:66-86``), the short convolution's cache
length must exceed one (``src/Inference/architecture_spec.jl:175``).  The HF-style keys,
``layer_types`` / ``full_attn_idxs`` and the ``block_ff_dim`` adjustment have no reader in
the reference and follow the architecture's published config.json.

The feed-forward width.  The reference's metadata carries the width the SwiGLU really has
(``feed_forward_length``, ``src/Inference/lfm2.jl:145``).  A config.json carries the width *before* the
architecture's adjustment, under ``block_ff_dim`` or, in files serialised by newer writers, under
``intermediate_size`` (one is an alias of the other); while ``block_auto_adjust_ff_dim`` is true, which
it is when the file leaves it out, the SwiGLU has two thirds of it, scaled by
``block_ffn_dim_multiplier`` and rounded up to ``block_multiple_of``.  A file that means its
``intermediate_size`` as the SwiGLU's own width says ``block_auto_adjust_ff_dim: false``;
:meth:`Lfm2Config.to_json` writes that for a configuration built with a direct width.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Optional, Tuple

from ..errors import ConfigError

CONV = "conv"
FULL_ATTENTION = "full_attention"

# Keys that describe initialisation, provenance or runtime defaults: read by nobody here.
_IGNORED = frozenset({
    "model_type", "torch_dtype", "dtype", "transformers_version", "use_cache",
    "initializer_range", "block_mlp_init_scale", "block_out_init_scale",
    "block_use_xavier_init", "conv_use_xavier_init", "_name_or_path",
    # where random weights came from
    "seed", "init_seed", "weights_seed", "std", "init_std", "name", "description", "comment",
    # what a serialized configuration carries whatever the architecture: output switches, generation defaults,
    # labels, tokenizer hints.  None of them describes the model's arithmetic.
    "return_dict", "output_hidden_states", "output_attentions", "torchscript", "use_bfloat16", "tf_legacy_loss",
    "pruned_heads", "chunk_size_feed_forward", "is_encoder_decoder", "is_decoder", "cross_attention_hidden_size",
    "add_cross_attention", "tie_encoder_decoder", "max_length", "min_length", "do_sample", "early_stopping",
    "num_beams", "num_beam_groups", "diversity_penalty", "temperature", "top_k", "top_p", "typical_p",
    "repetition_penalty", "length_penalty", "no_repeat_ngram_size", "encoder_no_repeat_ngram_size", "bad_words_ids",
    "num_return_sequences", "output_scores", "return_dict_in_generate", "forced_bos_token_id", "forced_eos_token_id",
    "remove_invalid_values", "exponential_decay_length_penalty", "suppress_tokens", "begin_suppress_tokens",
    "finetuning_task", "id2label", "label2id", "tokenizer_class", "prefix", "sep_token_id", "decoder_start_token_id",
    "task_specific_params", "problem_type", "attn_implementation", "auto_map", "chat_template",
})
# Keys that repeat another key or state a fixed property; they must agree with it.
_MUST_EQUAL = {
    "block_dim": "hidden_size", "conv_dim": "hidden_size", "conv_dim_out": "hidden_size",
    "num_heads": "num_attention_heads", "theta": "rope_theta", "block_norm_eps": "norm_eps",
}
_MUST_BE_TRUE = ("block_use_swiglu", "use_pos_enc")
# Features of other members of the family that dense LFM2 does not have (lfm2.jl:1-15).
_REFUSED = ("sliding_window", "sliding_window_pattern", "rope_scaling", "rope_freq_factors",
            "num_experts", "num_local_experts", "num_experts_per_tok", "moe_intermediate_size",
            "attention_bias", "partial_rotary_factor", "attention_dropout")
# The architecture's published defaults for keys a config.json may leave out.
DEFAULTS = {"conv_L_cache": 3, "norm_eps": 1e-5, "rope_theta": 1000000.0, "max_position_embeddings": 128000,
            "block_auto_adjust_ff_dim": True, "block_multiple_of": 256, "block_ffn_dim_multiplier": 1.0}
_KNOWN = frozenset({
    "architectures", "vocab_size", "hidden_size", "num_hidden_layers", "num_attention_heads",
    "num_key_value_heads", "layer_types", "full_attn_idxs", "conv_L_cache", "conv_bias",
    "block_ff_dim", "block_auto_adjust_ff_dim", "block_multiple_of", "block_ffn_dim_multiplier",
    "intermediate_size", "norm_eps", "rope_theta", "tie_word_embeddings", "tie_embedding",
    "max_position_embeddings", "eos_token_id", "bos_token_id", "pad_token_id",
    "head_dim", "rms_norm_eps", "rope_parameters", "hidden_act",
}) | _IGNORED | frozenset(_MUST_EQUAL) | frozenset(_MUST_BE_TRUE) | frozenset(_REFUSED)


def adjusted_ff_dim(block_ff_dim: int, multiple_of: int, multiplier: Optional[float]) -> int:
    """Width of the SwiGLU: two thirds of ``block_ff_dim``; with a multiplier, scaled by it and rounded up to
    ``multiple_of`` (without one, two thirds and nothing more)."""
    ff = int(2 * block_ff_dim / 3)
    if multiplier is not None:
        ff = int(multiplier * ff)
        ff = multiple_of * ((ff + multiple_of - 1) // multiple_of)
    return ff


@dataclass(frozen=True)
class Lfm2Config:
    vocab_size: int
    hidden_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    layer_types: Tuple[str, ...]
    conv_L_cache: int
    conv_bias: bool
    intermediate_size: int              # the SwiGLU width actually used
    norm_eps: float
    rope_theta: float
    tie_word_embeddings: bool
    max_position_embeddings: int
    eos_token_id: Optional[int] = None
    bos_token_id: Optional[int] = None
    pad_token_id: Optional[int] = None
    # how intermediate_size was given, kept so that to_json() writes the same keys back
    block_ff_dim: Optional[int] = None
    block_multiple_of: Optional[int] = None
    block_ffn_dim_multiplier: Optional[float] = None

    @property
    def head_dim(self) -> int:
        return self.hidden_size // self.num_attention_heads

    def __post_init__(self):
        c = self
        for name in ("vocab_size", "hidden_size", "num_hidden_layers", "num_attention_heads",
                     "num_key_value_heads", "intermediate_size", "max_position_embeddings"):
            v = getattr(c, name)
            if not (isinstance(v, int) and not isinstance(v, bool) and v > 0):
                raise ConfigError(f"{name} must be a positive integer, found {v!r}", key=name)
        if c.hidden_size % c.num_attention_heads:
            raise ConfigError("hidden_size must be a multiple of num_attention_heads "
                              "(attention width equals the hidden width)",
                              hidden_size=c.hidden_size, num_attention_heads=c.num_attention_heads)
        if c.num_attention_heads % c.num_key_value_heads:
            raise ConfigError("num_attention_heads must be a multiple of num_key_value_heads",
                              num_attention_heads=c.num_attention_heads,
                              num_key_value_heads=c.num_key_value_heads)
        if c.head_dim % 2:
            raise ConfigError("the head width must be even for half-split rotation", head_dim=c.head_dim)
        if not (isinstance(c.conv_L_cache, int) and c.conv_L_cache >= 2):
            raise ConfigError("conv_L_cache must be at least 2", conv_L_cache=c.conv_L_cache)
        if len(c.layer_types) != c.num_hidden_layers:
            raise ConfigError("layer_types must have one entry per layer",
                              entries=len(c.layer_types), num_hidden_layers=c.num_hidden_layers)
        for i, t in enumerate(c.layer_types):
            if t not in (CONV, FULL_ATTENTION):
                raise ConfigError(f"layer_types[{i}] = {t!r}: LFM2 has {CONV!r} and {FULL_ATTENTION!r}")
        if not (isinstance(c.norm_eps, float) and c.norm_eps > 0 and math.isfinite(c.norm_eps)):
            raise ConfigError("norm_eps must be a positive number", norm_eps=c.norm_eps)
        if not (isinstance(c.rope_theta, float) and c.rope_theta > 0 and math.isfinite(c.rope_theta)):
            raise ConfigError("rope_theta must be a positive number", rope_theta=c.rope_theta)
        for name in ("eos_token_id", "bos_token_id", "pad_token_id"):
            v = getattr(c, name)
            if v is not None and not (isinstance(v, int) and 0 <= v < c.vocab_size):
                raise ConfigError(f"{name} must lie inside the vocabulary", **{name: v})

    # ------------------------------------------------------------------ config.json

    @staticmethod
    def from_dict(raw: dict) -> "Lfm2Config":
        for key in raw:
            # (keys that start with an underscore are a writer's private notes)
            if key not in _KNOWN and not key.startswith("_"):
                raise ConfigError(f"unsupported config.json key {key!r} (no LFM2 feature declares it)", key=key)
        for key in _REFUSED:
            if raw.get(key) not in (None, False, 0):
                raise ConfigError(f"config.json asks for {key!r}, which dense LFM2 does not have", key=key)

        raw = dict(raw)
        # other spellings of the same facts: they must agree where both are given
        if "rms_norm_eps" in raw:
            if "norm_eps" in raw and raw["norm_eps"] != raw["rms_norm_eps"]:
                raise ConfigError("norm_eps and rms_norm_eps disagree")
            raw["norm_eps"] = raw.pop("rms_norm_eps")
        rp = raw.pop("rope_parameters", None)
        if rp is not None:
            if not isinstance(rp, dict) or rp.get("rope_type", "default") not in (None, "default") or \
                    set(rp) - {"rope_type", "rope_theta"}:
                raise ConfigError("rope_parameters: dense LFM2 has plain rotation only (rope_type default, rope_theta)")
            if "rope_theta" in rp:
                if "rope_theta" in raw and raw["rope_theta"] != rp["rope_theta"]:
                    raise ConfigError("rope_theta and rope_parameters.rope_theta disagree")
                raw["rope_theta"] = rp["rope_theta"]
        if raw.pop("hidden_act", "silu") != "silu":
            raise ConfigError("hidden_act: the LFM2 feed-forward is SwiGLU (silu)")

        def need(key, kind):
            if key not in raw:
                if key in DEFAULTS:
                    return DEFAULTS[key]
                raise ConfigError(f"config.json lacks the required key {key!r}", key=key)
            v = raw[key]
            if kind is float and isinstance(v, int) and not isinstance(v, bool):
                v = float(v)
            if not isinstance(v, kind) or (kind is int and isinstance(v, bool)):
                raise ConfigError(f"config.json key {key!r} must be {kind.__name__}, found {v!r}", key=key)
            return v

        n_layers = need("num_hidden_layers", int)
        has_types, has_idxs = "layer_types" in raw, "full_attn_idxs" in raw
        if not (has_types or has_idxs):
            raise ConfigError("config.json must give layer_types or full_attn_idxs")
        types = None
        if has_types:
            lt = raw["layer_types"]
            if not (isinstance(lt, list) and all(isinstance(t, str) for t in lt)):
                raise ConfigError("layer_types must be a list of strings")
            types = tuple(lt)
        if has_idxs:
            idxs = raw["full_attn_idxs"]
            if not (isinstance(idxs, list) and all(isinstance(i, int) and not isinstance(i, bool) for i in idxs)):
                raise ConfigError("full_attn_idxs must be a list of integers")
            for i in idxs:
                if not 0 <= i < n_layers:
                    raise ConfigError(f"full_attn_idxs names layer {i}, there are {n_layers}", index=i)
            if len(set(idxs)) != len(idxs):
                raise ConfigError("full_attn_idxs names a layer twice")
            from_idxs = tuple(FULL_ATTENTION if i in set(idxs) else CONV for i in range(n_layers))
            if types is not None and types != from_idxs:
                raise ConfigError("layer_types and full_attn_idxs disagree")
            types = from_idxs

        # the width before the adjustment, under either name (they must agree where a file has both; a file that
        # holds the adjusted width beside block_ff_dim, as older writers left it, is taken too)
        block_ff = mult_of = mult = None
        if "block_ff_dim" not in raw and "intermediate_size" not in raw:
            raise ConfigError("config.json lacks the feed-forward width: block_ff_dim or intermediate_size",
                              key="block_ff_dim")
        block_ff = need("block_ff_dim" if "block_ff_dim" in raw else "intermediate_size", int)
        if need("block_auto_adjust_ff_dim", bool):
            mult_of = need("block_multiple_of", int)
            if mult_of <= 0:
                raise ConfigError("block_multiple_of must be positive", block_multiple_of=mult_of)
            mult = need("block_ffn_dim_multiplier", float) if raw.get("block_ffn_dim_multiplier", 1.0) is not None else None
            ff = adjusted_ff_dim(block_ff, mult_of, mult)
        else:
            ff = block_ff
        if "block_ff_dim" in raw and "intermediate_size" in raw:
            given = need("intermediate_size", int)
            if given not in (block_ff, ff):
                raise ConfigError("intermediate_size is neither block_ff_dim nor the width adjusted from it",
                                  intermediate_size=given, block_ff_dim=block_ff, adjusted=ff)

        tie = True
        for key in ("tie_word_embeddings", "tie_embedding"):
            if key in raw:
                tie = need(key, bool)
        if "tie_word_embeddings" in raw and "tie_embedding" in raw and raw["tie_word_embeddings"] != raw["tie_embedding"]:
            raise ConfigError("tie_word_embeddings and tie_embedding disagree")

        cfg = Lfm2Config(
            vocab_size=need("vocab_size", int),
            hidden_size=need("hidden_size", int),
            num_hidden_layers=n_layers,
            num_attention_heads=need("num_attention_heads", int),
            num_key_value_heads=need("num_key_value_heads", int),
            layer_types=types,
            conv_L_cache=need("conv_L_cache", int),
            conv_bias=need("conv_bias", bool) if "conv_bias" in raw else False,
            intermediate_size=ff,
            norm_eps=need("norm_eps", float),
            rope_theta=need("rope_theta", float),
            tie_word_embeddings=tie,
            max_position_embeddings=need("max_position_embeddings", int),
            eos_token_id=raw.get("eos_token_id"),
            bos_token_id=raw.get("bos_token_id"),
            pad_token_id=raw.get("pad_token_id"),
            block_ff_dim=block_ff, block_multiple_of=mult_of, block_ffn_dim_multiplier=mult,
        )
        if raw.get("head_dim") is not None and raw["head_dim"] != cfg.head_dim:
            raise ConfigError("head_dim must equal hidden_size / num_attention_heads (the attention width is the "
                              "hidden width)", head_dim=raw["head_dim"], expected=cfg.head_dim)
        for key, other in _MUST_EQUAL.items():
            if key in raw and other in raw and raw[key] != raw[other]:
                raise ConfigError(f"config.json key {key!r} must equal {other!r}",
                                  **{key: raw[key], other: raw[other]})
        for key in _MUST_BE_TRUE:
            if key in raw and raw[key] is not True:
                raise ConfigError(f"config.json key {key!r} must be true for LFM2", key=key)
        return cfg

    def to_json(self) -> dict:
        out = {
            "architectures": ["Lfm2ForCausalLM"],
            "model_type": "lfm2",
            "vocab_size": self.vocab_size,
            "hidden_size": self.hidden_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "layer_types": list(self.layer_types),
            "conv_L_cache": self.conv_L_cache,
            "conv_bias": self.conv_bias,
            "norm_eps": self.norm_eps,
            "rope_theta": self.rope_theta,
            "tie_word_embeddings": self.tie_word_embeddings,
            "max_position_embeddings": self.max_position_embeddings,
        }
        if self.block_ff_dim is not None and self.block_multiple_of is not None:
            out["block_ff_dim"] = self.block_ff_dim
            out["block_auto_adjust_ff_dim"] = True
            out["block_multiple_of"] = self.block_multiple_of
            out["block_ffn_dim_multiplier"] = self.block_ffn_dim_multiplier
        else:
            # a direct width: said so, because a reader adjusts whatever width it finds unless told not to
            out["intermediate_size"] = self.intermediate_size
            out["block_auto_adjust_ff_dim"] = False
        for name in ("eos_token_id", "bos_token_id", "pad_token_id"):
            if getattr(self, name) is not None:
                out[name] = getattr(self, name)
        return out
