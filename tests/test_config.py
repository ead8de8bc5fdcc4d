"""The typed configuration, its errors, and the registry."""
import json

import pytest

import gesso_amd  # noqa: F401
from gesso_amd.config import (Lfm2Config, adjusted_ff_dim, architecture_of, load_config, register_architecture,
                              registered_architectures, unregister_architecture)
from gesso_amd.config.jsonio import loads_strict
from gesso_amd.errors import ConfigError
from gesso_amd.models.lfm2 import lfm2_spec
from gesso_amd.models.model import tensor_table

BASE = {
    "architectures": ["Lfm2ForCausalLM"], "model_type": "lfm2", "vocab_size": 65536, "hidden_size": 2048,
    "num_hidden_layers": 16, "num_attention_heads": 32, "num_key_value_heads": 8,
    "full_attn_idxs": [2, 5, 8, 10, 12, 14], "conv_L_cache": 3, "conv_bias": False, "block_ff_dim": 12288,
    "block_auto_adjust_ff_dim": True, "block_multiple_of": 256, "block_ffn_dim_multiplier": 1.0, "norm_eps": 1e-5,
    "rope_theta": 1000000.0, "tie_word_embeddings": True, "max_position_embeddings": 128000, "eos_token_id": 7,
    "bos_token_id": 1, "pad_token_id": 0, "block_dim": 2048, "conv_dim": 2048, "conv_dim_out": 2048,
    "num_heads": 32, "theta": 1000000.0, "block_norm_eps": 1e-5, "block_use_swiglu": True, "use_pos_enc": True,
    "torch_dtype": "bfloat16", "use_cache": True, "initializer_range": 0.02,
}


def test_ff_dim_adjustment_examples():
    # the three model sizes of the benchmark description
    assert adjusted_ff_dim(12288, 256, 1.0) == 8192
    assert adjusted_ff_dim(6656, 256, 1.0) == 4608
    assert adjusted_ff_dim(10752, 256, 1.0) == 7168
    assert adjusted_ff_dim(12288, 256, None) == 8192
    assert adjusted_ff_dim(300, 7, 1.0) == 203


def test_full_config_parses():
    c = Lfm2Config.from_dict(BASE)
    assert c.intermediate_size == 8192 and c.head_dim == 64
    assert [i for i, t in enumerate(c.layer_types) if t == "full_attention"] == [2, 5, 8, 10, 12, 14]
    assert c.eos_token_id == 7
    again = Lfm2Config.from_dict(c.to_json())
    assert again == c
    spec = lfm2_spec(c)
    assert len(spec.blocks) == 16 and spec.blocks[2].mixer.kind == "attention" and spec.blocks[0].mixer.kind == "short_conv"
    assert spec.blocks[2].mixer.position.theta == 1e6 and spec.blocks[0].mixer.width == 3
    assert spec.eos_token_ids == (7,)
    table = tensor_table(spec)
    assert table["model.layers.2.self_attn.k_proj.weight"].shape == (512, 2048)
    assert table["model.layers.0.conv.conv.weight"].shape == (2048, 1, 3)
    assert table["model.layers.0.feed_forward.w2.weight"].shape == (2048, 8192)
    assert "lm_head.weight" not in table
    n = sum(int(__import__("math").prod(t.shape)) for t in table.values())
    assert n == 1_170_340_608


def test_layer_types_and_idxs_agree():
    raw = dict(BASE)
    raw["layer_types"] = ["full_attention" if i in BASE["full_attn_idxs"] else "conv" for i in range(16)]
    assert Lfm2Config.from_dict(raw) == Lfm2Config.from_dict(BASE)
    del raw["full_attn_idxs"]
    assert Lfm2Config.from_dict(raw).layer_types == Lfm2Config.from_dict(BASE).layer_types
    raw["full_attn_idxs"] = [0]
    with pytest.raises(ConfigError, match="disagree"):
        Lfm2Config.from_dict(raw)


def test_the_feed_forward_width_under_either_name():
    """``intermediate_size`` is another name of ``block_ff_dim``: the width before the adjustment, which applies while
    ``block_auto_adjust_ff_dim`` is true or left out.  A direct width needs ``block_auto_adjust_ff_dim: false``."""
    bare = {k: v for k, v in BASE.items() if not k.startswith("block_ff") and k not in
            ("block_auto_adjust_ff_dim", "block_multiple_of")}
    # a file as newer writers serialise LFM2-1.2B: the width before the adjustment under intermediate_size
    for extra in ({}, {"block_auto_adjust_ff_dim": True}, {"block_auto_adjust_ff_dim": True, "block_multiple_of": 256,
                                                           "block_ffn_dim_multiplier": 1.0}):
        c = Lfm2Config.from_dict(dict(bare, intermediate_size=12288, **extra))
        assert c.intermediate_size == 8192 and c.block_ff_dim == 12288, extra
        assert Lfm2Config.from_dict(c.to_json()) == c
    assert Lfm2Config.from_dict(dict(bare, intermediate_size=6656)).intermediate_size == 4608
    assert Lfm2Config.from_dict(dict(bare, intermediate_size=10752)).intermediate_size == 7168
    # a direct width, said to be one
    c = Lfm2Config.from_dict(dict(bare, intermediate_size=1000, block_auto_adjust_ff_dim=False))
    assert c.intermediate_size == 1000
    assert Lfm2Config.from_dict(dict(BASE, block_auto_adjust_ff_dim=False)).intermediate_size == 12288
    # both names in one file: equal (the alias), or the adjusted width beside block_ff_dim; anything else is refused
    assert Lfm2Config.from_dict(dict(BASE, intermediate_size=12288)).intermediate_size == 8192
    assert Lfm2Config.from_dict(dict(BASE, intermediate_size=8192)).intermediate_size == 8192
    with pytest.raises(ConfigError, match="neither"):
        Lfm2Config.from_dict(dict(BASE, intermediate_size=8000))
    # the multiplier scales before the rounding; without one (null) two thirds stand as they are
    assert Lfm2Config.from_dict(dict(bare, intermediate_size=1000, block_ffn_dim_multiplier=1.3,
                                     block_multiple_of=7)).intermediate_size == 868
    assert Lfm2Config.from_dict(dict(bare, intermediate_size=1000, block_ffn_dim_multiplier=None)).intermediate_size == 666
    with pytest.raises(ConfigError, match="block_ff_dim or intermediate_size"):
        Lfm2Config.from_dict(bare)


def test_a_configuration_built_with_a_direct_width_is_written_so_that_any_reader_keeps_it():
    """``Lfm2Config(intermediate_size=192)`` means a SwiGLU of 192; its config.json says so with
    ``block_auto_adjust_ff_dim: false``, and reading it back gives 192 again (a reader that adjusted it would build a
    model whose weights do not fit the file's)."""
    c = Lfm2Config(vocab_size=256, hidden_size=64, num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2,
                   layer_types=("conv", "full_attention"), conv_L_cache=3, conv_bias=False, intermediate_size=192,
                   norm_eps=1e-5, rope_theta=1e4, tie_word_embeddings=True, max_position_embeddings=256)
    raw = c.to_json()
    assert raw["intermediate_size"] == 192 and raw["block_auto_adjust_ff_dim"] is False and "block_ff_dim" not in raw
    assert Lfm2Config.from_dict(raw).intermediate_size == 192
    assert tensor_table(lfm2_spec(Lfm2Config.from_dict(raw)))["model.layers.0.feed_forward.w1.weight"].shape == (192, 64)


@pytest.mark.parametrize("change,match", [
    ({"num_key_value_heads": 5}, "multiple of num_key_value_heads"),
    ({"hidden_size": 2050, "block_dim": 2050, "conv_dim": 2050, "conv_dim_out": 2050}, "multiple of num_attention_heads"),
    ({"conv_L_cache": 1}, "at least 2"),
    ({"full_attn_idxs": [2, 16]}, "names layer 16"),
    ({"full_attn_idxs": [2, 2]}, "twice"),
    ({"norm_eps": 0.0}, "norm_eps"),
    ({"rope_theta": -1.0, "theta": -1.0}, "rope_theta"),
    ({"vocab_size": 0}, "vocab_size"),
    ({"sliding_window": 128}, "sliding_window"),
    ({"rope_scaling": {"type": "linear"}}, "rope_scaling"),
    ({"num_experts": 8}, "num_experts"),
    ({"some_new_key": 1}, "some_new_key"),
    ({"block_dim": 1024}, "block_dim"),
    ({"block_use_swiglu": False}, "block_use_swiglu"),
    ({"eos_token_id": 70000}, "eos_token_id"),
    ({"vocab_size": "many"}, "vocab_size"),
    ({"tie_embedding": False}, "disagree"),
])
def test_malformed_fields_raise(change, match):
    with pytest.raises(ConfigError, match=match):
        Lfm2Config.from_dict(dict(BASE, **change))


@pytest.mark.parametrize("key", ["vocab_size", "hidden_size", "num_hidden_layers", "num_attention_heads",
                                 "num_key_value_heads"])
def test_required_keys(key):
    raw = dict(BASE)
    del raw[key]
    with pytest.raises(ConfigError, match=key):
        Lfm2Config.from_dict(raw)


def test_keys_that_may_be_left_out_take_the_published_defaults():
    raw = dict(BASE)
    for key in ("conv_L_cache", "norm_eps", "rope_theta", "max_position_embeddings", "block_multiple_of",
                "block_auto_adjust_ff_dim", "block_ffn_dim_multiplier"):
        raw.pop(key, None)
    c = Lfm2Config.from_dict(raw)
    assert (c.conv_L_cache, c.norm_eps, c.rope_theta, c.max_position_embeddings) == (3, 1e-5, 1e6, 128000)
    assert c.intermediate_size == 8192                      # 12288 -> two thirds -> up to a multiple of 256


def test_keys_that_say_nothing_about_the_arithmetic_are_passed_over():
    """What a serialized configuration carries whatever the architecture (output switches, generation defaults, a
    writer's private notes) is no LFM2 feature and no error; a key nobody knows still is."""
    c = Lfm2Config.from_dict({**BASE, "return_dict": True, "output_attentions": False, "temperature": 1.0, "top_p": 0.9,
                              "id2label": {"0": "a"}, "_private_note": "x", "seed": 3, "init_std": 0.02})
    assert c == Lfm2Config.from_dict(BASE)
    for key in ("rope_thetta", "quantization_config", "num_experts"):
        with pytest.raises(ConfigError, match=key):
            Lfm2Config.from_dict({**BASE, key: 1})


def test_other_spellings_of_the_same_facts():
    raw = dict(BASE)
    eps = raw.pop("norm_eps")
    theta = raw.pop("rope_theta")
    raw.update(rms_norm_eps=eps, rope_parameters={"rope_type": "default", "rope_theta": theta}, head_dim=64,
               hidden_act="silu")
    c = Lfm2Config.from_dict(raw)
    assert c.norm_eps == eps and c.rope_theta == theta
    with pytest.raises(ConfigError, match="head_dim"):
        Lfm2Config.from_dict(dict(BASE, head_dim=32))
    with pytest.raises(ConfigError, match="disagree"):
        Lfm2Config.from_dict(dict(BASE, rms_norm_eps=BASE["norm_eps"] * 2))
    with pytest.raises(ConfigError, match="rope_parameters"):
        Lfm2Config.from_dict(dict(BASE, rope_parameters={"rope_type": "yarn", "factor": 4.0}))
    with pytest.raises(ConfigError, match="hidden_act"):
        Lfm2Config.from_dict(dict(BASE, hidden_act="gelu"))


def test_layer_list_length_and_kinds():
    raw = dict(BASE)
    del raw["full_attn_idxs"]
    raw["layer_types"] = ["conv"] * 15
    with pytest.raises(ConfigError, match="one entry per layer"):
        Lfm2Config.from_dict(raw)
    raw["layer_types"] = ["conv"] * 15 + ["sliding_attention"]
    with pytest.raises(ConfigError, match="sliding_attention"):
        Lfm2Config.from_dict(raw)
    del raw["layer_types"]
    with pytest.raises(ConfigError, match="layer_types or full_attn_idxs"):
        Lfm2Config.from_dict(raw)


def test_odd_head_width():
    raw = dict(BASE, hidden_size=96, num_attention_heads=32, num_heads=32, num_key_value_heads=8, block_dim=96,
               conv_dim=96, conv_dim_out=96)
    with pytest.raises(ConfigError, match="even"):
        Lfm2Config.from_dict(raw)


def test_duplicate_json_keys_are_refused():
    with pytest.raises(ConfigError, match="duplicate key 'a'"):
        loads_strict('{"a": 1, "b": {"c": 2}, "a": 3}')
    with pytest.raises(ConfigError, match="JSON object"):
        loads_strict("[1, 2]")


def test_registry(tmp_path):
    assert "Lfm2ForCausalLM" in registered_architectures()
    with pytest.raises(ConfigError, match="unknown architecture 'NoSuchModel'") as e:
        architecture_of({"architectures": ["NoSuchModel"]})
    assert "Lfm2ForCausalLM" in str(e.value)
    with pytest.raises(ConfigError, match=r"architectures\[0\]"):
        architecture_of({"model_type": "lfm2"})
    (tmp_path / "config.json").write_text(json.dumps(BASE))
    arch, cfg = load_config(str(tmp_path))
    assert arch.name == "Lfm2ForCausalLM" and cfg.hidden_size == 2048
    with pytest.raises(ConfigError, match="already registered"):
        register_architecture("Lfm2ForCausalLM", None, None, None)
    register_architecture("ToyForTests", lambda raw: raw, lambda c: None, lambda c: c)
    try:
        assert architecture_of({"architectures": ["ToyForTests"]}).name == "ToyForTests"
    finally:
        unregister_architecture("ToyForTests")


def test_schedule_is_checked():
    from gesso_amd.config import LayerCall
    c = Lfm2Config.from_dict(BASE)
    spec = lfm2_spec(c)
    import dataclasses
    with pytest.raises(ValueError, match="names block 99"):
        dataclasses.replace(spec, schedule=(LayerCall(99),))
    with pytest.raises(ValueError, match="does not run before"):
        dataclasses.replace(spec, schedule=(LayerCall(0, cache=0),))
    ok = dataclasses.replace(spec, schedule=(LayerCall(2), LayerCall(2), LayerCall(5, cache=0)))
    assert len(ok.schedule) == 3


def test_the_benchmark_says_so_and_exits_with_2_when_asked_for_more_than_one_gpu():
    """The measurement's contract: one line and exit status 2 for N > 1, before anything touches a GPU."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    p = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       timeout=120)
    assert p.returncode == 2
    assert len(p.stdout.strip().splitlines()) == 1 and "one GPU" in p.stdout
