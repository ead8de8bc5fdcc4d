"""Weights by name: what is read, in which width, and the one error that lists all faults."""
import json
import os
import struct

import pytest
import torch

import gesso_amd  # noqa: F401
from gesso_amd.errors import WeightError
from gesso_amd.models.lfm2 import lfm2_spec
from gesso_amd.models.model import tensor_table, tied_aliases
from gesso_amd.weights import (SafetensorsFile, held_dtype, load_tensors, random_tensors, write_model_folder,
                               write_safetensors)
from tiny import STD, TINY_A, TINY_B


def folder(tmp_path, cfg=TINY_A, dtype=torch.bfloat16, seed=0):
    return write_model_folder(str(tmp_path / "m"), cfg, seed, dtype, std=STD)


def load(d, cfg=TINY_A, mode=torch.bfloat16):
    spec = lfm2_spec(cfg)
    return load_tensors(d, tensor_table(spec), mode, "cpu", aliases=tied_aliases(spec),
                        ignored_suffixes=spec.ignored_tensors)


def rewrite(d, change):
    """Load all tensors of the folder's file, let `change` edit the dict, write it back."""
    f = SafetensorsFile(os.path.join(d, "model.safetensors"))
    tensors = {n: f.tensor(n).clone() for n in f.names()}
    f.close()
    change(tensors)
    write_safetensors(os.path.join(d, "model.safetensors"), tensors)


def test_round_trip_and_widths(tmp_path):
    d = folder(tmp_path)
    t = load(d)
    spec = lfm2_spec(TINY_A)
    assert set(t) == set(tensor_table(spec))
    assert t["model.embed_tokens.weight"].dtype == torch.bfloat16           # matrices keep bfloat16
    assert t["model.layers.0.operator_norm.weight"].dtype == torch.float32  # small vectors are widened, exactly
    assert t["model.layers.0.conv.conv.weight"].dtype == torch.float32
    t32 = load(d, mode=torch.float32)
    assert all(v.dtype == torch.float32 for v in t32.values())
    assert torch.equal(t32["model.embed_tokens.weight"], t["model.embed_tokens.weight"].float())
    # the plain reader (the safetensors package) sees the same bytes
    from safetensors import safe_open
    with safe_open(os.path.join(d, "model.safetensors"), framework="pt") as f:
        assert set(f.keys()) == set(t)
        assert torch.equal(f.get_tensor("model.layers.1.self_attn.q_proj.weight"), t["model.layers.1.self_attn.q_proj.weight"])


def test_a_tensor_stored_in_32_bit_stays_so(tmp_path):
    d = folder(tmp_path)
    rewrite(d, lambda t: t.__setitem__("model.layers.1.self_attn.q_proj.weight",
                                       t["model.layers.1.self_attn.q_proj.weight"].float() + 1e-4))
    t = load(d)
    assert t["model.layers.1.self_attn.q_proj.weight"].dtype == torch.float32
    assert t["model.layers.1.self_attn.k_proj.weight"].dtype == torch.bfloat16
    assert held_dtype(torch.float16, "matrix", torch.bfloat16) == torch.float32
    assert held_dtype(torch.int64, "table", torch.bfloat16) == torch.int32


def test_axes_of_length_one_may_be_stored_or_left_out(tmp_path):
    d = folder(tmp_path)
    want = load(d)["model.layers.0.conv.conv.weight"]
    assert want.shape == (64, 1, 3)
    rewrite(d, lambda t: t.__setitem__("model.layers.0.conv.conv.weight", t["model.layers.0.conv.conv.weight"].reshape(64, 3)))
    got = load(d)["model.layers.0.conv.conv.weight"]
    assert got.shape == (64, 1, 3) and torch.equal(got, want)


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    d = folder(tmp_path)

    def change(t):
        del t["model.layers.0.conv.in_proj.weight"]
        del t["model.embedding_norm.weight"]
        t["model.layers.9.stray.weight"] = torch.zeros(2)
        t["model.layers.1.self_attn.k_proj.weight"] = torch.zeros(64, 64, dtype=torch.bfloat16)
        t["model.layers.2.ffn_norm.weight"] = torch.zeros(64, dtype=torch.int32)

    rewrite(d, change)
    with pytest.raises(WeightError) as e:
        load(d)
    msg = str(e.value)
    for needle in ("2 missing", "model.layers.0.conv.in_proj.weight", "model.embedding_norm.weight", "1 unexpected",
                   "model.layers.9.stray.weight", "wrong shape", "model.layers.1.self_attn.k_proj.weight",
                   "(64, 64)", "(32, 64)", "unusable type", "model.layers.2.ffn_norm.weight"):
        assert needle in msg, needle
    assert e.value.detail["missing"] == ["model.embedding_norm.weight", "model.layers.0.conv.in_proj.weight"]


def test_tied_head_rules(tmp_path):
    d = folder(tmp_path)
    rewrite(d, lambda t: t.__setitem__("lm_head.weight", t["model.embed_tokens.weight"].clone()))
    load(d)                                           # present and equal: accepted
    rewrite(d, lambda t: t.__setitem__("lm_head.weight", t["model.embed_tokens.weight"] * 2))
    with pytest.raises(WeightError, match="differs"):
        load(d)
    d2 = write_model_folder(str(tmp_path / "b"), TINY_B, 1, torch.bfloat16, std=STD)
    rewrite(d2, lambda t: t.pop("lm_head.weight"))
    with pytest.raises(WeightError, match="lm_head.weight"):
        load(d2, TINY_B)                              # untied without its head: missing


def test_ignored_buffers(tmp_path):
    d = folder(tmp_path)
    rewrite(d, lambda t: t.__setitem__("model.layers.1.self_attn.rotary_emb.inv_freq", torch.zeros(8)))
    load(d)


def test_random_weights_are_seeded_and_distributed(tmp_path):
    table = tensor_table(lfm2_spec(TINY_B))
    a, b, c = (random_tensors(table, s, torch.float32) for s in (5, 5, 6))
    assert all(torch.equal(a[k], b[k]) for k in a) and not torch.equal(a["lm_head.weight"], c["lm_head.weight"])
    w = a["lm_head.weight"]
    assert abs(float(w.mean())) < 2e-3 and abs(float(w.std()) - 0.02) < 2e-3
    n = a["model.layers.0.operator_norm.weight"]
    assert abs(float(n.mean()) - 1.0) < 0.02
    assert "model.layers.1.conv.in_proj.bias" in a and a["model.layers.1.conv.conv.weight"].shape == (96, 1, 4)
    # the bfloat16 folder is the rounding of the float32 one
    d32 = write_model_folder(str(tmp_path / "f"), TINY_B, 1, torch.float32)
    d16 = write_model_folder(str(tmp_path / "h"), TINY_B, 1, torch.bfloat16)
    t32, t16 = load(d32, TINY_B, torch.float32), load(d16, TINY_B, torch.float32)
    assert torch.equal(t32["lm_head.weight"].bfloat16().float(), t16["lm_head.weight"])
    assert json.load(open(os.path.join(d32, "config.json")))["architectures"] == ["Lfm2ForCausalLM"]


def _raw_file(path, header: dict, data: bytes, hlen=None):
    blob = json.dumps(header).encode()
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(blob) if hlen is None else hlen))
        f.write(blob)
        f.write(data)


def test_file_integrity(tmp_path):
    p = str(tmp_path / "x.safetensors")
    ok = {"a": {"dtype": "F32", "shape": [2], "data_offsets": [0, 8]}, "b": {"dtype": "BF16", "shape": [2, 2], "data_offsets": [8, 16]}}
    _raw_file(p, ok, b"\0" * 16)
    f = SafetensorsFile(p)
    assert f.shape("b") == (2, 2) and f.tensor("b").dtype == torch.bfloat16
    f.close()
    cases = {
        "outside the file": lambda: _raw_file(p, ok, b"\0" * 16, hlen=10 ** 9),
        "trailing bytes": lambda: _raw_file(p, ok, b"\0" * 20),
        "needs 8": lambda: _raw_file(p, dict(ok, a={"dtype": "F32", "shape": [2], "data_offsets": [0, 6]}), b"\0" * 16),
        "overlap": lambda: _raw_file(p, dict(ok, b={"dtype": "BF16", "shape": [2, 2], "data_offsets": [4, 12]}), b"\0" * 12),
        "belong to no tensor": lambda: _raw_file(p, dict(ok, b={"dtype": "BF16", "shape": [2, 2], "data_offsets": [12, 20]}), b"\0" * 20),
        "unsupported dtype": lambda: _raw_file(p, dict(ok, a={"dtype": "F8_E4M3", "shape": [8], "data_offsets": [0, 8]}), b"\0" * 16),
    }
    for match, make in cases.items():
        make()
        with pytest.raises(WeightError, match=match):
            SafetensorsFile(p)
    with open(p, "wb") as fh:
        fh.write(struct.pack("<Q", 30) + b'{"a": 1, "a": 2}              ')
    with pytest.raises(WeightError, match="duplicate"):
        SafetensorsFile(p)


def test_shards(tmp_path):
    d = folder(tmp_path)
    f = SafetensorsFile(os.path.join(d, "model.safetensors"))
    names = f.names()
    half = len(names) // 2
    parts = {"model-00001-of-00002.safetensors": names[:half], "model-00002-of-00002.safetensors": names[half:]}
    for fn, ns in parts.items():
        write_safetensors(os.path.join(d, fn), {n: f.tensor(n).clone() for n in ns})
    whole = {n: f.tensor(n).clone() for n in names}
    f.close()
    os.remove(os.path.join(d, "model.safetensors"))
    with open(os.path.join(d, "model.safetensors.index.json"), "w") as fh:
        json.dump({"weight_map": {n: fn for fn, ns in parts.items() for n in ns}}, fh)
    t = load(d)
    assert torch.equal(t["model.embed_tokens.weight"], whole["model.embed_tokens.weight"])
    os.remove(os.path.join(d, "model.safetensors.index.json"))
    with pytest.raises(WeightError, match="neither"):
        load(d)
