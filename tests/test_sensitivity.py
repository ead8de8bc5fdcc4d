"""The bound that bfloat16 whole-model tests use must see the faults it is there for (no GPU needed).

For every tiny configuration: the rounded plain model computed another way (float32 arithmetic) lies inside the bound
of ``tests/noise.py``; the rounded plain model with one fault planted lies outside.  The faults are the plausible ones
of an engine with a cache: (a) the short convolution's history is lost at every seventh token (a portion's start that
does not read its slot), (b) the taps are applied newest to oldest, (c) a query sees one key past its own position.
The reference plants controls of this kind in its own model tests (``test/test_lfm25.jl:189-235``).
"""
import math

import pytest
import torch

import plain_lfm2 as P
from noise import NoiseBound
from tiny import CONFIGS, random_ids, write_tiny

LENGTHS = (5, 33, 70)


def history_lost(real):
    def conv(bcx, taps, bias=None, hist=None):
        outs = []
        for a in range(0, bcx.shape[0], 7):
            o, hist = real(bcx[a:a + 7], taps, bias, None)
            outs.append(o)
        return torch.cat(outs), hist
    return conv


def taps_reversed(real):
    return lambda bcx, taps, bias=None, hist=None: real(bcx, taps.flip(1), bias, hist)


def one_key_too_many(real):
    def attention(q, k, v, window=0):
        L, nh, d = q.shape
        K, nkv, _ = k.shape
        out = torch.zeros_like(q)
        for h in range(nh):
            kh = h // (nh // nkv)
            for t in range(L):
                last = min(K - 1, K - L + t + 1)
                s = (k[:last + 1, kh] @ q[t, h]) / math.sqrt(d)
                p = torch.exp(s - s.max())
                out[t, h] = (p / p.sum()) @ v[:last + 1, kh]
        return out
    return attention


FAULTS = {"history lost": ("short_conv", history_lost), "taps reversed": ("short_conv", taps_reversed),
          "one key too many": ("causal_attention", one_key_too_many)}


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    root = str(tmp_path_factory.mktemp("sens"))
    out = {}
    for name, (cfg, seed) in CONFIGS.items():
        d = write_tiny(root, name, torch.bfloat16)
        c, w = P.read_config(d), P.read_weights(d)
        seqs = [random_ids(n, cfg.vocab_size, 50 * seed + n) for n in LENGTHS]
        ref = [P.forward(c, w, s).numpy() for s in seqs]
        rounded = [P.forward(c, w, s, store=P.to_bfloat16).numpy() for s in seqs]
        out[name] = (d, c, w, seqs, ref, rounded)
    return out


def bound_of(rows, ref, rounded):
    b = NoiseBound()
    for i, (x, r, n) in enumerate(zip(rows, ref, rounded)):
        for t in range(r.shape[0]):
            b.add(x[t], r[t], n[t], (i, t))
    return b


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_the_weights_are_drawn_as_wide_as_the_tests_say(models, name):
    """``write_tiny`` asks for a standard deviation of 0.1: every sub-layer then moves the stream by a good part of
    what the stream holds (at 0.02 a convolution mixer would move it by a thousandth)."""
    from tiny import STD
    d, c, w, *_ = models[name]
    m = w["model.layers.0.feed_forward.w1.weight"]
    assert abs(float(m.std()) - STD) < 0.1 * STD
    h = P.embedding(w["model.embed_tokens.weight"], [1, 2, 3, 4, 5, 6])
    for i, kind in enumerate(c["layers"]):
        pre = f"model.layers.{i}."
        if kind == "conv":
            h2, _ = P.conv_block(h, w, pre, c["eps"])
        else:
            h2 = P.attention_block(h, w, pre, c, list(range(6)))
        moved = float((h2 - h).norm() / h.norm())
        assert moved > 0.02, (i, kind, moved)
        h = P.feed_forward_block(h2, w, pre, c["eps"])


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_another_computation_of_the_rounded_model_lies_inside_the_bound(models, name):
    d, c, w, seqs, ref, rounded = models[name]
    w32 = P.read_weights(d, torch.float32)
    other = [P.forward(c, w32, s, store=P.to_bfloat16).double().numpy() for s in seqs]
    b = bound_of(other, ref, rounded)
    print(name, b.summary())
    assert b.failures() == []


@pytest.mark.parametrize("fault", sorted(FAULTS))
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_a_planted_fault_lies_outside_the_bound(models, monkeypatch, name, fault):
    d, c, w, seqs, ref, rounded = models[name]
    attr, make = FAULTS[fault]
    monkeypatch.setattr(P, attr, make(getattr(P, attr)))
    broken = [P.forward(c, w, s, store=P.to_bfloat16).numpy() for s in seqs]
    b = bound_of(broken, ref, rounded)
    print(name, fault, b.summary())
    bad = b.failures()
    # seen by the measure over all rows, the one least given to chance, and by the worst logit
    assert any("all rows" in m for m in bad) and any("worst logit" in m for m in bad), bad
    assert b.rms > 3 * b.noise_rms
