"""The whole model at the layer sizes of LFM2-1.2B, and at long contexts, against the plain implementation.

The tiny configurations never reach the kernel variants that the real sizes select (weight-streaming products with two
and three row tiles a block, products in parts of K with their adding pass, the vendor product at hundreds of rows, the
hand-written matrix-core product for float32 logits, attention with four query heads to a key head); here they run
inside a model.  The reference checks its device path the same way, prefill and greedy decode against its oracle
(``test/test_amdgpu_lfm2.jl:151-196``, bound ``:34``), and carries keys, values and convolution state across prompt
passes (``src/Inference/Inference.jl:2272-2530``).

Layer sizes are those of LFM2-1.2B (hidden 2048, 32 query and 8 key heads of 64, feed-forward 8192, vocabulary 65536,
three taps, tied head) with 4 layers (conv, conv, attention, conv) of its 16.  One folder, stored in bfloat16, serves
both precisions (float32 widens it exactly) and the plain implementation (float64 of the same values).

What bfloat16 is held to at these sizes.  Products over 2,048 and 8,192 terms of activations rounded to 8 bits of
mantissa leave every logit with a noise of about 1.5 % of the logits' spread, whoever computes them: the plain model
with nothing but those roundings put in (``plain_lfm2.forward(..., store=to_bfloat16)``, "the rounded model") stands
7.9e-2 from the plain model at its worst logit over 300 tokens x 65,536 logits, at a scale of 5.2, root mean square
1.4e-2; the bound of the tiny configurations (1.5e-2 x scale = 7.8e-2 at the worst logit) is then a coin toss that says
nothing about the engine (its first run stood at 8.25e-2, with a root mean square below the rounded model's).  Nor can
the engine be held close to the rounded model itself: roundings are chaotic (a difference in the seventh digit flips a
rounding here and there, each flip is a difference in the third digit, and a few stages later all roundings fall
independently), so that the rounded model computed in float32 and in float64 differs from itself by 4.9e-2 at the
worst logit.  What does hold, and what a fault breaks, is that the engine's distance from the plain model is noise of
the rounded model's size, row by row.  Between two such computations of the rounded model the ratio of a row's root
mean square distances lay in 0.88 .. 1.06 over 370 rows, that of all rows together at 1.00, that of the worst logits at
0.98 .. 1.02.  The engine is held to:

* each row: rms(engine - plain) <= 1.3 x rms(rounded - plain) of the same row (a fault that moves one row by as much as
  the noise does, 1.2e-2 or 0.2 % of the scale, shows: about six times tighter than the tiny configurations' bound);
* all rows together: rms <= 1.15 x the rounded model's;
* the worst logit: <= 1.25 x the rounded model's worst.

float32 keeps the bound of the tiny configurations, 1e-4 x scale.

The other two models the benchmark times run here as well, three layers each, in the four cuttings and through the
recorded decode step: LFM2-350M's layer sizes (hidden 1024, 16 query heads on 8 key heads, feed-forward 4608) and
LFM2-2.6B's (feed-forward 7168).
"""
import dataclasses
import os

import numpy as np
import pytest
import torch

import plain_lfm2 as P
import replay as R
from tiny import TINY_D, random_ids

pytestmark = pytest.mark.gpu

TOL = {"float32": 1e-4}
# bfloat16: the engine's distance from the plain model over the rounded plain model's distance from it
ROW_NOISE_FACTOR = 1.3      # root mean square over a row
NOISE_FACTOR = 1.15         # root mean square over all rows
WORST_FACTOR = 1.25         # the worst logit
LAYERS = ("conv", "conv", "full_attention", "conv")          # 4 of the model's 16 layers
LENGTHS = (3, 70, 150, 300)


# layer sizes of the three models the benchmark times: hidden, query heads, key heads, width before the adjustment
SIZES = {"1.2B": (2048, 32, 8, 12288), "350M": (1024, 16, 8, 6656), "2.6B": (2048, 32, 8, 10752)}
WIDTHS = {"1.2B": 8192, "350M": 4608, "2.6B": 7168}


def real_size_config(size="1.2B", layers=LAYERS):
    from gesso_amd.config import Lfm2Config
    H, nh, nkv, ff = SIZES[size]
    return Lfm2Config.from_dict({
        "architectures": ["Lfm2ForCausalLM"], "vocab_size": 65536, "hidden_size": H, "num_hidden_layers": len(layers),
        "num_attention_heads": nh, "num_key_value_heads": nkv, "layer_types": list(layers), "conv_L_cache": 3,
        "conv_bias": False, "block_ff_dim": ff, "block_auto_adjust_ff_dim": True, "block_multiple_of": 256,
        "block_ffn_dim_multiplier": 1.0, "norm_eps": 1e-5, "rope_theta": 1000000.0, "tie_word_embeddings": True,
        "max_position_embeddings": 4096})


def write_real_size_folder(path: str, taps_scale: float, size="1.2B", layers=LAYERS) -> str:
    """N(0, 0.02) everywhere, as the benchmark draws its weights; ``taps_scale`` multiplies the convolution taps.

    With taps of 0.02 a convolution mixer moves the stream by a thirtieth of what the feed-forward beside it does, and a
    fault in it would pass under the bfloat16 tolerance; with taps 25 times larger every sub-layer matters alike."""
    import json
    from gesso_amd.config.registry import architecture_of
    from gesso_amd.models.model import tensor_table
    from gesso_amd.weights.loader import random_tensors
    from gesso_amd.weights.safetensors_io import write_safetensors
    cfg = real_size_config(size, layers)
    assert cfg.intermediate_size == WIDTHS[size] and cfg.head_dim == 64
    raw = cfg.to_json()
    spec = architecture_of(raw).to_spec(cfg)
    tensors = random_tensors(tensor_table(spec), 1200, torch.bfloat16, std=0.02)
    for name in tensors:
        if name.endswith("conv.conv.weight"):
            tensors[name] = (tensors[name].float() * taps_scale).bfloat16()
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(raw, f)
    write_safetensors(os.path.join(path, "model.safetensors"), tensors, metadata={"format": "pt"})
    return path


class RealSize:
    """A folder, its sequences and the plain implementation's logits for them (made once per kind of weights)."""

    def __init__(self, root: str, taps_scale: float, lengths, size="1.2B", layers=LAYERS):
        self.dir = write_real_size_folder(os.path.join(root, f"real_{size}_{taps_scale:g}"), taps_scale, size, layers)
        self.cfg = P.read_config(self.dir)
        self.w = P.read_weights(self.dir, torch.float64)
        self.seqs = {f"s{i}": random_ids(n, 65536, 900 + n) for i, n in enumerate(lengths)}
        self.ref = {k: P.forward(self.cfg, self.w, ids).numpy() for k, ids in self.seqs.items()}
        self.ref16 = {k: P.forward(self.cfg, self.w, ids, store=P.to_bfloat16).numpy() for k, ids in self.seqs.items()}
        self.scale = max(1.0, max(float(np.abs(r).max()) for r in self.ref.values()))

    def check(self, dtype, trace, out_dir, extra=(), label=""):
        """Replay and hold the engine to the bounds of this file's opening text."""
        plain, noise = R.Distance(), R.Distance()
        rows = {"worst": 0.0, "where": None}

        def visit(name, pos, row):
            k = name.split(".", 1)[1]
            plain.add(row, self.ref[k][pos], (name, pos))
            if dtype == "bfloat16":
                noise.add(self.ref16[k][pos], self.ref[k][pos], (name, pos))
                mine = float(np.sqrt(np.mean((row - self.ref[k][pos]) ** 2)))
                theirs = float(np.sqrt(np.mean((self.ref16[k][pos] - self.ref[k][pos]) ** 2)))
                if not mine / theirs <= rows["worst"]:
                    rows["worst"], rows["where"] = mine / theirs, (name, pos)

        rc = R.visit_trace(self.dir, dtype, out_dir, trace, 65536, visit, extra=list(extra))
        assert rc == 0
        if dtype == "float32":
            print(f"{label} float32: worst |diff| {plain.worst:.3e} at {plain.where} (bound {TOL[dtype] * self.scale:.3e})")
            assert plain.worst <= TOL["float32"] * self.scale, f"first look at {plain.where}"
        else:
            print(f"{label} bfloat16: against the plain model rms {plain.rms:.3e}, worst {plain.worst:.3e} at {plain.where}; "
                  f"the rounded plain model: rms {noise.rms:.3e}, worst {noise.worst:.3e}; largest ratio of a row's rms "
                  f"{rows['worst']:.3f} at {rows['where']}")
            assert rows["worst"] <= ROW_NOISE_FACTOR, f"first look at {rows['where']}"
            assert plain.rms <= NOISE_FACTOR * noise.rms
            assert plain.worst <= WORST_FACTOR * noise.worst, f"first look at {plain.where}"


@pytest.fixture(scope="module")
def balanced(tmp_path_factory):
    return RealSize(str(tmp_path_factory.mktemp("real")), 25.0, LENGTHS)


@pytest.fixture(scope="module")
def as_benchmarked(tmp_path_factory):
    return RealSize(str(tmp_path_factory.mktemp("real")), 1.0, (70, 150))


def four_ways(seqs, seed):
    ways = {"whole": R.trace_whole, "tail": R.trace_tail,
            "portions": lambda s: R.trace_portions(s, sizes=(70, 3, 66, 2, 90, 17, 64, 65)),
            "mixed": lambda s: R.trace_mixed(s, seed=seed)}
    big = R.Trace()
    for way, make in ways.items():
        t = make({f"{way}.{k}": v for k, v in seqs.items()})
        for rec, rows in zip(t.steps, t.rows):
            big.steps.append(dict(rec, step=len(big.steps)))
            big.rows.append(rows)
        big.max_tokens = max(big.max_tokens, t.max_tokens)
    return big


@pytest.mark.parametrize("gemm", ["auto", "own"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_replay_at_the_real_layer_sizes(balanced, dtype, gemm, tmp_path):
    """Whole, tail of 32, portions that change between the kernels for few and for many rows, and four live requests
    in a pool at its peak, each position against the plain implementation."""
    if dtype == "float32" and gemm == "own":
        pytest.skip("float32 products have one kernel; the choice concerns bfloat16 only")
    balanced.check(dtype, four_ways(balanced.seqs, seed=5), str(tmp_path / "out"), extra=["--gemm", gemm],
                   label=f"1.2B layer sizes, {len(LAYERS)} of 16 layers, products {gemm},")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_replay_at_the_real_layer_sizes_with_the_benchmarks_weights(as_benchmarked, dtype, tmp_path):
    as_benchmarked.check(dtype, four_ways(as_benchmarked.seqs, seed=6), str(tmp_path / "out"),
                         label="1.2B layer sizes, weights N(0, 0.02),")


# the two other models the benchmark times, three layers each: LFM2-350M's sizes put two query heads to a key head
# (prompt and decode attention with groups of two) and feed-forward products over 4,608; LFM2-2.6B's over 7,168
OTHER_LAYERS = {"350M": ("conv", "full_attention", "conv"), "2.6B": ("full_attention", "conv", "conv")}


@pytest.fixture(scope="module")
def others(tmp_path_factory):
    made = {}

    def get(size):
        if size not in made:
            made[size] = RealSize(str(tmp_path_factory.mktemp("real")), 25.0, (3, 70, 150, 300), size, OTHER_LAYERS[size])
        return made[size]
    return get


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("size", ["350M", "2.6B"])
def test_replay_at_the_layer_sizes_of_the_other_benchmarked_models(others, size, dtype, tmp_path):
    """The four cuttings at the layer sizes of LFM2-350M (hidden 1024, 16 query and 8 key heads, feed-forward 4608) and
    LFM2-2.6B (feed-forward 7168), three layers each, every position against the plain implementation."""
    m = others(size)
    m.check(dtype, four_ways(m.seqs, seed=8), str(tmp_path / "out"),
            label=f"{size} layer sizes, {len(OTHER_LAYERS[size])} layers,")


@pytest.mark.parametrize("size,nreq,steps", [("1.2B", 3, 3), ("1.2B", 20, 2), ("1.2B", 40, 2), ("1.2B", 1, 3), ("1.2B", 8, 2),
                                             ("1.2B", 64, 2), ("350M", 8, 2), ("350M", 64, 2), ("2.6B", 40, 2),
                                             ("1.2B", 100, 2), ("350M", 130, 1)])
def test_recorded_decode_at_the_real_layer_sizes(balanced, others, size, nreq, steps):
    """The fused kernels of the recorded decode step, each row's logits against the plain implementation: at 3, 20 and
    40 rows (pre-weighted rows; more than sixteen; products in parts of K) and at the batches the benchmark times, 1, 8
    and 64 rows (capacities 1, 8 and 64 of the recording: one row tile, and four with the register ring), at the layer
    sizes of LFM2-1.2B; at 8 and 64 rows with LFM2-350M's (groups of two in decode attention, products over 4,608), at
    40 with LFM2-2.6B's (over 7,168).  And the loop for more than 64 rows, whose products are the library's: 100 rows
    (a capacity of 128) at LFM2-1.2B's sizes, 130 (of 256) at LFM2-350M's."""
    from gesso_amd import Engine, StepEntry
    from gesso_amd.engine.decode import _capacity
    m = balanced if size == "1.2B" else others(size)
    prompts = [random_ids(n, 65536, 7000 + 13 * i + n) for i, n in enumerate(([3, 18, 33] + [4 + (5 * i) % 17 for i in range(nreq)])[:nreq])]
    # poisoned: free pages, the scratch page and the scratch slot hold NaN, so the rows beyond the live batch (the
    # capacity is 4, 32 and 48) compute NaN throughout, and nothing of it may reach a live row
    eng = Engine.from_folder(m.dir, dtype="bfloat16", page_size=16, max_tokens=64 * nreq + 256, num_slots=nreq + 1,
                             poison=True)
    seqs, toks = [list(p) for p in prompts], []
    for i, p in enumerate(prompts):
        eng.add_request(i)
        toks.append(int(eng.step([StepEntry(i, p, [len(p) - 1])]).argmax()))
    kept = []
    for step in range(steps):
        for s, t in zip(seqs, toks):
            s.append(t)
        ids, bad = eng.decode(list(range(nreq)), toks, 1)
        assert not bad.any()
        kept.append(eng._runners[_capacity(nreq)].logits[:nreq].double().cpu())
        toks = ids[0].tolist()
    worst = 0.0
    for i, s in enumerate(seqs):               # a row of the whole sequence's logits is the last row of its prefix's
        ref, rounded = P.forward(m.cfg, m.w, s), P.forward(m.cfg, m.w, s, store=P.to_bfloat16)
        for step in range(steps):
            at = len(s) - steps + step
            noise = float((rounded[at] - ref[at]).pow(2).mean().sqrt())
            mine = float((kept[step][i] - ref[at]).pow(2).mean().sqrt())
            worst = max(worst, mine / noise)
            assert mine <= ROW_NOISE_FACTOR * noise, (step, i, mine, noise)
    print(f"{size} layer sizes, recorded decode of {nreq} rows: a row's rms against the plain model is at most {worst:.2f} "
          f"times the rounded plain model's")


# ------------------------------------------------------------------ long contexts

@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_long_context_in_portions_then_recorded_decoding(dtype, tmp_path):
    """About 6,000 tokens prefilled in portions of 2,048, then 40 decode steps through the recorded loop: the last row
    of every portion and every decoded row against the plain implementation.  Reaches what short sequences do not:
    decode attention with its keys split over blocks and the merge kernel, the recordings for contexts of 4,096 and
    8,192, the prompt kernel's window of page numbers refilled many times, portions over a long prefix."""
    from gesso_amd import Engine, StepEntry
    from gesso_amd.weights import write_model_folder
    from tiny import STD
    cfg_d = dataclasses.replace(TINY_D, max_position_embeddings=8192)
    tdtype = torch.float32 if dtype == "float32" else torch.bfloat16
    d = write_model_folder(str(tmp_path / "long"), cfg_d, 21, tdtype, std=STD)
    cfg, w = P.read_config(d), P.read_weights(d)
    n_prompt, n_decode = 6000, 40
    seq = random_ids(n_prompt, cfg["V"], 777)
    eng = Engine.from_folder(d, dtype=dtype, page_size=16, max_tokens=8192, num_slots=2)
    eng.add_request("r")
    ends, last = [], None
    for at in range(0, n_prompt, 2048):
        part = seq[at:at + 2048]
        last = eng.step([StepEntry("r", part, [len(part) - 1])])[0].double().cpu()
        ends.append((at + len(part) - 1, last))
    tok = int(last.argmax())
    rows = []
    for step in range(n_decode):
        seq.append(tok)
        ids, bad = eng.decode(["r"], [tok], 1)
        assert not bad.any()
        rows.append((len(seq) - 1, eng._runners[1].logits[0].double().cpu()))
        tok = int(ids[0][0])
    ref = P.forward(cfg, w, seq)
    if dtype == "float32":
        scale = max(1.0, float(ref.abs().max()))
        worst, where = 0.0, None
        for pos, row in ends + rows:
            dlt = float((row - ref[pos]).abs().max())
            if not dlt <= worst:
                worst, where = dlt, pos
        print(f"long context, float32: worst |diff| {worst:.3e} at position {where} (tolerance {1e-4 * scale:.3e})")
        assert worst <= 1e-4 * scale, f"first look at position {where}"
    else:
        # this model is one of the tiny configurations: their bound.  The forty decoded rows sit at neighbouring
        # positions behind one context of 6,000 tokens and share almost all of what their errors come from: over four
        # seeds of the weights the ratio over all rows came out at 1.29, 0.95, 0.83 and 0.96 through the recorded loop
        # and at 0.85 to 0.97 through single steps and as a prompt portion, which is the scatter of some four
        # independent rows, not of forty-three (decode attention itself rounds once: its output stands 0.29 bfloat16
        # steps rms from the exact one at 6,040 keys, what a single rounding leaves)
        from noise import NoiseBound
        rounded = P.forward(cfg, w, seq, store=P.to_bfloat16)
        bound = NoiseBound(independent=4)
        for pos, row in ends + rows:
            bound.add(row, ref[pos], rounded[pos], pos)
        bound.check("long context,")
    if dtype == "bfloat16":
        assert len(eng._runners[1].graphs) == 1 and (8192, False) in eng._runners[1].graphs


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
def test_pages_beyond_four_giga_elements_of_a_layers_cache(dtype, tmp_path):
    """A cache sized for a machine of this kind holds more than 2^32 elements a layer.  An engine with a pool of 540,000
    pages that hands out its highest pages first gives, bit for bit, the logits and the tokens of one with 256 pages: long
    portions, short ones beside them, single tokens, the recorded decode loop (offsets into the pages are 64 bits wide,
    or 32 bits in units of 16 bytes, in every kernel that reads or writes the cache)."""
    from gesso_amd import Engine, StepEntry

    d = write_real_size_folder(str(tmp_path / "m"), 25.0, "350M")
    pages = 540_000
    small = Engine.from_folder(d, dtype=dtype, page_size=16, num_pages=256, num_slots=5)
    huge = Engine.from_folder(d, dtype=dtype, page_size=16, num_pages=pages, num_slots=5)
    assert huge.storage.keys[0].numel() > 2 ** 32
    for pool in huge.manager.pools:
        pool._free.reverse()                       # the highest pages first
    ids = {k: random_ids(n, 65536, 7 + n) for k, n in {"a": 700, "b": 300, "c": 90}.items()}

    def run(eng):
        out = []
        for k in ids:
            eng.add_request(k)
        out.append(eng.step([StepEntry("a", ids["a"][:600], [599])]))
        out.append(eng.step([StepEntry("a", ids["a"][600:640], [39]), StepEntry("b", ids["b"][:200], [0, 199])]))
        out.append(eng.step([StepEntry("a", ids["a"][640:641], [0]), StepEntry("b", ids["b"][200:230], [29]),
                             StepEntry("c", ids["c"][:90], [89])]))
        out.append(eng.step([StepEntry("a", ids["a"][641:642], [0]), StepEntry("b", ids["b"][230:231], [0]),
                             StepEntry("c", [5], [0])]))
        chosen, bad = eng.decode(["a", "b", "c"], [1, 2, 3], 6)
        assert not bad.any()
        out.append(torch.from_numpy(chosen.copy()))
        top = max(max(t for t in eng.manager.get(k).tables[0] if t >= 0) for k in ids)
        for k in ids:
            eng.finish_request(k)
        return out, top

    (a, top_a), (b, top_b) = run(small), run(huge)
    assert top_a < 256 and top_b >= pages - 200
    for i, (x, y) in enumerate(zip(a, b)):
        assert torch.isfinite(x.float()).all(), i
        assert torch.equal(x.cpu(), y.cpu()), (i, (x.float().cpu() - y.float().cpu()).abs().max().item())


@pytest.mark.gpu
def test_recorded_steps_at_the_real_layer_sizes_replay_what_was_launched(tmp_path):
    """At LFM2-1.2B's layer sizes the library takes other kernels for its products than at tiny sizes (work shared out
    over K among them).  A prompt of 2,048 tokens and steps of 1,024 tokens in portions, recorded and replayed eight times
    each with launched steps of other shapes between the replays: every replay's logits are, bit for bit, those of an
    engine that launches the same steps."""
    from gesso_amd import Engine, StepEntry
    from gesso_amd.parts import RuntimeOptions

    d = write_real_size_folder(str(tmp_path / "m"), 25.0, "1.2B")
    kw = dict(dtype="bfloat16", page_size=16, max_tokens=6 * 2304, num_slots=7, poison=True)
    launched = Engine.from_folder(d, **kw)
    replayed = Engine.from_folder(d, options=RuntimeOptions(record_portions=True), **kw)
    whole = [random_ids(2048, 65536, 30 + i) for i in range(12)]
    parts = [random_ids(1500, 65536, 60 + i) for i in range(4)]
    for turn in range(12):
        outs = []
        for eng in (launched, replayed):
            eng.add_request(("w", turn))
            a = eng.step([StepEntry(("w", turn), whole[turn], [2047, 5])])
            # steps of 1,024 tokens: two portions of 500 and one of 24; then a launched step of another shape
            for i in range(3):
                eng.add_request(("p", turn, i))
            b = eng.step([StepEntry(("p", turn, 0), parts[turn % 4][:500], [499]), StepEntry(("p", turn, 1), parts[(turn + 1) % 4][:500], []),
                          StepEntry(("p", turn, 2), parts[(turn + 2) % 4][:24], [23])])
            c = eng.step([StepEntry(("p", turn, 0), parts[turn % 4][500:500 + 70 + turn], [69 + turn])])
            outs.append((a, b, c))
            for rid in [("w", turn)] + [("p", turn, i) for i in range(3)]:
                eng.finish_request(rid)
        for x, y in zip(*outs):
            assert torch.isfinite(x).all() and torch.equal(x, y), (turn, (x - y).abs().max().item())
    rec = replayed.recorder
    assert not rec.refused and rec.replays == 2 * (12 - rec.SEEN_BEFORE), (rec.replays, rec.refused)
