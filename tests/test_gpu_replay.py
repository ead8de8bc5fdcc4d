"""bin/trace_run against the plain implementation, in the four ways of cutting the work.

One process of trace_run per (configuration, precision) replays: each request alone and whole;
most of it in one step and the last 32 tokens one by one; portions of changing size down to two
tokens; and a mix of up to four live requests with a pool so small that pages are used again.
Every fed position's logits are compared with the plain implementation's whole-sequence logits.

Bounds: float32 ``1e-4 * max(1, max|ref|)`` at the worst logit (the reference's own device bound,
``test/test_amdgpu_lfm2.jl:34``); bfloat16: the distance that the plain model itself takes when its activations are
rounded to bfloat16, row by row, over all rows and at the worst logit (``tests/noise.py``; ``tests/test_sensitivity.py``
shows without a GPU that a lost convolution history, reversed taps or a key past the causal edge break it at every
configuration here).  The weights are drawn with a standard deviation of 0.1, at which any bfloat16 pipeline stands
some 2 % of the logits' spread from the plain model: a fixed tolerance would be narrower than that noise or wider than
a fault.
"""
import pytest
import torch

import replay as R
from tiny import CONFIGS, random_ids, write_tiny

pytestmark = pytest.mark.gpu


# sequence lengths: the benchmark description's prompts plus generated tokens
LENGTHS = {"A": (5 + 16, 17 + 16, 32 + 16, 70), "B": (1 + 24, 9 + 24, 40 + 24, 100 + 24), "C": (3, 50, 97),
           "D": (2, 40, 66, 150)}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    return str(tmp_path_factory.mktemp("models"))


def sequences(name):
    cfg, seed = CONFIGS[name]
    return {f"s{i}": random_ids(n, cfg.vocab_size, 100 * seed + i) for i, n in enumerate(LENGTHS[name])}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_replay_four_ways(name, dtype, folders, tmp_path):
    cfg, _ = CONFIGS[name]
    model_dir = write_tiny(folders, name, torch.float32 if dtype == "float32" else torch.bfloat16)
    seqs = sequences(name)
    plain = R.Plain(model_dir, seqs, dtype)

    # the four ways in one process: names differ per way so that all requests are distinct
    ways = {"whole": R.trace_whole, "tail": R.trace_tail, "portions": R.trace_portions,
            "mixed": lambda s: R.trace_mixed(s, seed=7)}
    big = R.Trace()
    owner = []
    for way, make in ways.items():
        t = make({f"{way}.{k}": v for k, v in seqs.items()})
        for rec, rows in zip(t.steps, t.rows):
            rec = dict(rec, step=len(big.steps))
            big.steps.append(rec)
            big.rows.append(rows)
            owner.append(way)
        big.max_tokens = max(big.max_tokens, t.max_tokens)
    got, rc = R.run_trace(model_dir, dtype, str(tmp_path / "out"), big, cfg.vocab_size)
    assert rc == 0
    for way in ways:
        mine = {k.split(".", 1)[1]: v for k, v in got.items() if k.startswith(way + ".")}
        assert {k: len(v) for k, v in mine.items()} == {k: len(v) for k, v in seqs.items()}, way
        plain.check(mine, f"{name} {way}")


def random_config(seed: int):
    """A configuration drawn from a seed: head widths in steps of 16, any number of heads and groups, widths and
    vocabularies that are no powers of two, two to five layers of either kind."""
    import random
    from gesso_amd.config import Lfm2Config
    rng = random.Random(seed)
    d = rng.choice([16, 32, 48, 64, 80, 96, 128])
    nkv = rng.choice([1, 2, 3])
    nh = nkv * (rng.choice([1, 2, 3, 4]) if d <= 64 else rng.choice([1, 2]))
    layers = rng.randint(2, 5)
    types = [rng.choice(["conv", "full_attention"]) for _ in range(layers)]
    types[rng.randrange(layers)] = "full_attention"
    types[(types.index("full_attention") + 1) % layers] = "conv"
    return Lfm2Config(vocab_size=rng.choice([97, 200, 301, 512, 1000]), hidden_size=nh * d, num_hidden_layers=layers,
                      num_attention_heads=nh, num_key_value_heads=nkv, layer_types=tuple(types),
                      conv_L_cache=rng.choice([2, 3, 4]), conv_bias=rng.random() < 0.4,
                      intermediate_size=rng.choice([40, 100, 136, 192, 320, 500]),
                      norm_eps=rng.choice([1e-5, 1e-6, 1e-4]), rope_theta=rng.choice([1e4, 1e5, 1e6]),
                      tie_word_embeddings=rng.random() < 0.5, max_position_embeddings=rng.choice([192, 256, 400]))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", [11, 12, 13])
def test_replay_of_configurations_drawn_at_random(seed, dtype, tmp_path):
    import random
    from gesso_amd.weights import write_model_folder
    from tiny import STD
    cfg = random_config(seed)
    rng = random.Random(seed)
    model_dir = write_model_folder(str(tmp_path / "m"), cfg, seed, torch.float32 if dtype == "float32" else torch.bfloat16,
                                   std=STD)
    lens = [rng.randint(1, 6), rng.randint(20, 60), rng.randint(61, 110), rng.randint(111, 170)]
    seqs = {f"s{i}": random_ids(n, cfg.vocab_size, seed * 10 + i) for i, n in enumerate(lens)}
    plain = R.Plain(model_dir, seqs, dtype)
    ways = {"whole": R.trace_whole, "tail": R.trace_tail, "portions": R.trace_portions,
            "mixed": lambda s: R.trace_mixed(s, seed=seed)}
    big = R.Trace()
    for way, make in ways.items():
        t = make({f"{way}.{k}": v for k, v in seqs.items()})
        for rec, rows in zip(t.steps, t.rows):
            big.steps.append(dict(rec, step=len(big.steps)))
            big.rows.append(rows)
        big.max_tokens = max(big.max_tokens, t.max_tokens)
    got, rc = R.run_trace(model_dir, dtype, str(tmp_path / "out"), big, cfg.vocab_size)
    assert rc == 0
    for way in ways:
        mine = {k.split(".", 1)[1]: v for k, v in got.items() if k.startswith(way + ".")}
        plain.check(mine, f"seed {seed} ({cfg.num_attention_heads}/{cfg.num_key_value_heads} heads of {cfg.head_dim}) {way}")


@pytest.mark.parametrize("name", ["B", "D"])
def test_replay_with_the_hand_written_product_for_many_rows(name, folders, tmp_path):
    """Prompts of more than 64 tokens through the hand-written matrix-core product (with its SwiGLU epilogue) instead of
    the vendor library's: whole, and in portions that change between that kernel and the weight-streaming one."""
    cfg, _ = CONFIGS[name]
    model_dir = write_tiny(folders, name, torch.bfloat16)
    seqs = sequences(name)
    plain = R.Plain(model_dir, seqs, "bfloat16")
    for way, make in (("whole", R.trace_whole), ("portions", lambda s: R.trace_portions(s, sizes=(70, 3, 66, 2, 90)))):
        got, rc = R.run_trace(model_dir, "bfloat16", str(tmp_path / way), make(seqs), cfg.vocab_size,
                              extra=["--gemm", "own"])
        assert rc == 0
        plain.check(got, f"{name} own product, {way}")


@pytest.mark.parametrize("poison", [False, True])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_replay_with_pages_of_eight_and_portions_of_thirteen(dtype, poison, folders, tmp_path):
    """The second tiny configuration as its workload is described: pages of 8 tokens, prompts of 1, 9, 40 and 100 tokens
    plus 24 more, portions of 13.  With ``poison`` every page and slot that is given back is filled with NaN before the
    next step: a kernel that reads a row of a page that is not its sequence's (the rest of a last page, a page of
    someone who has finished) would carry the NaN into the logits."""
    cfg, _ = CONFIGS["B"]
    model_dir = write_tiny(folders, "B", torch.float32 if dtype == "float32" else torch.bfloat16)
    seqs = sequences("B")
    plain = R.Plain(model_dir, seqs, dtype)
    ways = {"whole": R.trace_whole, "tail": R.trace_tail, "portions": lambda s: R.trace_portions(s, sizes=(13,)),
            "mixed": lambda s: R.trace_mixed(s, seed=3)}
    big = R.Trace()
    for way, make in ways.items():
        t = make({f"{way}.{k}": v for k, v in seqs.items()})
        for rec, rows in zip(t.steps, t.rows):
            big.steps.append(dict(rec, step=len(big.steps)))
            big.rows.append(rows)
        big.max_tokens = max(big.max_tokens, t.max_tokens)
    got, rc = R.run_trace(model_dir, dtype, str(tmp_path / "out"), big, cfg.vocab_size, page_size=8,
                          extra=["--poison"] if poison else [])
    assert rc == 0
    for way in ways:
        mine = {k.split(".", 1)[1]: v for k, v in got.items() if k.startswith(way + ".")}
        assert {k: len(v) for k, v in mine.items()} == {k: len(v) for k, v in seqs.items()}, way
        plain.check(mine, f"B, pages of 8, poison {poison}, {way}")
