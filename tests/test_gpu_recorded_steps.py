"""Steps of prompt portions through a recording (gesso_amd/engine/planned.py) give the logits of the same steps launched
kernel by kernel, bit for bit: the same kernels run with the same arguments.  Two engines over one model folder take the
same steps, one with ``record_portions``; the steps keep their token count while the sequences in them come, grow
and go, and pages and slots are used again (poisoned in between)."""
import random

import pytest
import torch

from gesso_amd.config import Lfm2Config
from gesso_amd.weights import write_model_folder
from tiny import STD, random_ids

pytestmark = pytest.mark.gpu

# heads 64 wide (the kernel for long portions takes no others); E has four query heads to a key head, a bias on the
# convolution and room for thousands of keys
WIDE_D = Lfm2Config(
    vocab_size=200, hidden_size=128, num_hidden_layers=3, num_attention_heads=2, num_key_value_heads=1,
    layer_types=("full_attention", "conv", "full_attention"), conv_L_cache=3, conv_bias=False,
    intermediate_size=136, norm_eps=1e-5, rope_theta=1e5, tie_word_embeddings=True, max_position_embeddings=1024)
WIDE_E = Lfm2Config(
    vocab_size=333, hidden_size=256, num_hidden_layers=4, num_attention_heads=4, num_key_value_heads=1,
    layer_types=("conv", "full_attention", "conv", "full_attention"), conv_L_cache=4, conv_bias=True,
    intermediate_size=344, norm_eps=1e-6, rope_theta=1e6, tie_word_embeddings=False, max_position_embeddings=8192)


def engines(folder, **kw):
    from gesso_amd import Engine
    from gesso_amd.parts import RuntimeOptions

    plain = Engine.from_folder(folder, dtype="bfloat16", poison=True, **kw)
    recorded = Engine.from_folder(folder, dtype="bfloat16", poison=True, options=RuntimeOptions(record_portions=True), **kw)
    assert plain.recorder is None and recorded.recorder is not None
    return plain, recorded


class Workload:
    """Requests with prompts of random lengths; every step holds ``T`` tokens: the decoded tokens of the requests whose
    prompts are through (at the head), then portions of the prompts that are not, cut where the step is full."""

    def __init__(self, vocab, T, seed, prompt_lens, new_tokens=(3, 9), live=6, tag="w"):
        self.rng = random.Random(seed)
        self.vocab, self.T, self.live_max = vocab, T, live
        self.prompts = [random_ids(n, vocab, seed * 100 + i) for i, n in enumerate(prompt_lens)]
        self.new_tokens = new_tokens
        self.next_rid, self.tag = 0, tag
        self.live = {}          # rid -> dict(prompt, done, left, token)

    def admit(self, engines_):
        while len(self.live) < self.live_max and self.next_rid < len(self.prompts):
            rid = (self.tag, self.next_rid)
            self.live[rid] = dict(prompt=self.prompts[self.next_rid], done=0, left=self.rng.randint(*self.new_tokens), token=None)
            self.next_rid += 1
            for e in engines_:
                e.add_request(rid)

    def step_entries(self):
        from gesso_amd import StepEntry
        entries, room = [], self.T
        for rid, r in self.live.items():
            if r["token"] is not None and room > 2:
                entries.append(StepEntry(rid, [r["token"]], [0]))
                room -= 1
        for rid, r in self.live.items():
            rest = len(r["prompt"]) - r["done"]
            if r["token"] is None and rest and room >= 2:
                n = min(rest, room)
                if rest - n == 1:          # (never leave a single token of a prompt over: it would look like a decoded one)
                    n -= 1
                if n < 2:
                    continue
                last = r["done"] + n == len(r["prompt"])
                entries.append(StepEntry(rid, r["prompt"][r["done"]:r["done"] + n], [n - 1] if last else []))
                room -= n
        return entries

    def advance(self, entries, logits, engines_):
        row = 0
        for e in entries:
            r = self.live[e.rid]
            if r["token"] is None:
                r["done"] += len(e.tokens)
            if e.want:
                r["token"] = int(logits[row].argmax())
                row += 1
                r["left"] -= 1
                if r["left"] == 0:
                    del self.live[e.rid]
                    for eng in engines_:
                        eng.finish_request(e.rid)


def run_both(plain, recorded, work, steps, kinds):
    """``kinds``: how often each kind of step came (None: a step that is not to be recorded)."""
    for s in range(steps):
        work.admit((plain, recorded))
        entries = work.step_entries()
        if not entries:
            break
        kind = recorded.recorder.kind_of(entries)
        kinds[kind] = kinds.get(kind, 0) + 1
        a = plain.step(entries)
        b = recorded.step(entries)
        assert (a is None) == (b is None), s
        if a is not None:
            assert torch.isfinite(a).all(), s
            assert torch.equal(a, b), (s, [(e.rid, len(e.tokens)) for e in entries], (a - b).abs().max().item())
        work.advance(entries, a if a is not None else [], (plain, recorded))


def replays_expected(kinds, recorder):
    """Every step of a kind after the first few, for the kinds that were recorded (the first that came often enough)."""
    assert not recorder.refused, recorder.refused
    made = [k for k, r in recorder.recordings.items() if r is not None]
    assert set(made) <= {k for k, n in kinds.items() if k is not None and n > recorder.SEEN_BEFORE}
    assert len(made) == min(recorder.MAX_RECORDINGS, sum(1 for k, n in kinds.items() if k is not None and n > recorder.SEEN_BEFORE))
    return sum(kinds[k] - recorder.SEEN_BEFORE for k in made)


@pytest.mark.parametrize("name,T", [("D", 96), ("E", 160), ("E", 72)])
def test_recorded_steps_of_portions_equal_the_launched_ones(tmp_path, name, T):
    cfg = {"D": WIDE_D, "E": WIDE_E}[name]
    folder = str(tmp_path / name)
    write_model_folder(folder, cfg, 11, torch.bfloat16, std=STD)
    # so few pages that they are used again: six live requests of up to 400 tokens
    plain, recorded = engines(folder, page_size=16, max_tokens=6 * 448, num_slots=7)
    rng = random.Random(T)
    work = Workload(cfg.vocab_size, T, seed=T, prompt_lens=[rng.randint(20, 400) for _ in range(40)])
    kinds = {}
    run_both(plain, recorded, work, 60, kinds)
    rec = recorded.recorder
    assert rec.replays == replays_expected(kinds, rec) and rec.replays >= 20, (rec.replays, kinds)


def test_recorded_steps_with_thousands_of_keys_walk_them_whole(tmp_path):
    """A sequence with more keys than a walk in halves takes makes a kind of its own (another walk, a longer block table);
    both kinds are recorded and both give the launched steps' logits."""
    from gesso_amd import StepEntry

    folder = str(tmp_path / "E")
    write_model_folder(folder, WIDE_E, 12, torch.bfloat16, std=STD)
    plain, recorded = engines(folder, page_size=16, max_tokens=4608 + 6 * 448, num_slots=8)
    T = 128
    rng = random.Random(5)
    work = Workload(WIDE_E.vocab_size, T, seed=5, prompt_lens=[rng.randint(30, 300) for _ in range(30)], live=5)
    kinds = {}
    run_both(plain, recorded, work, 12, kinds)
    # a long request beside them: most of its prompt in one step of its own, the rest in portions among the others
    long_prompt = random_ids(4400, WIDE_E.vocab_size, 77)
    for eng in (plain, recorded):
        eng.add_request("long")
        assert eng.step([StepEntry("long", long_prompt[:4000], [])]) is None
    work.prompts.append(long_prompt)
    work.live["long"] = dict(prompt=long_prompt, done=4000, left=6, token=None)
    run_both(plain, recorded, work, 25, kinds)
    rec = recorded.recorder
    assert rec.replays == replays_expected(kinds, rec) and rec.replays >= 20, (rec.replays, kinds)
    made = [k for k, r in rec.recordings.items() if r is not None]
    assert {k[1] for k in made} == {4096, 8192}, made       # block tables for 4,096 and for 8,192 keys
    assert {k[2] for k in made if k[1] == 8192} != {k[2] for k in made if k[1] == 4096}, made     # and another walk


def test_the_scheduler_over_recorded_steps_generates_the_same_ids(tmp_path):
    """Through the entry point: prompts cut into portions under a token budget, greedy; the ids are the same with
    recording on and off, and most steps were replays."""
    from gesso_amd import Session
    from gesso_amd.parts import RuntimeOptions

    folder = str(tmp_path / "E")
    write_model_folder(folder, WIDE_E, 13, torch.bfloat16, std=STD)
    rng = random.Random(3)
    prompts = [random_ids(rng.randint(100, 700), WIDE_E.vocab_size, 300 + i) for i in range(24)]
    out = []
    for on in (False, True):
        s = Session(folder, dtype="bfloat16", max_num_seqs=8, max_num_batched_tokens=256, chunk_size=256,
                    kernel_options=RuntimeOptions(record_portions=on), max_tokens=8 * 1024)
        out.append(s.generate(prompts, max_new_tokens=12))
        if on:
            rec = s.engine.recorder
            assert not rec.refused and rec.replays >= 20, (rec.refused, rec.replays, rec.seen)
            assert s.last_stats["replayed_steps"] == rec.replays
        s.close()
    assert out[0] == out[1]


def test_recorded_steps_over_two_page_groups_one_of_them_windowed(tmp_path):
    """A model of parts put together by hand: an attention layer that sees all keys, one that sees the last 40 (pages of
    its own, given back as the window passes them and poisoned), a short convolution.  Recorded steps give the launched
    steps' logits here too: block tables of both groups, entries of pages that are gone, the windowed walk."""
    from gesso_amd import Engine
    from gesso_amd.config import AttentionSpec, BlockSpec, LayerCall, ModelSpec, RMSNormSpec, RopeSpec, ShortConvSpec, SwiGLUSpec
    from gesso_amd.models.model import tensor_table
    from gesso_amd.parts import RuntimeOptions
    from gesso_amd.weights import random_tensors
    from gesso_amd.weights.loader import held_dtype

    H, V, eps = 128, 90, 1e-5
    norm = RMSNormSpec(H, eps)
    rope = RopeSpec(head_dim=64, rotary_dim=64, theta=1e4, max_position=1024)
    full = AttentionSpec(hidden=H, n_heads=2, n_kv_heads=1, head_dim=64, position=rope, qk_norm=RMSNormSpec(64, eps))
    near = AttentionSpec(hidden=H, n_heads=2, n_kv_heads=2, head_dim=64, position=rope, qk_norm=None, window=40)

    def names(i, mixer_names, ffn=True):
        n = {f"mixer.{k}": f"L{i}.{k}" for k in mixer_names}
        n["mixer_norm.weight"] = f"L{i}.n1"
        if ffn:
            n.update({"ffn_norm.weight": f"L{i}.n2", "ffn.w1.weight": f"L{i}.w1", "ffn.w3.weight": f"L{i}.w3", "ffn.w2.weight": f"L{i}.w2"})
        return n

    proj = ["q_proj.weight", "k_proj.weight", "v_proj.weight", "out_proj.weight"]
    blocks = (BlockSpec(full, norm, SwiGLUSpec(H, 96), norm, names(0, proj + ["q_norm.weight", "k_norm.weight"])),
              BlockSpec(near, norm, SwiGLUSpec(H, 64), norm, names(1, proj)),
              BlockSpec(ShortConvSpec(H, 3), norm, None, None, names(2, ["in_proj.weight", "conv.weight", "out_proj.weight"], False)))
    spec = ModelSpec(architecture="ToyTwoGroups", hidden=H, vocab=V, blocks=blocks,
                     schedule=(LayerCall(0), LayerCall(1), LayerCall(2)), final_norm=norm, tie_embeddings=True,
                     max_position=1024, names={"embed": "emb", "final_norm.weight": "fn"})
    table = tensor_table(spec)
    cpu = random_tensors(table, 29, torch.bfloat16, std=0.15)
    dev = "cuda:0"
    tensors = {k: v.to(dev, held_dtype(v.dtype, table[k].role, torch.bfloat16)) for k, v in cpu.items()}
    made = []
    for on in (False, True):
        # the kernel for long portions at every length, so that steps whose longest portion is short are recorded too
        made.append(Engine(spec, tensors, torch.bfloat16, dev, page_size=4, max_tokens=6 * 448, num_slots=7, poison=True,
                           options=RuntimeOptions(record_portions=on, prompt_attention="wide")))
    plain, recorded = made
    assert [g.need.window for g in recorded.manager.layout.paged] == [None, 40]
    rng = random.Random(9)
    work = Workload(V, 80, seed=9, prompt_lens=[rng.randint(20, 400) for _ in range(30)])
    kinds = {}
    run_both(plain, recorded, work, 50, kinds)
    rec = recorded.recorder
    assert rec.replays == replays_expected(kinds, rec) and rec.replays >= 20, (rec.replays, kinds)
    plain.manager.check(); recorded.manager.check()
    # Seventy requests of this model through the decode loop for many rows (a capacity of 128; the windowed group gives
    # pages back on the way, poisoned) against the same tokens as ordinary steps of seventy single tokens: the same
    # kernels but for the final norm's laziness, so the logits agree to the last bits and the tokens are the same.
    from gesso_amd import StepEntry
    from gesso_amd.engine.decode import _capacity
    for eng in made:
        for rid in list(eng.manager.requests):
            eng.finish_request(rid)
    n = 70
    wide = Engine(spec, tensors, torch.bfloat16, dev, page_size=4, max_tokens=n * 96, num_slots=n + 1, poison=True)
    steps = Engine(spec, tensors, torch.bfloat16, dev, page_size=4, max_tokens=n * 96, num_slots=n + 1, poison=True)
    toks = []
    for i in range(n):
        prompt = random_ids(3 + (7 * i) % 50, V, 600 + i)
        for eng in (wide, steps):
            eng.add_request(i)
            first = eng.step([StepEntry(i, prompt, [len(prompt) - 1])])
        toks.append(int(first.argmax()))
    for s in range(12):
        a = steps.step([StepEntry(i, [t], [0]) for i, t in enumerate(toks)])
        ids, bad = wide.decode(list(range(n)), toks, 1)
        b = wide._runners[_capacity(n)].logits[:n]
        assert not bad.any() and torch.isfinite(a).all()
        assert float((a - b).abs().max()) <= 2e-2 * float(a.abs().max()), (s, float((a - b).abs().max()), float(a.abs().max()))
        toks = ids[0].tolist()
        assert sum(int(x) != y for x, y in zip(a.argmax(1).tolist(), toks)) <= 1, s
    assert _capacity(n) == 128 and len(wide.manager.get(0).tables) == 2


def test_a_recording_that_lies_idle_makes_room_for_another_kind(tmp_path):
    """With room for one recording: steps of 96 tokens are recorded; when the steps turn to 80 tokens that recording is
    given up after a few idle steps and the new kind recorded, and back again; the logits stay those of the launched steps."""
    folder = str(tmp_path / "D")
    write_model_folder(folder, WIDE_D, 14, torch.bfloat16, std=STD)
    plain, recorded = engines(folder, page_size=16, max_tokens=12 * 448, num_slots=13)
    rec = recorded.recorder
    rec.MAX_RECORDINGS, rec.IDLE_STEPS = 1, 5
    held = []
    for turn, T in enumerate((96, 80, 96)):
        rng = random.Random(T + turn)
        work = Workload(WIDE_D.vocab_size, T, seed=T + turn, prompt_lens=[rng.randint(70, 400) for _ in range(12)], tag=turn)
        before = rec.replays
        run_both(plain, recorded, work, 16, {})
        assert not rec.refused, rec.refused
        made = [k for k, r in rec.recordings.items() if r is not None]
        assert len(made) == 1 and made[0][0] == T, (T, made)
        assert rec.replays - before >= 4, (T, rec.replays - before)
        held.append(made[0])
        for rid in list(work.live):             # what this turn left unfinished
            plain.finish_request(rid); recorded.finish_request(rid)
    assert held[0] == held[2] != held[1]


def test_recorded_steps_of_more_single_tokens_than_the_decode_loop_takes(tmp_path):
    """140 sequences that bring one token each (the recorded decode loop takes 64): such steps run on the library's
    products and are recorded like steps with portions; the same logits as launched, while sequences end and others
    take their pages and slots."""
    from gesso_amd import StepEntry

    folder = str(tmp_path / "E")
    write_model_folder(folder, WIDE_E, 15, torch.bfloat16, std=STD)
    n = 140
    plain, recorded = engines(folder, page_size=16, max_tokens=n * 96, num_slots=n + 1)
    assert n > recorded.DECODE_MAX_BATCH
    rng = random.Random(2)
    tokens = {}
    for a in range(0, n, 20):
        entries = [StepEntry(i, random_ids(rng.randint(5, 60), WIDE_E.vocab_size, 40 + i), []) for i in range(a, a + 20)]
        for eng in (plain, recorded):
            for e in entries:
                eng.add_request(e.rid)
            assert eng.step(entries) is None
    for i in range(n):
        tokens[i] = rng.randrange(WIDE_E.vocab_size)
    fresh = n
    for s in range(14):
        entries = [StepEntry(i, [t], [0]) for i, t in tokens.items()]
        a, b = plain.step(entries), recorded.step(entries)
        assert torch.isfinite(a).all() and torch.equal(a, b), (s, (a - b).abs().max().item())
        picks = a.argmax(1).tolist()
        tokens = {e.rid: p for e, p in zip(entries, picks)}
        # three sequences end and three new ones of one token begin (their first token decodes from an empty cache)
        for rid in list(tokens)[s % 5::50][:3]:
            del tokens[rid]
            for eng in (plain, recorded):
                eng.finish_request(rid)
                eng.add_request(fresh)
            tokens[fresh] = rng.randrange(WIDE_E.vocab_size)
            fresh += 1
    rec = recorded.recorder
    assert not rec.refused, rec.refused
    (kind, step_), = [(k, r) for k, r in rec.recordings.items() if r is not None]
    assert step_.single and kind[0] == n and rec.replays == 14 - rec.SEEN_BEFORE
    plain.manager.check(); recorded.manager.check()


def test_recorded_steps_with_more_sequences_than_sixty_four(tmp_path):
    """A hundred live requests: steps of 230 tokens hold some eighty decoded tokens beside portions; their recording has
    room for 128 sequences, and the logits are the launched steps'."""
    folder = str(tmp_path / "E")
    write_model_folder(folder, WIDE_E, 16, torch.bfloat16, std=STD)
    live = 100
    plain, recorded = engines(folder, page_size=16, max_tokens=live * 256, num_slots=live + 1)
    rng = random.Random(4)
    work = Workload(WIDE_E.vocab_size, 230, seed=4, prompt_lens=[rng.randint(20, 150) for _ in range(400)],
                    new_tokens=(50, 80), live=live)
    kinds = {}
    run_both(plain, recorded, work, 80, kinds)
    rec = recorded.recorder
    made = [k for k, r in rec.recordings.items() if r is not None]
    assert any(k[3] == 128 for k in made), (made, kinds)
    assert rec.replays == replays_expected(kinds, rec) and rec.replays >= 10, (rec.replays, kinds)


def test_steps_that_want_nothing_follow_each_other_while_the_device_lags(tmp_path):
    """Portions in the middle of a prompt want no logits, so the host waits for nothing and fills in the next step while the
    device has not begun the last one: each step's indices must still be its own when the device copies them.  A long
    product keeps the device busy; twelve steps of 192 tokens are queued behind it without a wait, the last wants its
    logits; they are the launched steps' (with the pages of earlier requests poisoned in between)."""
    from gesso_amd import StepEntry

    folder = str(tmp_path / "E")
    write_model_folder(folder, WIDE_E, 17, torch.bfloat16, std=STD)
    plain, recorded = engines(folder, page_size=16, max_tokens=3 * 1280, num_slots=4)
    busy = torch.randn(8192, 8192, device="cuda:0")
    for turn in range(3):
        prompts = {(turn, i): random_ids(12 * 64, WIDE_E.vocab_size, 50 * turn + i) for i in range(3)}
        got = []
        for eng in (plain, recorded):
            for rid in prompts:
                eng.add_request(rid)
            torch.cuda.synchronize()
            if eng is recorded:
                for _ in range(40):
                    busy @ busy                           # some tens of milliseconds of work before the steps' first kernel
            for s in range(12):
                last = s == 11
                out = eng.step([StepEntry(rid, p[64 * s:64 * s + 64], [63] if last else []) for rid, p in prompts.items()])
                assert (out is not None) == last
            got.append(out)
            for rid in prompts:
                eng.finish_request(rid)
        assert torch.isfinite(got[0]).all() and torch.equal(got[0], got[1]), (turn, (got[0] - got[1]).abs().max().item())
    assert recorded.recorder.replays >= 3 * 12 - recorded.recorder.SEEN_BEFORE and not recorded.recorder.refused


def test_the_scheduler_short_of_pages_over_recorded_steps(tmp_path):
    """Six long prompts in portions of 64 under a budget of 128 tokens, with so few pages that requests are preempted
    dozens of times and their pages poisoned: many steps hold portions only and want no logits.  The ids are the
    launched steps' ids (this is the case that showed a step's indices overwritten before the device had copied them)."""
    from gesso_amd import Session
    from gesso_amd.parts import RuntimeOptions

    folder = str(tmp_path / "E")
    write_model_folder(folder, WIDE_E, 5, torch.bfloat16, std=STD)
    lens = [462, 477, 464, 365, 499, 214]
    prompts = [random_ids(n, WIDE_E.vocab_size, 12900 + i) for i, n in enumerate(lens)]
    out = []
    for on in (False, True):
        s = Session(folder, dtype="bfloat16", context_length=640, num_pages=66, page_size=16, chunk_size=64, max_num_seqs=7,
                    max_num_batched_tokens=128, watermark=0.0, poison=True,
                    kernel_options=RuntimeOptions(record_portions=on, prompt_attention="wide"))
        out.append(s.generate(prompts, max_new_tokens=18, eos_ids=()))
        assert s.last_stats["preemptions"] >= 10
        if on:
            assert s.last_stats["replayed_steps"] >= 30 and not s.engine.recorder.refused
        st = s.engine.manager.stats()
        assert st["pages_free"] == st["pages_total"] and st["slots_free"] == st["slots_total"]
        s.close()
    assert out[0] == out[1]
