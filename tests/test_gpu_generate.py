"""Generation through the entry points, against the plain implementation's whole re-forwards."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_lfm2 as P
from noise import WORST, NoiseBound, supported
from tiny import CONFIGS, STD, TINY_B, random_ids, write_tiny

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

# the benchmark description's workloads for the two tiny configurations
PROMPTS = {"A": (5, 17, 32), "B": (1, 9, 40, 100), "D": (3, 22, 45, 70)}
NEW = {"A": 16, "B": 24, "D": 20}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    return str(tmp_path_factory.mktemp("gen"))


@pytest.fixture(scope="module")
def plain(folders):
    out = {}
    for name in ("A", "B"):
        d = write_tiny(folders, name, torch.float32)
        out[name] = (d, P.read_config(d), P.read_weights(d))
    return out


def prompts_of(name):
    cfg, seed = CONFIGS[name]
    return [random_ids(n, cfg.vocab_size, 1000 * seed + n) for n in PROMPTS[name]]


@pytest.mark.parametrize("name", ["A", "B"])
def test_greedy_float32_equals_plain_greedy(plain, name):
    from gesso_amd import Session
    d, cfg, w = plain[name]
    s = Session(d, dtype="float32", context_length=160, page_size=8 if name == "B" else 16, chunk_size=13 if name == "B" else 7)
    prompts = prompts_of(name)
    got = s.generate(prompts, max_new_tokens=NEW[name], eos_ids=())
    for p, g in zip(prompts, got):
        assert g == P.greedy(cfg, w, p, NEW[name])
    # one prompt alone gives what it gave in the batch; nothing new returns the prompt
    assert s.generate(prompts[1], max_new_tokens=NEW[name], eos_ids=()) == got[1]
    assert s.generate(prompts[0], max_new_tokens=0) == prompts[0]
    # the first new token is the argmax of the prompt's last row (test/test_reference_generate.jl:24-46)
    lg = s.prefill(prompts[2])
    assert lg.shape == (len(prompts[2]), cfg["V"]) and int(lg[-1].argmax()) == got[2][len(prompts[2])]
    st = s.engine.manager.stats()
    assert st["pages_free"] == st["pages_total"] and st["slots_free"] == st["slots_total"]


@pytest.mark.parametrize("name,poison", [("A", False), ("B", False), ("A", True), ("B", True), ("D", True)])
def test_greedy_bfloat16_picks_tokens_the_plain_logits_support(folders, name, poison):
    """With ``poison``: pages of 4, two requests at a time, so that the later requests run on pages and slots that the
    earlier ones gave back, filled with NaN in between: the recorded decode step with its fused kernels (D: heads of
    64, where decode attention writes the step's key itself) must not meet what a page held before."""
    from gesso_amd import Session
    d = write_tiny(folders, name, torch.bfloat16)
    cfg, w = P.read_config(d), P.read_weights(d)
    if poison:
        s = Session(d, dtype="bfloat16", context_length=160, page_size=4, max_num_seqs=2, num_pages=64, poison=True)
    else:
        s = Session(d, dtype="bfloat16", context_length=160)
    prompts = prompts_of(name)
    got = s.generate(prompts, max_new_tokens=NEW[name], eos_ids=())
    for p, g in zip(prompts, got):
        ref = P.forward(cfg, w, g[:-1])
        # the token chosen is the plain argmax, or as good as it within twice what bfloat16 logits may stand from the
        # plain ones (the worst logit of the rounded plain model over this sequence, times the bound's factor)
        slack = 2 * WORST * float((P.forward(cfg, w, g[:-1], store=P.to_bfloat16) - ref).abs().max())
        for i in range(len(p), len(g)):
            assert supported(ref[i - 1], g[i], slack), (i, g[i], slack)


def test_seventy_requests_at_once_decode_through_the_recorded_loop_in_groups(plain):
    """More requests than the recorded loop takes at once (64): a group of 64 and a group of 6 per run; every request's
    tokens are the plain greedy ones."""
    from gesso_amd import Session
    d, cfg, w = plain["A"]
    s = Session(d, dtype="float32", context_length=64, max_num_seqs=80, max_tokens=80 * 64)
    prompts = [random_ids(2 + i % 7, cfg["V"], 700 + i) for i in range(70)]
    got = s.generate(prompts, max_new_tokens=6, eos_ids=())
    for i in (0, 13, 63, 64, 69):
        assert got[i] == P.greedy(cfg, w, prompts[i], 6), i
    assert sorted(s.engine._runners) == [8, 64]          # capacities of the groups: 64, and 6 rounded up
    st = s.engine.manager.stats()
    assert st["pages_free"] == st["pages_total"] and st["slots_free"] == st["slots_total"]


@pytest.mark.parametrize("record", [False, True])
def test_a_hundred_and_fifty_requests_at_once_decode_through_the_loop_for_many_rows(folders, record):
    """In bfloat16 more requests than the weight-streaming products take rows (64) decode through a recording of the
    loop with the many-row products (a capacity of 256 here, then 128 and the fused loop as requests end); steps that
    hold prompt portions beside their tokens are launched, or with ``record_portions`` replayed.  The tokens are ones the
    plain logits support, requests end at different lengths and their pages and slots come back."""
    from gesso_amd import Session
    from gesso_amd.parts import RuntimeOptions
    d = write_tiny(folders, "D", torch.bfloat16)
    cfg, w = P.read_config(d), P.read_weights(d)
    n = 150
    s = Session(d, dtype="bfloat16", context_length=96, max_num_seqs=160, max_tokens=160 * 96,
                kernel_options=RuntimeOptions(record_portions=record))
    assert s.engine.DECODE_WIDE_MAX >= 256
    prompts = [random_ids(3 + i % 11, cfg["V"], 900 + i) for i in range(n)]
    stops = {}                                          # some requests stop early, so that the steps shrink
    got = s.generate(prompts, max_new_tokens=12, eos_ids=(),
                     on_token=lambda i, tok: stops.setdefault(i, 0) is None or (stops.__setitem__(i, stops[i] + 1) or stops[i] < 6 + i % 7))
    assert 256 in s.engine._runners, sorted(s.engine._runners)
    if record:
        assert not s.engine.recorder.refused
    for i in (0, 7, 64, 128, 149):
        p, g = prompts[i], got[i]
        assert len(g) - len(p) == 6 + i % 7, (i, len(g) - len(p))
        ref = P.forward(cfg, w, g[:-1])
        slack = 2 * WORST * float((P.forward(cfg, w, g[:-1], store=P.to_bfloat16) - ref).abs().max())
        for j in range(len(p), len(g)):
            assert supported(ref[j - 1], g[j], slack), (i, j, g[j], slack)
    st = s.engine.manager.stats()
    assert st["pages_free"] == st["pages_total"] and st["slots_free"] == st["slots_total"]
    # every row drawing from a nucleus, on the device: one seed gives the same ids again, other ids than the greedy ones
    from gesso_amd import Sampler
    drawn = [s.generate(prompts, max_new_tokens=5, eos_ids=(), sampler=Sampler(0.9, 0.8, seed=11)) for _ in range(2)]
    assert drawn[0] == drawn[1]
    assert sum(a[len(p):len(p) + 5] != b[len(p):len(p) + 5] for a, b, p in zip(drawn[0], got, prompts)) > n // 2


def test_temperature_sampling_follows_the_plain_sampler(plain):
    from gesso_amd import Sampler, Session
    d, cfg, w = plain["B"]
    s = Session(d, dtype="float32", context_length=160, page_size=8, chunk_size=13)
    prompts = prompts_of("B")[:3]
    got = s.generate(prompts, max_new_tokens=12, sampler=Sampler(temperature=0.8, seed=7), eos_ids=())
    for i, (p, g) in enumerate(zip(prompts, got)):
        ids, state = list(p), 7 + i
        for _ in range(12):
            tok, state = P.sample_id(P.forward(cfg, w, ids)[-1].tolist(), 0.8, 1.0, state)
            ids.append(tok)
        assert g == ids
    # the same seed gives the same ids again; top_p narrows the choice and stays reproducible
    again = s.generate(prompts, max_new_tokens=12, temperature=0.8, seed=7, eos_ids=())
    assert again == got
    one = s.generate(prompts[2], max_new_tokens=8, temperature=0.8, top_p=0.5, seed=3, eos_ids=())
    ids, state = list(prompts[2]), 3
    for _ in range(8):
        tok, state = P.sample_id(P.forward(cfg, w, ids)[-1].tolist(), 0.8, 0.5, state)
        ids.append(tok)
    assert one == ids


def test_long_decoding_and_first_tokens(plain):
    """One token a step for 150 steps after a prompt of one token: every row against the plain model."""
    from gesso_amd import Engine, StepEntry
    d, cfg, w = plain["B"]
    ids = random_ids(151, cfg["V"], 77)
    ref = P.forward(cfg, w, ids).numpy()
    eng = Engine.from_folder(d, dtype="float32", page_size=8, max_tokens=192)
    eng.add_request("r")
    rows = [eng.step([StepEntry("r", [t], [0])])[0].cpu().numpy() for t in ids]
    got = np.stack(rows)
    d_first = np.abs(got[:2] - ref[:2]).max()
    assert d_first <= 1e-4 * max(1.0, np.abs(ref).max())            # the first tokens of a sequence
    assert np.abs(got - ref).max() <= 1e-4 * max(1.0, np.abs(ref).max())
    assert eng.length("r") == 151


def test_a_far_token_decides(plain):
    """The logits at the end depend on the first token through hundreds of cached keys."""
    from gesso_amd import Engine, StepEntry
    d, cfg, w = plain["A"]
    ids = random_ids(240, cfg["V"], 5)
    other = [(ids[0] + 1) % cfg["V"]] + ids[1:]
    ref_a, ref_b = P.forward(cfg, w, ids)[-1].numpy(), P.forward(cfg, w, other)[-1].numpy()
    assert np.abs(ref_a - ref_b).max() > 1e-3                        # it matters in the plain model ...
    eng = Engine.from_folder(d, dtype="float32", page_size=16, max_tokens=512)
    out = []
    for name, seq in (("a", ids), ("b", other)):
        eng.add_request(name)
        eng.step([StepEntry(name, seq[:200], [])])
        for t in seq[200:-1]:
            eng.step([StepEntry(name, [t], [])])
        out.append(eng.step([StepEntry(name, [seq[-1]], [0])])[0].cpu().numpy())
    scale = max(1.0, np.abs(ref_a).max())
    assert np.abs(out[0] - ref_a).max() <= 1e-4 * scale and np.abs(out[1] - ref_b).max() <= 1e-4 * scale


def test_preemption_on_the_gpu_changes_no_output(plain):
    from gesso_amd import Session
    d, cfg, w = plain["A"]
    prompts = [random_ids(n, cfg["V"], 50 + n) for n in (20, 33, 9, 41, 15)]
    roomy = Session(d, dtype="float32", context_length=128, max_tokens=1024)
    want = roomy.generate(prompts, max_new_tokens=20, eos_ids=())
    # with the margin at admission switched off, so that the pool runs dry in the middle of decoding; pages and slots
    # that come back are filled with NaN before they are used again: a request computed again must not see them
    tight = Session(d, dtype="float32", context_length=128, num_pages=7, page_size=16, chunk_size=16, max_num_seqs=3,
                    watermark=0.0, poison=True)
    got = tight.generate(prompts, max_new_tokens=20, eos_ids=())
    assert got == want
    assert tight.last_stats["preemptions"] > 0
    st = tight.engine.manager.stats()
    assert st["pages_free"] == [7] and st["slots_free"] == st["slots_total"]


def test_a_sampled_request_that_is_preempted_draws_on_where_it_stopped(plain):
    """Requests that draw at a temperature, in a pool so small that some are preempted and computed again: each must
    come out as in a roomy pool, token for token (the sampler's state is kept across the preemption, and a draw is made
    once per token, never again for a token that is already there)."""
    from gesso_amd import Sampler, Session
    d, cfg, w = plain["A"]
    prompts = [random_ids(n, cfg["V"], 90 + n) for n in (20, 33, 9, 41, 15)]
    roomy = Session(d, dtype="float32", context_length=128, max_tokens=1024)
    want = roomy.generate(prompts, max_new_tokens=20, sampler=Sampler(0.8, seed=7), eos_ids=())
    tight = Session(d, dtype="float32", context_length=128, num_pages=7, page_size=16, chunk_size=16, max_num_seqs=3,
                    watermark=0.0)
    got = tight.generate(prompts, max_new_tokens=20, sampler=Sampler(0.8, seed=7), eos_ids=())
    assert tight.last_stats["preemptions"] > 0
    assert got == want
    ids, state = list(prompts[0]), 7                       # and the roomy run is the plain sampler's
    for _ in range(20):
        tok, state = P.sample_id(P.forward(cfg, w, ids)[-1].tolist(), 0.8, 1.0, state)
        ids.append(tok)
    assert want[0] == ids


def test_poison_fills_what_is_given_back_and_a_read_past_the_end_shows_it(plain):
    from gesso_amd import Engine, StepEntry
    d, cfg, w = plain["A"]
    eng = Engine.from_folder(d, dtype="float32", page_size=8, num_pages=6, num_slots=2, poison=True)
    look = lambda: torch.stack([eng.storage.keys[0], eng.storage.values[0]], dim=1)    # (members, K/V, pages + 1, ...)
    assert bool(torch.isnan(look()[:, :, :-1]).all())                # nothing holds a stale value from the start
    ids = random_ids(13, cfg["V"], 31)
    eng.add_request("a")
    logits = eng.step([StepEntry("a", ids, [12])])
    ref = P.forward(cfg, w, ids)[-1]
    assert float((logits[0].double().cpu() - ref).abs().max()) <= 1e-4 * max(1.0, float(ref.abs().max()))
    pages = list(eng.manager.get("a").tables[0])
    slot = eng.manager.get("a").slot
    kv = look()
    assert len(pages) == 2 and not torch.isnan(kv[:, :, pages[0]]).any()
    # the second page holds rows 8..12; its last three rows belong to nobody yet
    assert not torch.isnan(kv[:, :, pages[1], :, :5]).any() and bool(torch.isnan(kv[:, :, pages[1], :, 5:]).all())
    # a read one row past the end, through the generic attention kernel: the NaN arrives on the host
    ops = eng.rt.ops
    m = eng.model.blocks[1].mixer.spec
    q = torch.ones((1, m.n_heads * m.head_dim), device=eng.device)
    table = torch.tensor([pages], dtype=torch.int32, device=eng.device)
    zero = torch.zeros(1, dtype=torch.int32, device=eng.device)

    def attend(last_key):
        pos = torch.tensor([last_key], dtype=torch.int32, device=eng.device)
        return ops.attention_generic(q, q.shape[1], kv[0, 0], kv[0, 1], pos, zero, table, 8, None, 0.25, m.n_heads,
                                     m.n_kv_heads, m.head_dim, 1)

    assert bool(torch.isfinite(attend(12)).all()) and bool(torch.isnan(attend(13)).any())
    eng.finish_request("a")
    eng.add_request("b")                                              # the next step poisons what "a" gave back
    eng.step([StepEntry("b", ids[:3], [])])
    held = eng.manager.get("b").tables[0]
    for p in pages:
        if p not in held:
            assert bool(torch.isnan(look()[:, :, p]).all())
    state = eng.storage.state[0]["history"]
    if eng.manager.get("b").slot != slot:
        assert bool(torch.isnan(state[slot]).all())
    assert not torch.isnan(state[eng.manager.get("b").slot]).any()


def test_a_step_that_fails_in_the_middle_releases_its_requests(plain):
    """A kernel refuses in the middle of the model (here: a feed-forward that raises at its second call): histories
    are partly advanced and pages partly written, so the step's requests are dropped whole; others are untouched."""
    from gesso_amd import Engine, StepEntry
    from gesso_amd.errors import InvalidPlan, KernelError, StepFailed
    d, cfg, w = plain["A"]
    eng = Engine.from_folder(d, dtype="float32", page_size=8, max_tokens=256, num_slots=4)
    ids = random_ids(20, cfg["V"], 8)
    eng.add_request("bystander")
    eng.step([StepEntry("bystander", ids[:9], [])])
    ffn = eng.model.blocks[2].ffn
    real, calls = ffn.forward, []

    def failing(x, ctx):
        calls.append(1)
        raise KernelError("refused, for the test")

    eng.add_request("a"); eng.add_request("b")
    ffn.forward = failing
    with pytest.raises(StepFailed) as info:
        eng.step([StepEntry("a", ids[:5], [4]), StepEntry("b", ids[:2], [])])
    ffn.forward = real
    assert calls and sorted(info.value.detail["requests"]) == ["a", "b"] and isinstance(info.value.__cause__, KernelError)
    assert not eng.has_request("a") and not eng.has_request("b") and eng.has_request("bystander")
    eng.manager.check()
    with pytest.raises(InvalidPlan, match="not live"):
        eng.step([StepEntry("a", ids[5:7], [])])
    # the bystander goes on as if nothing had happened, and a new request under the old name starts from nothing
    got = eng.step([StepEntry("bystander", ids[9:], [len(ids) - 10])])[0].double().cpu()
    ref = P.forward(cfg, w, ids)
    assert float((got - ref[-1]).abs().max()) <= 1e-4 * max(1.0, float(ref.abs().max()))
    eng.add_request("a")
    got = eng.step([StepEntry("a", ids[:5], [4])])[0].double().cpu()
    assert float((got - ref[4]).abs().max()) <= 1e-4 * max(1.0, float(ref.abs().max()))


def test_a_pass_that_breaks_off_inside_a_scheduled_run_fails_its_requests_only(plain):
    """``run_batch`` with room for two requests at a time: the step that holds the first two prompts breaks off in the
    middle of the model (a feed-forward that raises once).  Those two end as failed with nothing generated; the third,
    admitted afterwards, generates what the plain model does; every page and slot is back (the reference stops only
    the request whose pass failed, ``src/Runtime/Runtime.jl:175-178``)."""
    from gesso_amd import BatchRequest, Session, run_batch
    from gesso_amd.errors import KernelError, StepFailed
    d, cfg, w = plain["A"]
    s = Session(d, dtype="float32", context_length=64, max_tokens=256, max_num_seqs=2, page_size=8)
    ffn = s.engine.model.blocks[1].ffn
    real, calls = ffn.forward, []

    def failing_once(x, ctx):
        calls.append(1)
        if len(calls) == 1:
            raise KernelError("refused, for the test")
        return real(x, ctx)

    ffn.forward = failing_once
    p = [random_ids(n, cfg["V"], 30 + n) for n in (6, 11, 9)]
    try:
        res = run_batch([BatchRequest(s, p[0], max_new_tokens=5), BatchRequest(s, p[1], max_new_tokens=5),
                         BatchRequest(s, p[2], max_new_tokens=7)])
    finally:
        ffn.forward = real
    assert [r.status for r in res] == ["failed", "failed", "complete"]
    assert all(isinstance(r.error, StepFailed) and isinstance(r.error.__cause__, KernelError) for r in res[:2])
    assert res[0].ids == p[0] and res[1].ids == p[1]
    assert res[2].ids == P.greedy(cfg, w, p[2], 7)
    st = s.engine.manager.stats()
    assert st["pages_free"] == st["pages_total"] and st["slots_free"] == st["slots_total"]
    s.engine.manager.check()
    # and the session serves on: the two that failed come out right when asked again
    got = s.generate(p[:2], max_new_tokens=5, eos_ids=())
    assert got == [P.greedy(cfg, w, q, 5) for q in p[:2]]


def test_one_requests_failure_leaves_the_others_their_results(plain):
    from gesso_amd import BatchRequest, Session, run_batch
    from gesso_amd.errors import InvalidPlan, ResourceLimit
    d, cfg, w = plain["A"]
    s = Session(d, dtype="float32", context_length=48, max_tokens=256)
    p = random_ids(6, cfg["V"], 9)
    long = random_ids(40, cfg["V"], 10)
    # run_batch: a request whose new tokens outgrow the context fails when it gets there; the others complete
    res = run_batch([BatchRequest(s, p, max_new_tokens=5), BatchRequest(s, long, max_new_tokens=20),
                     BatchRequest(s, p[:3], max_new_tokens=4), BatchRequest(s, [1, 999999], max_new_tokens=2)])
    assert [r.status for r in res] == ["complete", "failed", "complete", "failed"]
    assert isinstance(res[1].error, ResourceLimit) and isinstance(res[3].error, InvalidPlan)
    assert res[0].ids == P.greedy(cfg, w, p, 5) and res[2].ids == P.greedy(cfg, w, p[:3], 4)
    assert res[1].ids == P.greedy(cfg, w, long, 9)            # 48 tokens in the cache, and the token chosen from them
    # generate: the failure is raised after all have run; what the others made is at hand
    with pytest.raises(InvalidPlan, match="outside the vocabulary") as info:
        s.generate([p, [1, 999999], p[:3]], max_new_tokens=4)
    results = info.value.detail["results"]
    assert [r.status for r in results] == ["complete", "failed", "complete"] and results is s.last_results
    assert results[0].ids == P.greedy(cfg, w, p, 4) and results[2].ids == P.greedy(cfg, w, p[:3], 4)
    st = s.engine.manager.stats()
    assert st["pages_free"] == st["pages_total"] and st["slots_free"] == st["slots_total"]


def test_run_batch_statuses_and_cancel(plain):
    from gesso_amd import BatchRequest, Session, cancel, run_batch
    d, cfg, w = plain["B"]       # the untied model: its greedy tokens vary, so one of them can serve as the end
    s = Session(d, dtype="float32", context_length=64)
    p = random_ids(6, cfg["V"], 9)
    full = P.greedy(cfg, w, p, 8)
    new = full[6:]
    # an id that ends a request: the first new token that has not occurred before among the new ones, after the first
    k = next(i for i in range(1, 8) if new[i] not in new[:i])
    s.eos_ids = (new[k],)

    def until_eos(n):
        out = []
        for t in new[:n]:
            out.append(t)
            if t == new[k]:
                break
        return p + out

    reqs = [BatchRequest(s, p, max_new_tokens=8), BatchRequest(s, p, max_new_tokens=1),
            BatchRequest(s, p, max_new_tokens=8), BatchRequest(s, p[:3], max_new_tokens=0)]
    seen = []

    def on_token(i, tok):
        seen.append((i, tok))
        if i == 2:
            cancel(reqs[2])

    res = run_batch(reqs, on_token=on_token)
    assert [r.status for r in res] == ["eos", "complete", "cancelled", "complete"]
    assert res[0].ids == until_eos(8) and res[1].ids == p + new[:1] and res[2].ids == p + new[:1] and res[3].ids == p[:3]
    assert [t for i, t in seen if i == 0] == res[0].ids[6:]
    with pytest.raises(Exception):
        BatchRequest(s, p, max_new_tokens=-1)


def test_non_finite_logits_fail_their_request(folders):
    from gesso_amd import BatchRequest, Session, run_batch
    from gesso_amd.errors import InvalidPlan, NumericalInstability
    d = write_tiny(folders, "A", torch.float32)
    s = Session(d, dtype="float32", context_length=64)
    s.engine.model.final_norm.weight[3] = float("nan")               # a planted NaN
    res = run_batch([BatchRequest(s, [1, 2, 3], max_new_tokens=4)])
    assert res[0].status == "failed" and isinstance(res[0].error, NumericalInstability) and res[0].ids == [1, 2, 3]
    with pytest.raises(NumericalInstability):
        s.generate([1, 2, 3], max_new_tokens=2)
    with pytest.raises(InvalidPlan, match="outside the vocabulary"):
        s.generate([1, 999999], max_new_tokens=2)
    with pytest.raises(InvalidPlan, match="exceed the context"):
        s.generate(list(range(60)), max_new_tokens=10)
    st = s.engine.manager.stats()
    assert st["pages_free"] == st["pages_total"] and st["slots_free"] == st["slots_total"]


@pytest.mark.parametrize("bad_at", [4, 12])
def test_a_request_that_turns_non_finite_fails_alone_and_what_it_leaves_behind_harms_nobody(tmp_path, bad_at):
    """One request meets a token whose embedding row is NaN (in its first portion, or in a later one, after finite
    portions); its rows are NaN from there through every kernel, in steps it shares with the others (prompt portions of
    8 beside decoded tokens, bfloat16, heads of 64).  It fails alone; the others, of which two run later on the pages
    and the slot it gave back with NaN in them, produce what they produce without it."""
    import dataclasses
    from gesso_amd import BatchRequest, Session, run_batch
    from gesso_amd.errors import NumericalInstability
    from gesso_amd.weights import write_model_folder
    from tiny import TINY_D
    cfg = dataclasses.replace(TINY_D, tie_word_embeddings=False)
    d = write_model_folder(str(tmp_path / "m"), cfg, seed=4, dtype=torch.bfloat16, std=STD)
    prompts = [random_ids(n, cfg.vocab_size, 300 + n) for n in (20, 19, 33, 14)]
    kw = dict(dtype="bfloat16", context_length=96, page_size=4, max_num_seqs=2, num_pages=40, chunk_size=8,
              max_num_batched_tokens=12)
    clean = Session(d, **kw)
    want = [r.ids for r in run_batch([BatchRequest(clean, p, max_new_tokens=12) for p in prompts])]
    used = {t for g in want for t in g}
    nan_id = next(t for t in range(cfg.vocab_size) if t not in used)
    s = Session(d, **kw)
    s.engine.model.embed[nan_id] = float("nan")
    marred = prompts[1][:bad_at] + [nan_id] + prompts[1][bad_at + 1:]
    res = run_batch([BatchRequest(s, p, max_new_tokens=12) for p in (prompts[0], marred, prompts[2], prompts[3])])
    assert res[1].status == "failed" and isinstance(res[1].error, NumericalInstability)
    for i in (0, 2, 3):
        assert res[i].status != "failed" and res[i].ids == want[i], i
    st = s.engine.manager.stats()
    assert st["pages_free"] == st["pages_total"] and st["slots_free"] == st["slots_total"]


@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
@pytest.mark.parametrize("name", ["A", "B", "D"])
def test_nothing_reads_what_nobody_wrote(folders, monkeypatch, name, dtype):
    """Every buffer that the engine asks for without a value (``torch.empty``: activations, partial results, tiled rows
    with their padding) starts as NaN instead of whatever the allocator held: the tokens of five requests, in portions
    beside decoded tokens and through the recorded loop, are the same as without."""
    from gesso_amd import Session
    d = write_tiny(folders, name, torch.bfloat16 if dtype == "bfloat16" else torch.float32)
    cfg, seed = CONFIGS[name]
    prompts = [random_ids(n, cfg.vocab_size, 10 * seed + n) for n in (3, 22, 45, 70, 17)]
    kw = dict(dtype=dtype, context_length=160, page_size=4, max_num_seqs=3, num_pages=96, chunk_size=16,
              max_num_batched_tokens=24)
    want = Session(d, **kw).generate(prompts, max_new_tokens=20, eos_ids=())
    real = torch.empty

    def nan_empty(*a, **k):
        t = real(*a, **k)
        if t.is_floating_point() and t.is_cuda:
            t.fill_(float("nan"))
        return t

    monkeypatch.setattr(torch, "empty", nan_empty)
    got = Session(d, **kw).generate(prompts, max_new_tokens=20, eos_ids=())
    assert got == want


def test_a_cache_sized_by_a_share_of_the_free_memory(folders):
    """``memory_fraction``: as many pages as that share of the free device memory holds, and they serve."""
    from gesso_amd import Engine, Session
    from gesso_amd.errors import InvalidPlan

    d = write_tiny(folders, "A", torch.bfloat16)
    free, _ = torch.cuda.mem_get_info(0)
    eng = Engine.from_folder(d, dtype="bfloat16", page_size=16, memory_fraction=1e-4)
    cfg = CONFIGS["A"][0]
    n_attn = sum(t == "full_attention" for t in cfg.layer_types)
    per_page = n_attn * cfg.num_key_value_heads * 16 * 2 * cfg.head_dim * 2
    pages = eng.manager.stats()["pages_total"][0]
    assert 0.8 * (free * 1e-4 / per_page) <= pages <= free * 1e-4 / per_page, (pages, free, per_page)
    assert eng.storage.keys[0].shape[1] == pages + 1
    with pytest.raises(InvalidPlan, match="memory_fraction"):
        Engine.from_folder(d, dtype="bfloat16", memory_fraction=1.5)
    with pytest.raises(InvalidPlan, match="num_pages, max_tokens or memory_fraction"):
        Engine.from_folder(d, dtype="bfloat16")
    s = Session(d, dtype="bfloat16", memory_fraction=1e-4)
    roomy = Session(d, dtype="bfloat16")
    prompt = random_ids(40, cfg.vocab_size, 5)
    assert s.generate(prompt, max_new_tokens=8) == roomy.generate(prompt, max_new_tokens=8)


def test_random_weights_session_and_cli(tmp_path):
    from gesso_amd import Session
    s = Session(TINY_B, random_weights_seed=4, random_weights_std=STD, dtype="bfloat16", context_length=64)
    a = s.generate([5, 6, 7], max_new_tokens=5, eos_ids=())
    assert len(a) == 8 and a == s.generate([5, 6, 7], max_new_tokens=5, eos_ids=())
    env = dict(os.environ, PYTHONPATH=ROOT)
    r = subprocess.run([sys.executable, "-m", "gesso_amd", "--check"], capture_output=True, text=True, env=env, cwd=ROOT)
    assert r.returncode == 0 and "check ok" in r.stdout, r.stderr[-2000:]
    d = write_tiny(str(tmp_path), "A", torch.float32)
    r = subprocess.run([sys.executable, "-m", "gesso_amd", "--model", d, "--dtype", "float32", "--prompt-ids", "1,2,3",
                        "--prompt-ids", "9 8", "--max-new-tokens", "4", "--n-ctx", "32", "--model-id", "tiny-a"],
                       capture_output=True, text=True, env=env, cwd=ROOT)
    assert r.returncode == 0, r.stderr[-2000:]
    out = json.loads(r.stdout.strip().splitlines()[-1])
    cfg, w = P.read_config(d), P.read_weights(d)
    assert out["model"] == "tiny-a" and out["ids"][0][:3] == [1, 2, 3] and len(out["ids"][1]) <= 6
    assert out["ids"][0] == P.greedy(cfg, w, [1, 2, 3], 4)[:len(out["ids"][0])]
    r = subprocess.run([sys.executable, "-m", "gesso_amd", "--model", d, "--gguf", "x"], capture_output=True, text=True,
                       env=env, cwd=ROOT)
    assert r.returncode != 0 and "unrecognized" in r.stderr


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_recorded_decode_loop_equals_single_steps(folders, name, dtype):
    """Replays of the recorded step, several runs with other work between them, against step-by-step decoding."""
    from gesso_amd import Engine, Sampler, StepEntry
    d = write_tiny(folders, name, torch.float32 if dtype == "float32" else torch.bfloat16)
    cfg, _ = CONFIGS[name]
    prompts = [random_ids(n, cfg.vocab_size, 300 + n) for n in (7, 19, 33)]
    # float32: one request draws at a temperature; bfloat16: all greedy, so that each token can be held against the
    # plain logits (a draw has no such check: where it falls depends on every logit's rounding)
    samplers = lambda: [None, Sampler(0.8, 1.0, 5) if dtype == "float32" else None, None]

    def prefill(eng):
        firsts = []
        for i, p in enumerate(prompts):
            eng.add_request(i)
            firsts.append(int(eng.step([StepEntry(i, p, [len(p) - 1])]).argmax()))
        return firsts

    # step by step through the plain step function
    eng = Engine.from_folder(d, dtype=dtype, page_size=8, max_tokens=512)
    toks, sm, ref = prefill(eng), samplers(), []
    from gesso_amd.sampling import choose
    for _ in range(21):
        logits = eng.step([StepEntry(i, [t], [0]) for i, t in enumerate(toks)])
        toks = choose(eng.rt.ops, logits, sm)
        ref.append(list(toks))
    # the recorded loop: runs of 1, 8, 5 and 7 steps, with unrelated work between the runs
    eng2 = Engine.from_folder(d, dtype=dtype, page_size=8, max_tokens=512)
    first = prefill(eng2)
    toks, sm, got = list(first), samplers(), []
    for n in (1, 8, 5, 7):
        ids, bad = eng2.decode([0, 1, 2], toks, n, sm)
        assert not bad.any()
        got += ids.tolist()
        toks = ids[-1].tolist()
        eng2.add_request("other")                        # eager work and a synchronisation between replays
        eng2.step([StepEntry("other", prompts[0], [0])])
        eng2.finish_request("other")
        torch.cuda.synchronize()
    if dtype == "float32":
        assert got == ref
    else:
        # bfloat16: the recorded loop's fused kernels round elsewhere than the step-by-step ones, so a near-tie may fall
        # the other way; every token it chose must be the plain model's best, or as good within the logits' tolerance
        cfgp, w = P.read_config(d), P.read_weights(d)
        for i, p in enumerate(prompts):
            seq = list(p) + [first[i]] + [row[i] for row in got]
            plain_rows = P.forward(cfgp, w, seq[:-1])
            slack = 2 * WORST * float((P.forward(cfgp, w, seq[:-1], store=P.to_bfloat16) - plain_rows).abs().max())
            for at in range(len(p) + 1, len(seq)):
                assert supported(plain_rows[at - 1], seq[at], slack), (i, at, slack)
    assert [eng2.length(i) for i in range(3)] == [len(p) + 21 for p in prompts]


@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
@pytest.mark.parametrize("nreq,steps", [(3, 20), (20, 4), (40, 4), (70, 3), (130, 2)])
def test_recorded_decode_logits_follow_the_plain_model(folders, name, nreq, steps):
    """The fused kernels of the recorded step, row by row against the plain implementation (bfloat16): few rows
    (rows pre-weighted for the next norm), more than sixteen, and more than thirty-two (products in parts of K); and
    more than sixty-four, in capacities of 128 and 256: the loop with the many-row products."""
    from gesso_amd import Engine, StepEntry
    from gesso_amd.engine.decode import _capacity
    d = write_tiny(folders, name, torch.bfloat16)
    cfg, w = P.read_config(d), P.read_weights(d)
    prompts = [random_ids(n, cfg["V"], 700 + n) for n in ([3, 18, 40] + [5 + (7 * i) % 23 for i in range(nreq)])[:nreq]]
    eng = Engine.from_folder(d, dtype="bfloat16", page_size=16, max_tokens=64 * nreq + 256, num_slots=nreq + 1)
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
    bound = NoiseBound()
    for i, s in enumerate(seqs):          # a row of the whole sequence's logits is the last row of its prefix's
        ref, rounded = P.forward(cfg, w, s), P.forward(cfg, w, s, store=P.to_bfloat16)
        for step in range(steps):
            at = len(s) - steps + step
            bound.add(kept[step][i], ref[at], rounded[at], (step, i))
    bound.check(f"{name}, recorded decode of {nreq} requests,")


def test_recorded_decode_across_a_bound_on_the_context(tmp_path):
    """The decode step is recorded per bound on the context length (1024, 2048, ...); a request that grows past a
    bound moves to another recording in the middle of its decoding, and its logits stay those of the plain model."""
    import dataclasses
    from gesso_amd import Engine, StepEntry
    from gesso_amd.weights import write_model_folder
    from tiny import TINY_D, STD
    cfg_d = dataclasses.replace(TINY_D, max_position_embeddings=1536)
    d = write_model_folder(str(tmp_path / "long_d"), cfg_d, 11, torch.bfloat16, std=STD)
    cfg, w = P.read_config(d), P.read_weights(d)
    seq = random_ids(1010, cfg["V"], 4242)
    eng = Engine.from_folder(d, dtype="bfloat16", page_size=16, max_tokens=2048, num_slots=2)
    eng.add_request("r")
    tok = int(eng.step([StepEntry("r", seq, [len(seq) - 1])]).argmax())
    checked, bound = 0, NoiseBound()
    for step in range(24):
        seq.append(tok)
        ids, bad = eng.decode(["r"], [tok], 1)
        assert not bad.any()
        if len(seq) in (1020, 1023, 1024, 1025, 1030):          # around the bound: the second recording takes over
            logits = eng._runners[1].logits[0].double().cpu()
            bound.add(logits, P.forward(cfg, w, seq)[-1], P.forward(cfg, w, seq, store=P.to_bfloat16)[-1], len(seq))
            checked += 1
        tok = int(ids[0][0])
    bound.check("across a bound on the context,")
    assert checked == 5 and len(eng._runners[1].graphs) == 2


def test_a_full_run_before_a_new_recording_leaves_the_rings_alone(tmp_path):
    """A run of the most steps a run may have leaves every row's counter one past the rings; the recording that a
    longer context then asks for starts with an eager step, which must not write there.  Rows beside the rings are
    watched, and the tokens are those of the plain model."""
    import dataclasses
    from gesso_amd import Engine, StepEntry
    from gesso_amd.engine.decode import DecodeRunner
    from gesso_amd.weights import write_model_folder
    from tiny import TINY_D, STD
    cfg_d = dataclasses.replace(TINY_D, max_position_embeddings=1536)
    d = write_model_folder(str(tmp_path / "long_d"), cfg_d, 12, torch.bfloat16, std=STD)
    cfg, w = P.read_config(d), P.read_weights(d)
    seqs = [random_ids(n, cfg["V"], 5000 + n) for n in (960, 950, 957, 941)]
    eng = Engine.from_folder(d, dtype="bfloat16", page_size=16, max_tokens=4 * 1152, num_slots=5)
    runner = eng._runners[4] = DecodeRunner(eng, 4)
    steps = DecodeRunner.MAX_STEPS
    guard = {}
    for name in ("ring", "bad_ring"):                      # the rings as the middle rows of larger buffers
        big = torch.full((steps + 2, 4), -7, dtype=torch.int32, device=eng.device)
        guard[name] = big
        setattr(runner, name, big[1:steps + 1])
    toks = []
    for i, s in enumerate(seqs):
        eng.add_request(i)
        toks.append(int(eng.step([StepEntry(i, s, [len(s) - 1])]).argmax()))
    rids = list(range(4))
    bound = NoiseBound()
    for n in (steps, steps, 8):                             # 960 -> 992 -> 1024 (first recording), then beyond it
        ids, bad = eng.decode(rids, toks, n)
        assert not bad.any()
        for step in range(n):
            for s, t in zip(seqs, toks):
                s.append(t)
            toks = ids[step].tolist()
        logits = runner.logits[:4].double().cpu()          # of the run's last step
        for i, s in enumerate(seqs):
            bound.add(logits[i], P.forward(cfg, w, s)[-1], P.forward(cfg, w, s, store=P.to_bfloat16)[-1], (n, i))
    bound.check("full runs before a new recording,")
    assert len(runner.graphs) == 2
    for name, big in guard.items():
        assert bool((big[0] == -7).all()) and bool((big[-1] == -7).all()), f"a step wrote beside {name}"


def test_decode_stage_profiler(folders):
    """Stages of a decode step, timed by HIP events: disjoint, named as the reference names them, summing to less than
    the step; sub-stages beside them; the tokens are those of the unprofiled run; prompts are not counted."""
    from gesso_amd import Session
    d = write_tiny(folders, "B", torch.bfloat16)
    s = Session(d, dtype="bfloat16", context_length=96)
    prompts = [[3, 141, 59, 26, 500], [7, 8, 9]]
    want = s.generate(prompts, max_new_tokens=10, eos_ids=())
    prof = s.engine.profile_decode(True)
    got = s.generate(prompts, max_new_tokens=10, eos_ids=())
    assert got == want
    r = s.last_stats["decode_profile"]
    # the first token of each request comes from its prompt's step; the other nine from decode steps
    assert r["steps"] == 9 and r["step_ms"] > 0
    assert set(r["stages_ms"]) == {"embed", "conv_mixer", "attn_mixer", "norm", "dense_ffn", "lm_head", "sample"} - \
        ({"norm"} if r["stages_ms"].get("norm") is None else set())
    assert sum(r["stages_ms"].values()) <= r["step_ms"] * 1.001 and r["other_ms"] >= 0
    calls = r["calls_per_step"]
    assert calls["conv_mixer"] == 3 and calls["attn_mixer"] == 3 and calls["dense_ffn"] == 6 and calls["lm_head"] == 1
    assert {"conv_in", "conv_out", "attn_proj", "attn_core", "attn_outproj", "ffn_gateup", "ffn_down"} <= set(r["substages_ms"])
    assert r["substages_ms"]["ffn_gateup"] + r["substages_ms"]["ffn_down"] <= r["stages_ms"]["dense_ffn"] * 1.001
    s.engine.profile_decode(False)
    assert s.generate(prompts, max_new_tokens=10, eos_ids=()) == want and "decode_profile" not in s.last_stats
