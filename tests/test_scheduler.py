"""The scheduler's decisions, on a host-only stand-in for the engine.

The stand-in keeps the real cache manager, checks that every request's tokens arrive in order
and exactly once since its (re)admission, and answers with logits that depend on all tokens a
request has been fed, so that a request computed again after a preemption must come out the same.
"""
import numpy as np
import pytest

from gesso_amd.cache import CacheLayout, CacheManager
from gesso_amd.engine.scheduler import Request, Scheduler
from gesso_amd.errors import InvalidPlan, NumericalInstability, ResourceLimit
from gesso_amd.parts.base import PagedKV, SlotState
from gesso_amd.sampling.sampler import Sampler

V = 50


def next_token(tokens):
    h = 7
    for t in tokens:
        h = (h * 31 + t + 1) % 1000003
    return h % V


class FakeEngine:
    def __init__(self, num_pages=64, page_size=4, num_slots=8, max_length=256):
        lay = CacheLayout.plan([SlotState((("history", (4, 2), "float32"),)), PagedKV(1, 16, None)], [None, None])
        self.manager = CacheManager(lay, page_size, num_pages, num_slots, max_length)
        self.fed = {}
        self.batches = []

    def add_request(self, rid):
        self.manager.admit(rid)
        self.fed[rid] = []

    def finish_request(self, rid):
        self.manager.release(rid)
        del self.fed[rid]

    def step(self, entries):
        self.manager.reserve_many([(e.rid, len(e.tokens)) for e in entries])
        rows = []
        self.batches.append([(e.rid, len(e.tokens), list(e.want)) for e in entries])
        for e in entries:
            assert self.manager.get(e.rid).length == len(self.fed[e.rid])
            for i, t in enumerate(e.tokens):
                self.fed[e.rid].append(t)
                if i in e.want:
                    row = np.zeros(V, dtype=np.float32)
                    row[next_token(self.fed[e.rid])] = 1.0
                    rows.append(row)
            self.manager.commit(e.rid, len(e.tokens))
        self.manager.check()
        return np.stack(rows) if rows else None


def choose(logits, samplers):
    out = []
    for row, s in zip(logits, samplers):
        if not np.isfinite(row).all():
            out.append(NumericalInstability("non-finite logits"))
        elif s is None:
            out.append(int(np.argmax(row)))
        else:
            s.unit()
            out.append(int(np.argmax(row)))
    return out


def expected(prompt, n, eos=()):
    ids = list(prompt)
    for _ in range(n):
        t = next_token(ids)
        ids.append(t)
        if t in eos:
            break
    return ids


def make(engine=None, **kw):
    engine = engine or FakeEngine()
    return engine, Scheduler(engine, choose, **kw)


def test_single_request_chunks_then_decodes():
    eng, s = make(chunk_size=5, max_num_batched_tokens=16)
    r = s.add(Request("a", list(range(12)), max_new_tokens=3))
    s.run()
    assert r.tokens == expected(range(12), 3) and r.finish_reason == "complete"
    # portions of at most 5; only the last portion of the prompt asks for logits; then single tokens
    assert eng.batches == [[("a", 5, [])], [("a", 5, [])], [("a", 2, [1])], [("a", 1, [0])], [("a", 1, [0])]]
    assert eng.manager.stats()["pages_free"] == [64] and eng.manager.stats()["slots_free"] == 8
    assert s.stats["prompt_tokens"] == 12 and s.stats["decode_tokens"] == 3


def test_decodes_go_first_and_prompts_share_the_budget():
    eng, s = make(chunk_size=8, max_num_batched_tokens=10)
    a = s.add(Request("a", [1, 2, 3], max_new_tokens=6))
    s.step()                                            # a's whole prompt
    b = s.add(Request("b", list(range(20)), max_new_tokens=2))
    c = s.add(Request("c", list(range(5)), max_new_tokens=2))
    s.step()
    # a decodes (1 token), b gets a portion of 8, c the one token the budget has left
    assert eng.batches[-1] == [("a", 1, [0]), ("b", 8, []), ("c", 1, [])]
    s.step()
    assert eng.batches[-1] == [("a", 1, [0]), ("b", 8, []), ("c", 1, [])]
    s.run()
    for r, p in ((a, [1, 2, 3]), (b, range(20)), (c, range(5))):
        assert r.tokens == expected(p, r.max_new_tokens)
    assert sum(n for batch in eng.batches for _, n, _ in batch) == sum(len(r.tokens) - 1 for r in (a, b, c))
    assert all(sum(n for _, n, _ in batch) <= 10 for batch in eng.batches)


def test_max_num_seqs_and_slots_bound_admission():
    eng, s = make(FakeEngine(num_slots=2), max_num_seqs=3)
    rs = [s.add(Request(i, [i, i + 1], max_new_tokens=4)) for i in range(5)]
    s.step()
    assert len(s.running) == 2 and len(s.waiting) == 3           # two slots
    s.run()
    assert all(r.tokens == expected([i, i + 1], 4) for i, r in enumerate(rs))
    eng2, s2 = make(FakeEngine(num_slots=8), max_num_seqs=3)
    for i in range(5):
        s2.add(Request(i, [i], max_new_tokens=2))
    s2.step()
    assert len(s2.running) == 3


def test_eos_is_returned_and_not_fed():
    prompt = [3, 4, 5]
    full = expected(prompt, 6)
    eos = full[5]                                          # the third new token
    eng, s = make()
    r = s.add(Request("a", prompt, max_new_tokens=6, eos_ids=(eos,)))
    s.run()
    assert r.tokens == full[:6] and r.finish_reason == "eos"
    assert sum(n for b in eng.batches for _, n, _ in b) == 5   # 3 prompt tokens + 2 generated ones; the eos never
    r2 = s.add(Request("b", prompt, max_new_tokens=6, stop_ids=(eos,)))
    s.run()
    assert r2.tokens == full[:6] and r2.finish_reason == "eos"


def test_zero_budget_returns_the_prompt():
    eng, s = make()
    r = s.add(Request("a", [1, 2], max_new_tokens=0))
    assert r.finish_reason == "complete" and r.tokens == [1, 2] and not s.has_work() and eng.batches == []
    with pytest.raises(InvalidPlan):
        Request("b", [], max_new_tokens=1)
    with pytest.raises(InvalidPlan):
        Request("b", [1], max_new_tokens=-1)


def test_on_token_and_cancel():
    eng, s = make()
    seen = []
    a = s.add(Request("a", [1], max_new_tokens=10, on_token=lambda t: (seen.append(t), len(seen) < 3)[1]))
    b = s.add(Request("b", [2], max_new_tokens=10))
    c = s.add(Request("c", [3], max_new_tokens=10))
    c.cancelled = True                                     # cancelled before it ever ran
    s.step(); s.step()
    b.cancelled = True                                     # cancelled between tokens
    s.run()
    assert a.finish_reason == "cancelled" and len(a.output) == 3 and seen == a.output
    assert b.finish_reason == "cancelled" and len(b.output) == 2
    assert c.finish_reason == "cancelled" and c.output == []
    assert eng.manager.stats()["pages_free"] == [64] and eng.manager.stats()["slots_free"] == 8

    def boom(t):
        raise RuntimeError("callback failed")

    d = s.add(Request("d", [4], max_new_tokens=5, on_token=boom))
    e = s.add(Request("e", [5], max_new_tokens=5))
    s.run()
    assert d.finish_reason == "failed" and isinstance(d.error, RuntimeError)
    assert e.finish_reason == "complete" and e.tokens == expected([5], 5)   # one request's failure is its own


def test_out_of_pages_preempts_the_youngest_and_recomputes_it():
    # 6 pages of 4 = 24 tokens; two requests that grow to 16 each cannot both stay
    eng, s = make(FakeEngine(num_pages=6, page_size=4), chunk_size=8, max_num_batched_tokens=16)
    a = s.add(Request("a", list(range(8)), max_new_tokens=8, sampler=Sampler(0.7, 1.0, 1)))
    b = s.add(Request("b", list(range(10, 18)), max_new_tokens=8, sampler=Sampler(0.7, 1.0, 2)))
    s.run()
    assert s.stats["preemptions"] >= 1 and b.preemptions >= 1 and a.preemptions == 0
    assert a.tokens == expected(range(8), 8) and b.tokens == expected(range(10, 18), 8)
    # each sampler drew exactly once per token it emitted, preemption or not
    ref = Sampler(0.7, 1.0, 2)
    for _ in range(8):
        ref.unit()
    assert b.sampler.state == ref.state
    assert eng.manager.stats()["pages_free"] == [6]
    # the recomputation fed prompt and generated tokens again, from position 0
    fed_b = [n for batch in eng.batches for rid, n, _ in batch if rid == "b"]
    assert sum(fed_b) > len(b.tokens) - 1


def test_a_request_larger_than_the_pool_fails_alone():
    eng, s = make(FakeEngine(num_pages=3, page_size=4), chunk_size=8)
    big = s.add(Request("big", list(range(20)), max_new_tokens=2))
    ok = s.add(Request("ok", [1, 2, 3], max_new_tokens=2))
    s.run()
    assert big.finish_reason == "failed" and isinstance(big.error, ResourceLimit)
    assert ok.finish_reason == "complete" and ok.tokens == expected([1, 2, 3], 2)
    assert eng.manager.stats()["pages_free"] == [3] and eng.manager.stats()["slots_free"] == 8


def test_a_bad_row_fails_its_request_only():
    class Poisoned(FakeEngine):
        def step(self, entries):
            logits = super().step(entries)
            if logits is not None and entries[0].rid == "bad":
                logits[0, 3] = np.nan
            return logits

    eng, s = make(Poisoned())
    bad = s.add(Request("bad", [1, 2], max_new_tokens=3))
    good = s.add(Request("good", [5, 6], max_new_tokens=3))
    s.run()
    assert bad.finish_reason == "failed" and isinstance(bad.error, NumericalInstability) and bad.output == []
    assert good.tokens == expected([5, 6], 3)
    assert eng.manager.stats()["slots_free"] == 8


def test_many_requests_under_pressure_all_come_out_right():
    import random
    rng = random.Random(3)
    eng, s = make(FakeEngine(num_pages=20, page_size=4, num_slots=4), chunk_size=7, max_num_batched_tokens=12,
                  max_num_seqs=4)
    reqs = []
    for i in range(25):
        p = [rng.randrange(V) for _ in range(rng.randint(1, 30))]
        reqs.append((p, s.add(Request(i, p, max_new_tokens=rng.randint(1, 12)))))
    s.run()
    for p, r in reqs:
        assert r.finish_reason == "complete" and r.tokens == expected(p, r.max_new_tokens), r.rid
    assert eng.manager.stats()["pages_free"] == [20] and eng.manager.stats()["slots_free"] == 4
    assert s.stats["preemptions"] > 0


class FakeDecodeEngine(FakeEngine):
    """The stand-in with a recorded decode loop: n steps at once, tokens fed back inside."""

    DECODE_MAX_BATCH = 4

    def __init__(self, *a, **kw):
        super().__init__(*a, **kw)
        self.runs = []

    def decode(self, rids, tokens, n, samplers=None):
        self.manager.reserve_many([(r, n) for r in rids])
        self.runs.append((list(rids), n))
        ids = np.zeros((n, len(rids)), dtype=np.int64)
        bad = np.zeros((n, len(rids)), dtype=np.int64)
        toks = list(tokens)
        for s in range(n):
            for i, r in enumerate(rids):
                assert self.manager.get(r).length + s == len(self.fed[r])
                self.fed[r].append(toks[i])
                toks[i] = next_token(self.fed[r])
                ids[s, i] = toks[i]
                if samplers and samplers[i] is not None:
                    samplers[i].unit()
        for r in rids:
            self.manager.commit(r, n)
        self.manager.check()
        return ids, bad


def test_decode_runs_of_several_steps():
    eng, s = make(FakeDecodeEngine(), decode_run_steps=5)
    a = s.add(Request("a", [1, 2, 3], max_new_tokens=12))
    b = s.add(Request("b", [9], max_new_tokens=7, sampler=Sampler(0.9, 1.0, 3)))
    s.run()
    assert a.tokens == expected([1, 2, 3], 12) and b.tokens == expected([9], 7)
    # the first step holds a's prompt: an ordinary step; then runs of 5, bounded by what b may still generate
    assert eng.runs[0][1] == 5 and all(n <= 5 for _, n in eng.runs)
    assert sum(n for rids, n in eng.runs if "b" in rids) == 6            # b's first token came with a's prompt step
    ref = Sampler(0.9, 1.0, 3)
    for _ in range(7):
        ref.unit()
    assert b.sampler.state == ref.state
    assert eng.manager.stats()["pages_free"] == [64] and eng.manager.stats()["slots_free"] == 8


def test_more_requests_than_the_recorded_loop_takes_run_through_it_in_groups():
    """Six decoding requests, a loop that takes four at once: every run of steps goes through it as a group of four and
    a group of two, and every request gets what it gets alone."""
    eng, s = make(FakeDecodeEngine(), decode_run_steps=4, max_num_seqs=6)
    reqs = [s.add(Request(chr(97 + i), [i + 1, i + 2], max_new_tokens=6 + i)) for i in range(6)]
    s.run()
    for i, r in enumerate(reqs):
        assert r.tokens == expected([i + 1, i + 2], 6 + i), i
    sizes = [len(rids) for rids, _ in eng.runs]
    assert max(sizes) == 4 and [4, 2] == sizes[:2]
    assert eng.manager.stats()["pages_free"] == [64] and eng.manager.stats()["slots_free"] == 8


def test_a_request_that_ends_inside_a_run_keeps_its_tokens_up_to_there():
    full = expected([4, 5], 10)
    eos = full[2 + 3]
    eng, s = make(FakeDecodeEngine(), decode_run_steps=8)
    seen = []
    a = s.add(Request("a", [4, 5], max_new_tokens=10, eos_ids=(eos,)))
    b = s.add(Request("b", [6, 7], max_new_tokens=10, on_token=lambda t: (seen.append(t), len(seen) < 5)[1]))
    s.run()
    assert a.tokens == full[:6] and a.finish_reason == "eos"
    assert b.finish_reason == "cancelled" and b.tokens == expected([6, 7], 5) and seen == b.output
    assert eng.manager.stats()["pages_free"] == [64] and eng.manager.stats()["slots_free"] == 8


def test_while_someone_waits_runs_are_single_steps():
    eng, s = make(FakeDecodeEngine(num_slots=1), decode_run_steps=8)
    a = s.add(Request("a", [1, 2], max_new_tokens=4))
    b = s.add(Request("b", [3, 4], max_new_tokens=6))
    s.run()
    assert a.tokens == expected([1, 2], 4) and b.tokens == expected([3, 4], 6)
    assert all(n == 1 for rids, n in eng.runs if rids == ["a"])           # b waited for the slot
    assert any(n > 1 for rids, n in eng.runs if rids == ["b"])


def test_runs_shrink_to_the_pages_that_are_left_and_nucleus_requests_run_like_the_others():
    eng, s = make(FakeDecodeEngine(num_pages=3, page_size=4), decode_run_steps=8)
    a = s.add(Request("a", [1, 2, 3], max_new_tokens=8))
    s.run()
    assert a.tokens == expected([1, 2, 3], 8)
    eng2, s2 = make(FakeDecodeEngine(), decode_run_steps=8)
    c = s2.add(Request("c", [1, 2, 3], max_new_tokens=5, sampler=Sampler(0.9, 0.5, 3)))
    s2.run()
    assert c.tokens == expected([1, 2, 3], 5) and eng2.runs and eng2.runs[0][1] > 1


def test_a_request_that_outgrows_the_context_fails_alone_and_keeps_its_tokens():
    # b's prompt of 14 tokens fits a context of 16, its 8 new tokens do not: it fails when the 17th token would be fed
    for engine in (FakeEngine(max_length=16), FakeDecodeEngine(max_length=16)):
        eng, s = make(engine, decode_run_steps=8)
        a = s.add(Request("a", [1, 2, 3], max_new_tokens=6))
        b = s.add(Request("b", list(range(14)), max_new_tokens=8))
        c = s.add(Request("c", list(range(30)), max_new_tokens=1))            # never fits
        s.run()
        assert a.finish_reason == "complete" and a.tokens == expected([1, 2, 3], 6)
        assert b.finish_reason == "failed" and isinstance(b.error, ResourceLimit)
        # tokens at positions 14, 15, 16 were chosen from 14, 15 and 16 cached tokens; the next would need a 17th fed
        assert b.tokens == expected(range(14), 3)
        assert c.finish_reason == "failed" and isinstance(c.error, ResourceLimit) and c.output == []
        assert eng.manager.stats()["pages_free"] == [64] and eng.manager.stats()["slots_free"] == 8


def test_admission_leaves_the_watermark_free_for_those_who_run():
    # 10 pages of 4; a holds 5 after its prompt.  b's prompt needs 4: with a margin of 2 pages (0.2 of 10) it waits
    eng, s = make(FakeEngine(num_pages=10, page_size=4), chunk_size=32, max_num_batched_tokens=64, watermark=0.2)
    a = s.add(Request("a", list(range(20)), max_new_tokens=4))
    s.step()
    b = s.add(Request("b", list(range(16)), max_new_tokens=2))
    s.step()
    assert b.status == "waiting" and s.stats["preemptions"] == 0
    s.run()
    assert a.tokens == expected(range(20), 4) and b.tokens == expected(range(16), 2)
    assert s.stats["preemptions"] == 0
    # without a margin the same request is admitted at once
    eng2, s2 = make(FakeEngine(num_pages=10, page_size=4), chunk_size=32, max_num_batched_tokens=64, watermark=0.0)
    s2.add(Request("a", list(range(20)), max_new_tokens=4))
    s2.step()
    b2 = s2.add(Request("b", list(range(16)), max_new_tokens=2))
    s2.step()
    assert b2.status == "running"
    # an idle engine admits without the margin: a request that needs every page still runs
    eng3, s3 = make(FakeEngine(num_pages=4, page_size=4), chunk_size=32, max_num_batched_tokens=64, watermark=0.5)
    c = s3.add(Request("c", list(range(14)), max_new_tokens=2))
    s3.run()
    assert c.finish_reason == "complete" and c.tokens == expected(range(14), 2)
    with pytest.raises(InvalidPlan):
        make(watermark=1.0)


class FailingEngine(FakeEngine):
    """The stand-in with passes that break off as the engine's do: the requests of the pass are released, then
    ``StepFailed`` names them (``Engine.fail_requests``)."""

    def __init__(self, *a, fail_steps=(), fail_runs=(), **kw):
        super().__init__(*a, **kw)
        self.fail_steps, self.fail_runs = set(fail_steps), set(fail_runs)
        self.n_steps = self.n_runs = 0

    def has_request(self, rid):
        return rid in self.manager.requests

    def _break(self, rids):
        from gesso_amd.errors import StepFailed
        for r in rids:
            self.finish_request(r)
        return StepFailed("a kernel refused its sizes", requests=list(rids))

    def step(self, entries):
        self.n_steps += 1
        if self.n_steps in self.fail_steps:
            self.manager.reserve_many([(e.rid, len(e.tokens)) for e in entries])
            raise self._break([e.rid for e in entries])
        return super().step(entries)


class FailingDecodeEngine(FailingEngine, FakeDecodeEngine):
    def decode(self, rids, tokens, n, samplers=None):
        self.n_runs += 1
        if self.n_runs in self.fail_runs:
            self.manager.reserve_many([(r, n) for r in rids])
            raise self._break(rids)
        return super().decode(rids, tokens, n, samplers)


def test_a_step_that_breaks_off_fails_its_requests_and_nobody_else():
    """The second step (a decoding beside b's second portion) breaks off: both end as failed with what they had; c,
    which waited, comes out as it does alone; nothing is released twice, nothing is lost."""
    from gesso_amd.errors import StepFailed
    eng = FailingEngine(fail_steps={2})
    s = Scheduler(eng, choose, chunk_size=4, max_num_batched_tokens=8, max_num_seqs=2)
    a = s.add(Request("a", [1, 2, 3], max_new_tokens=5))
    b = s.add(Request("b", list(range(9)), max_new_tokens=3))
    c = s.add(Request("c", [7, 8], max_new_tokens=4))
    s.run()
    assert a.finish_reason == "failed" and isinstance(a.error, StepFailed) and a.tokens == expected([1, 2, 3], 1)
    assert b.finish_reason == "failed" and isinstance(b.error, StepFailed) and b.output == []
    assert c.finish_reason == "complete" and c.tokens == expected([7, 8], 4)
    assert s.stats["failed_passes"] == 1 and not s.running and not s.waiting
    assert eng.manager.stats()["pages_free"] == [64] and eng.manager.stats()["slots_free"] == 8
    eng.manager.check()


def test_a_group_of_a_decode_run_that_breaks_off_leaves_the_other_groups_their_tokens():
    """Six requests through a loop of four: the second group's first run breaks off.  Its two requests fail with the
    token their prompts gave them; the four of the first group keep the run's tokens and finish as they do alone."""
    from gesso_amd.errors import StepFailed
    eng = FailingDecodeEngine(fail_runs={2})
    s = Scheduler(eng, choose, decode_run_steps=4, max_num_seqs=6)
    reqs = [s.add(Request(chr(97 + i), [i + 1, i + 2], max_new_tokens=6)) for i in range(6)]
    s.run()
    for i, r in enumerate(reqs[:4]):
        assert r.finish_reason == "complete" and r.tokens == expected([i + 1, i + 2], 6), i
    for i, r in enumerate(reqs[4:], start=4):
        assert r.finish_reason == "failed" and isinstance(r.error, StepFailed), i
        assert r.tokens == expected([i + 1, i + 2], 1), i
    assert eng.manager.stats()["pages_free"] == [64] and eng.manager.stats()["slots_free"] == 8
    eng.manager.check()


def test_sub_tiles_of_prompt_attention_pair_late_queries_with_early_ones():
    """Every query row occurs once; a block's sub-tiles belong to one sequence; with pairing the (query, key) pairs
    of the blocks of one causal prompt differ by at most one sub-tile's worth, without it by the whole prompt's."""
    from gesso_amd.engine.batch import subtile_lists
    lens = [1, 1, 300, 2048, 33]
    for wq in (1, 2, 4, 8):
        for paired in (False, True):
            seq, row, cnt = subtile_lists(lens, wq, skip=2, paired=paired)
            assert len(seq) % wq == 0
            covered = sorted(r + j for r, c in zip(row, cnt) for j in range(c))
            assert covered == list(range(2, sum(lens)))
            for b in range(0, len(seq), wq):
                assert len(set(seq[b:b + wq])) == 1 and all(0 <= c <= 32 for c in cnt[b:b + wq])
    starts = [0, 1, 2, 302, 2350]

    def work(wq, paired):
        seq, row, cnt = subtile_lists(lens, wq, skip=2, paired=paired)
        out = []
        for b in range(0, len(seq), wq):
            if seq[b] == 3:
                out.append(sum((r - starts[3]) + c for r, c in zip(row[b:b + wq], cnt[b:b + wq]) if c))
        return out
    for wq in (2, 4, 8):
        even, uneven = work(wq, True), work(wq, False)
        assert max(even) - min(even) <= 32 * wq and max(uneven) - min(uneven) > 1500
    # the late sub-tiles stand in the first half of a block's entries, their partners in the second
    seq, row, cnt = subtile_lists([256], 4, 0, True)
    assert row[:4] == [224, 192, 0, 32] and row[4:] == [160, 128, 64, 96]
