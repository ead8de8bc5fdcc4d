"""Helpers for the replay tests: traces in the four ways of cutting, a driver for bin/trace_run,
and the plain implementation's logits to compare with."""
import json
import os
import random
import subprocess
import sys

import numpy as np
import torch

import plain_lfm2 as P

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TRACE_RUN = os.path.join(ROOT, "bin", "trace_run")


def plain_logits(model_dir: str, ids, rounded: bool = False) -> np.ndarray:
    """(T, V) float64 logits of the whole sequence by the plain implementation; ``rounded``: with its activations
    rounded to bfloat16 wherever a pipeline with bfloat16 activations stores one."""
    cfg = P.read_config(model_dir)
    w = P.read_weights(model_dir, torch.float64)
    return P.forward(cfg, w, list(ids), **({"store": P.to_bfloat16} if rounded else {})).numpy()


class Plain:
    """The plain logits of some sequences (``ref``), the rounded model's for bfloat16 (``rounded``), and the
    comparison of an engine's rows with them: float32 to ``1e-4 x max(1, max |ref|)`` at the worst logit (the
    reference's own device bound, ``test/test_amdgpu_lfm2.jl:34``), bfloat16 to the rounded model's own distance
    (``tests/noise.py``)."""

    F32 = 1e-4

    def __init__(self, model_dir: str, seqs: dict, dtype: str):
        self.dtype = dtype
        self.ref = {k: plain_logits(model_dir, ids) for k, ids in seqs.items()}
        self.rounded = {k: plain_logits(model_dir, ids, rounded=True) for k, ids in seqs.items()} \
            if dtype == "bfloat16" else None
        self.scale = max(1.0, max(float(np.abs(r).max()) for r in self.ref.values()))

    def check(self, got: dict, label: str) -> None:
        """``got``: {sequence name: {position: logits row}}."""
        if self.dtype == "float32":
            w, where = worst(got, self.ref)
            print(f"{label} float32: worst |diff| {w:.3e} at {where} (bound {self.F32 * self.scale:.3e})")
            assert w <= self.F32 * self.scale, f"{label}: first look at {where}"
            return
        from noise import NoiseBound
        b = NoiseBound()
        for name, rows in got.items():
            for pos, row in rows.items():
                b.add(row, self.ref[name][pos], self.rounded[name][pos], (name, pos))
        b.check(label)


def round64(n: int) -> int:
    return -(-n // 64) * 64


class Trace:
    """Steps for trace_run, with a record of which (sequence, position) each wanted row is."""

    def __init__(self):
        self.steps = []
        self.rows = []          # per step: list of (seq name, position)
        self.held = {}          # live request -> tokens held
        self.max_tokens = 0

    def add(self, entries, end=()):
        """entries: list of (name, start position, tokens); every fed position is wanted."""
        rec = {"step": len(self.steps), "entries": [], "end": list(end)}
        rows = []
        for name, start, toks in entries:
            assert self.held.get(name, 0) == start, (name, start, self.held.get(name))
            rec["entries"].append({"id": name, "tokens": list(toks), "want": list(range(len(toks)))})
            rows += [(name, start + i) for i in range(len(toks))]
            self.held[name] = start + len(toks)
        self.max_tokens = max(self.max_tokens, sum(round64(n) for n in self.held.values()))
        for name in end:
            del self.held[name]
        self.steps.append(rec)
        self.rows.append(rows)
        assert len(self.held) <= 4


def trace_whole(seqs) -> Trace:
    t = Trace()
    for name, ids in seqs.items():
        t.add([(name, 0, ids)], end=[name])
    return t


def trace_tail(seqs, tail=32) -> Trace:
    """Most of a sequence in one step, its last `tail` tokens one by one."""
    t = Trace()
    for name, ids in seqs.items():
        head = max(1, len(ids) - tail)
        t.add([(name, 0, ids[:head])])
        for i in range(head, len(ids)):
            t.add([(name, i, ids[i:i + 1])], end=[name] if i == len(ids) - 1 else [])
        if head == len(ids):
            t.steps[-1]["end"] = [name]
            del t.held[name]
    return t


def trace_portions(seqs, sizes=(7, 13, 2, 5, 3, 16, 2, 31, 1, 17)) -> Trace:
    t = Trace()
    k = 0
    for name, ids in seqs.items():
        at = 0
        while at < len(ids):
            n = min(sizes[k % len(sizes)], len(ids) - at)
            k += 1
            t.add([(name, at, ids[at:at + n])], end=[name] if at + n == len(ids) else [])
            at += n
    return t


def trace_mixed(seqs, seed=0, live=4, decode_tail=12) -> Trace:
    """Up to `live` requests at a time; portions of some beside single tokens of others; some sit a step out."""
    rng = random.Random(seed)
    t = Trace()
    waiting = list(seqs.items())
    running = {}                       # name -> [ids, position]
    while waiting or running:
        while waiting and len(running) < live:
            name, ids = waiting.pop(0)
            running[name] = [ids, 0]
        entries, end = [], []
        for name, (ids, at) in list(running.items()):
            if len(running) > 1 and rng.random() < 0.2:
                continue               # left out of this step, goes on later
            left = len(ids) - at
            if left <= decode_tail:
                n = 1
            else:
                n = min(rng.choice((2, 3, 5, 7, 13, 16, 17, 29)), left - decode_tail) or 1
            entries.append((name, at, ids[at:at + n]))
            running[name][1] = at + n
            if at + n == len(ids):
                end.append(name)
                del running[name]
        if entries:
            t.add(entries, end=end)
    return t


class TraceRun:
    """A running bin/trace_run; steps go in one by one, each answered by `done <step>`."""

    def __init__(self, model_dir, dtype, out_dir, max_tokens, extra=()):
        os.makedirs(out_dir, exist_ok=True)
        self.out_dir = out_dir
        self.proc = subprocess.Popen(
            [sys.executable, TRACE_RUN, "--model", model_dir, "--dtype", dtype, "--out", out_dir,
             "--max-tokens", str(max_tokens), *extra],
            stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True, bufsize=1)

    def step(self, rec) -> None:
        self.proc.stdin.write(json.dumps(rec) + "\n")
        self.proc.stdin.flush()
        line = self.proc.stdout.readline()
        if line.strip() != f"done {rec['step']}":
            rc = self.proc.poll()
            raise RuntimeError(f"trace_run answered {line!r} to step {rec['step']} (exit status {rc})")

    def logits(self, step: int, vocab: int) -> np.ndarray:
        return np.fromfile(os.path.join(self.out_dir, f"{step}.f32"), dtype="<f4").reshape(-1, vocab)

    def close(self) -> int:
        self.proc.stdin.close()
        rc = self.proc.wait(timeout=60)
        return rc


def run_trace(model_dir, dtype, out_dir, trace: Trace, vocab: int, max_tokens=None, page_size=None, extra=()):
    """Replay `trace`; returns {name: {position: logits row}} and the exit status."""
    extra = list(extra) + (["--page-size", str(page_size)] if page_size is not None else [])
    tr = TraceRun(model_dir, dtype, out_dir, max_tokens or trace.max_tokens, extra=extra)
    got = {}
    try:
        for rec, rows in zip(trace.steps, trace.rows):
            tr.step(rec)
            if rows:
                lg = tr.logits(rec["step"], vocab)
                assert lg.shape[0] == len(rows), (lg.shape, len(rows))
                for (name, pos), row in zip(rows, lg):
                    got.setdefault(name, {})[pos] = row
    finally:
        rc = tr.close()
    return got, rc


def worst(got, ref):
    """Largest absolute difference over all positions, with the place it occurs."""
    w, where = 0.0, None
    for name, rows in got.items():
        for pos, row in rows.items():
            d = float(np.abs(row.astype(np.float64) - ref[name][pos]).max())
            if not np.isfinite(d):
                return float("inf"), (name, pos)
            if d > w:
                w, where = d, (name, pos)
    return w, where


def visit_trace(model_dir, dtype, out_dir, trace: Trace, vocab: int, visit, max_tokens=None, extra=()):
    """Replay `trace` and hand every wanted row to `visit(name, position, row)` as it comes (nothing is kept: for
    vocabularies of tens of thousands).  Returns the exit status."""
    tr = TraceRun(model_dir, dtype, out_dir, max_tokens or trace.max_tokens, extra=extra)
    try:
        for rec, rows in zip(trace.steps, trace.rows):
            tr.step(rec)
            if rows:
                lg = tr.logits(rec["step"], vocab)
                os.remove(os.path.join(out_dir, f"{rec['step']}.f32"))
                assert lg.shape[0] == len(rows), (lg.shape, len(rows))
                for (name, pos), row in zip(rows, lg):
                    visit(name, pos, row.astype(np.float64))
    finally:
        rc = tr.close()
    return rc


class Distance:
    """Running largest and root-mean-square difference between rows, with the place of the largest."""

    def __init__(self):
        self.worst, self.where, self.sq, self.n = 0.0, None, 0.0, 0

    def add(self, a, b, where):
        d = np.abs(a - b)
        m = float(d.max())
        if not np.isfinite(m):
            m = float("inf")
        if m > self.worst:
            self.worst, self.where = m, where
        self.sq += float((d * d).sum())
        self.n += d.size

    @property
    def rms(self):
        return (self.sq / max(1, self.n)) ** 0.5
