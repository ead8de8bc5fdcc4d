"""The decode fast path: steps in which every request brings one token, recorded once as a HIP graph.

A decode step of a small batch is bound by launch overhead, not by arithmetic: more than a
hundred kernels of a few microseconds each.  So the step (embedding, all blocks, head, the choice
of the next token, the advance of positions) is recorded into a graph per batch capacity and
replayed; everything that changes between steps lives in device buffers the kernels read
(tokens, positions, block tables, slots, the rows' step counters).  The token a step chooses is written
where the next step's embedding reads it, so ``n`` steps run back to back without the host; the
host reads the chosen tokens once per call.  The reference decodes one row per call with one
host round trip per token (``src/Inference/Inference.jl:2547-2712``).

Rows beyond the live batch (the capacity is the batch rounded up to a power of two, or to 48) point at the
scratch page and the scratch slot, so they compute and write garbage that nobody reads.

Graph hygiene: nothing in the graph clears memory with a memset node; the step counters are reset by
an ordinary fill before the replays.
"""
from __future__ import annotations

import gc

from typing import Dict, Hashable, List, Sequence, Tuple

import numpy as np
import torch

from ..errors import InvalidPlan
from .batch import BatchContext


def _capacity(n: int) -> int:
    """The batch rounded up to a power of two, or to 48: the products take rows in tiles of 16, and a step of three
    tiles is measurably shorter than one of four.  (The most requests a step takes is the engine's
    ``DECODE_MAX_BATCH``, which it has from the runtime's product kernels.)"""
    c = 1
    while c < n:
        c *= 2
    return 48 if 32 < n <= 48 else c


class DecodeContext(BatchContext):
    """The recorded decode step as the parts see it: every field a static device buffer of the runner, or a fact
    that holds for every replay (one token per sequence, every row wanted, in order)."""

    def __init__(self, runner):
        r = runner
        self._set(r.engine.storage, T=r.cap, nseq=r.cap, n_want=r.cap, q_lens=[1] * r.cap, all_single=True,
                  max_q_len=1, max_kv_len=None, decode_only=True, token_ids=r.tok, positions=r.pos,
                  seq_of_token=r.seq_of_token, q_start=r.q_start, kv_len=r.kv_len, slots=r.slots,
                  want_rows=r.seq_of_token, block_tables=r.block_tables)


class DecodeRunner:
    """Static buffers and the recorded graph for one batch capacity."""

    MAX_STEPS = 32

    def __init__(self, engine, cap: int):
        self.engine, self.cap = engine, cap
        dev = engine.device
        i32 = dict(dtype=torch.int32, device=dev)
        self.max_blocks = -(-engine.max_context // engine.page_size)
        st = engine.storage
        self.tok = torch.zeros(cap, **i32)
        self.pos = torch.zeros(cap, **i32)
        self.kv_len = torch.ones(cap, **i32)
        self.slots = torch.full((cap,), st.scratch_slot, **i32)
        self.live = torch.zeros(cap, **i32)
        self.seq_of_token = torch.arange(cap, **i32)
        self.q_start = torch.arange(cap + 1, **i32)
        self.block_tables = [torch.full((cap, self.max_blocks), n, **i32) for n in st.num_pages]
        self.temperature = torch.zeros(cap, dtype=torch.float64, device=dev)
        self.top_p = torch.ones(cap, dtype=torch.float64, device=dev)
        self.weights, self.wide = engine.choice_scratch(max(cap, engine.DECODE_MAX_BATCH))      # shared by all capacities
        self.u = torch.zeros((self.MAX_STEPS, cap), dtype=torch.float64, device=dev)
        self.counter = torch.zeros(cap, **i32)          # steps made since the host last looked, per row
        self.ring = torch.zeros((self.MAX_STEPS, cap), **i32)
        self.bad_ring = torch.zeros((self.MAX_STEPS, cap), **i32)
        self.ctx = DecodeContext(self)
        # one recording per bound on the context length (launch shapes, how attention splits its keys, depend on it)
        # and per kind of choice: all rows greedy (one kernel), or some rows draw (three, the weights by many blocks)
        self.graphs: Dict[Tuple[int, bool], torch.cuda.CUDAGraph] = {}
        self.draws = False

    def _body(self) -> None:
        ops = self.engine.rt.ops
        rt = self.engine.rt
        # up to the weight-streaming products' limit of rows: their fused forms, no library call in the graph; beyond
        # it the kernels of prompt steps, the library's products among them (their plans are made by the eager run
        # that goes before every recording)
        streaming = self.cap <= rt.streaming_rows_max
        rt.no_library = streaming
        rt.fused = streaming and rt.dtype == torch.bfloat16
        try:
            logits = self.engine.model.forward(self.ctx)
        finally:
            rt.no_library = rt.fused = False
        self.logits = logits
        with rt.stage("sample"):
            if self.draws:
                ops.decode_choose(logits, self.temperature, self.u, self.counter, self.tok, self.ring, self.bad_ring,
                                  self.pos, self.kv_len, self.live, self.wide, top_p=self.top_p, wbuf=self.weights)
            else:
                ops.decode_choose_greedy(logits, self.counter, self.tok, self.ring, self.bad_ring, self.pos, self.kv_len,
                                         self.live)

    def _bound(self, longest: int) -> int:
        """The recording that serves contexts of up to ``longest`` tokens: 1024, 2048, 4096, ... tokens."""
        b = 1024
        while b < longest:
            b *= 2
        return b

    def _record(self, bound: int, draws: bool) -> None:
        """One eager run on scratch rows (everything lazily initialised gets initialised), then the capture."""
        self.ctx.max_kv_len = bound
        self.draws = draws
        # the eager run reads the rows' counters and temperatures as the last run left them (a run of MAX_STEPS steps
        # leaves the counters at MAX_STEPS, one row past the rings): both start from zero here
        self.counter.zero_()
        self.temperature.zero_()
        self.top_p.fill_(1.0)
        side = torch.cuda.Stream(device=self.engine.device)
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            self._body()
        torch.cuda.current_stream().wait_stream(side)
        self.counter.zero_()
        graph = torch.cuda.CUDAGraph()
        # no collection of cyclic garbage while the stream is capturing: a finalizer that frees pinned memory or a
        # graph of an engine long gone makes calls the capture forbids, and the process aborts
        collecting = gc.isenabled()
        gc.collect()
        gc.disable()
        try:
            with torch.cuda.graph(graph):
                self._body()
        finally:
            if collecting:
                gc.enable()
        self.graphs[(bound, draws)] = graph

    def run(self, rids: Sequence[Hashable], tokens: Sequence[int], n: int, samplers=None
            ) -> Tuple[np.ndarray, np.ndarray]:
        """``n`` steps for the requests ``rids`` whose next input tokens are ``tokens``.

        Returns ``(ids (n, batch), bad (n, batch))``.  Pages for ``n`` more tokens are reserved first;
        :class:`~gesso_amd.errors.OutOfPages` leaves everything as it was.
        """
        eng, cap, B = self.engine, self.cap, len(rids)
        if not 1 <= n <= self.MAX_STEPS:
            raise InvalidPlan(f"a decode run takes 1 to {self.MAX_STEPS} steps, not {n}")
        mgr, st = eng.manager, eng.storage
        rcs = [mgr.get(r) for r in rids]
        bound = self._bound(max(rc.length for rc in rcs) + n)
        draws = samplers is not None and any(s is not None for s in samplers)
        if (bound, draws) not in self.graphs:
            # before any live row is set: the eager run sees scratch rows only
            self.slots.fill_(st.scratch_slot)
            self.live.zero_()
            self.pos.zero_()
            self.kv_len.fill_(1)
            for g, bt in enumerate(self.block_tables):
                bt.fill_(st.num_pages[g])
            self._record(bound, draws)
        graph = self.graphs[(bound, draws)]
        for t in tokens:
            if not 0 <= int(t) < eng.spec.vocab:
                raise InvalidPlan(f"token id {int(t)} outside the vocabulary of {eng.spec.vocab}")
        mgr.reserve_many([(r, n) for r in rids])
        # from here on the cache is written: an error leaves these requests without a usable state
        try:
            ids, bad = self._run(rids, rcs, tokens, n, samplers, graph)
        except Exception as err:
            raise eng.fail_requests(rids, err) from err
        for r in rids:
            mgr.commit(r, n)
        eng.steps += n
        return ids, bad

    def _run(self, rids, rcs, tokens, n, samplers, graph):
        eng, cap, B = self.engine, self.cap, len(rids)
        st = eng.storage
        eng.prepare_cache()
        # one int32 buffer for the per-row facts, one copy
        host = np.zeros((5, cap), dtype=np.int32)
        host[0, :B] = tokens
        host[1, :B] = [rc.length for rc in rcs]
        host[2] = 1
        host[2, :B] = [rc.length + 1 for rc in rcs]
        host[3] = st.scratch_slot
        host[3, :B] = [st.scratch_slot if rc.slot is None else rc.slot for rc in rcs]
        host[4, :B] = 1
        dev = torch.from_numpy(host).pin_memory().to(eng.device, non_blocking=True)
        self.tok.copy_(dev[0]); self.pos.copy_(dev[1]); self.kv_len.copy_(dev[2])
        self.slots.copy_(dev[3]); self.live.copy_(dev[4])
        width = max(1, max(-(-(rc.length + n) // eng.page_size) for rc in rcs))
        for g, bt in enumerate(self.block_tables):
            tab = np.full((cap, width), st.num_pages[g], dtype=np.int32)
            for i, rc in enumerate(rcs):
                row = np.asarray(rc.tables[g][:width], dtype=np.int32)
                row[row < 0] = st.num_pages[g]
                tab[i, :len(row)] = row
            bt[:, :width].copy_(torch.from_numpy(tab).pin_memory().to(eng.device, non_blocking=True))
        temp = np.zeros((2, cap), dtype=np.float64)          # temperatures, then top_p (1: the whole row)
        temp[1] = 1.0
        before = {}               # row -> the sampler's state before each of its draws
        if samplers is not None and any(s is not None for s in samplers):
            u = np.zeros((n, cap), dtype=np.float64)
            for i, s in enumerate(samplers):
                if s is not None:
                    temp[0, i] = s.temperature
                    temp[1, i] = s.top_p
                    before[i] = []
                    for k in range(n):
                        before[i].append(s.state)
                        u[k, i] = s.unit()
            self.u[:n].copy_(torch.from_numpy(u).pin_memory().to(eng.device, non_blocking=True))
        tp = torch.from_numpy(temp).pin_memory().to(eng.device, non_blocking=True)
        self.temperature.copy_(tp[0]); self.top_p.copy_(tp[1])
        self.counter.zero_()
        profile = eng.rt.profile
        if profile is None:
            for _ in range(n):
                graph.replay()
        else:
            # profiled: the same step, launched kernel by kernel, with a pair of events around every stage
            self.ctx.max_kv_len = self._bound(max(rc.length for rc in rcs) + n)
            self.draws = samplers is not None and any(s is not None for s in samplers)
            profile.window = True
            try:
                for _ in range(n):
                    with profile.bracket("__step__"):
                        self._body()
            finally:
                profile.window = False
        ids = self.ring[:n, :B].cpu().numpy()
        bad = self.bad_ring[:n, :B].cpu().numpy()
        # a step whose logits were not finite emits no token and makes no draw (as the step-by-step choice does):
        # the draws were made up front, so the sampler goes back to where it stood before that step
        for i, states in before.items():
            hit = np.flatnonzero(bad[:, i])
            if hit.size:
                samplers[i].state = states[int(hit[0])]
        return ids, bad


class DecodeLoop:
    """Continue requests whose prompts are in the cache: ``run(n)`` makes ``n`` steps for all of them (greedy, or each
    row with its sampler)."""

    def __init__(self, engine, rids: Sequence[Hashable], first_tokens: Sequence[int], samplers=None):
        self.engine = engine
        self.rids = list(rids)
        self.tokens = [int(t) for t in first_tokens]
        self.samplers = samplers

    def run(self, n: int) -> List[List[int]]:
        out: List[List[int]] = []
        while n > 0:
            k = min(n, DecodeRunner.MAX_STEPS)
            ids, bad = self.engine.decode(self.rids, self.tokens, k, self.samplers)
            if bad.any():
                from ..errors import NumericalInstability
                raise NumericalInstability("non-finite logits in the decode loop")
            out += ids.tolist()
            self.tokens = ids[-1].tolist()
            n -= k
        return out

    def close(self) -> None:
        pass
