"""The scheduler: which requests run in the next step, with which tokens.

It admits requests in arrival order, cuts prompts into portions under a token budget, lets every
request whose prompt is consumed decode one token per step, finishes requests and frees what
they hold at once.  The reference has no counterpart above one sequence: its ``run_batch``
prefills each request whole and then decodes them round-robin (``src/Runtime/Runtime.jl:98-182``),
with passes bounded by ``GESSO_PREFILL_CHUNK`` (``src/Inference/Inference.jl:1765-1773``); the
statuses a request ends with are the reference's (``Runtime.jl:167-178``): ``eos``, ``complete``,
``cancelled``, ``failed``.

Decisions, all tested without a GPU:

* Order within a step: decoding requests first (one token each), then portions of prompts,
  oldest request first, each at most ``chunk_size`` and together at most the step's budget of
  ``max_num_batched_tokens``.
* Admission: while fewer than ``max_num_seqs`` requests run, a slot is free and pages for the
  first portion are free, with ``watermark`` (a fraction of each pool, rounded up to whole pages) left
  over for the requests that already run; into an idle engine a request is admitted without that margin.
* Context: a request whose known tokens no longer fit into the context (``manager.max_length``) ends as
  ``failed`` with :class:`~gesso_amd.errors.ResourceLimit` and keeps the tokens it has; nothing else stops
  (the reference's ``ERR_RESOURCE_LIMIT``, ``src/Inference/kv_manager.jl:246-257``).
* Out of pages: the request admitted last is preempted: everything it holds is given back, and
  it returns to the front of the waiting line to be computed again from its prompt and the
  tokens it has generated (its sampler state is kept, so a sampled request draws on where it
  stopped).  This repeats until the step fits.  A request that does not fit into the empty pool
  on its own ends as ``failed`` with :class:`~gesso_amd.errors.ResourceLimit`; nothing else stops.
* The token that ends a request (an id in ``eos_ids``/``stop_ids``) is returned and never fed.
* When a step holds nothing but decoding requests and the executor has a recorded decode loop
  (``decode``), several steps run back to back on the device: as many as every request still has
  tokens to generate, at most ``decode_run_steps``, and one only while requests wait for admission
  (more requests than the loop takes at once go through it in groups, one group after the other).
  Tokens come back together; a request that ends within the run (end token, callback) keeps its
  tokens up to there, what the device computed beyond is dropped with the request's cache.
* A pass that breaks off in the middle (the executor raises :class:`~gesso_amd.errors.StepFailed` and has
  released the requests of that pass) ends those requests as ``failed`` with the tokens they had; every other
  request goes on, a group of a decode run that ran before the failing group keeps its tokens
  (the reference stops only the request whose pass failed, ``src/Runtime/Runtime.jl:175-178``).
"""
from __future__ import annotations

import math
from collections import deque
from dataclasses import dataclass, field
from typing import Callable, Deque, Hashable, List, Optional, Sequence, Tuple

from ..errors import GessoError, InvalidPlan, NumericalInstability, OutOfPages, OutOfSlots, ResourceLimit, StepFailed
from ..sampling.sampler import Sampler
from .batch import StepEntry

WAITING, RUNNING, FINISHED = "waiting", "running", "finished"


@dataclass(eq=False)                                 # a request is itself: compared and hashed by identity
class Request:
    rid: Hashable
    prompt: List[int]
    max_new_tokens: int = 8
    sampler: Optional[Sampler] = None               # None = greedy
    eos_ids: Tuple[int, ...] = ()
    stop_ids: Tuple[int, ...] = ()
    on_token: Optional[Callable[[int], Optional[bool]]] = None
    # ---- state
    output: List[int] = field(default_factory=list)
    computed: int = 0                                # tokens whose state is in the cache
    status: str = WAITING
    finish_reason: Optional[str] = None              # eos | complete | cancelled | failed
    error: Optional[Exception] = None
    cancelled: bool = False
    preemptions: int = 0

    def __post_init__(self):
        self.prompt = [int(t) for t in self.prompt]
        if not self.prompt:
            raise InvalidPlan("a request needs a prompt of at least one token")
        if self.max_new_tokens < 0:
            raise InvalidPlan("the token budget must be nonnegative")

    @property
    def tokens(self) -> List[int]:
        return self.prompt + self.output

    @property
    def last_token(self) -> int:
        return self.output[-1] if self.output else self.prompt[-1]

    def span(self, start: int, count: int) -> List[int]:
        """``tokens[start:start + count]`` without building the whole list."""
        n = len(self.prompt)
        if start + count <= n:
            return self.prompt[start:start + count]
        if start >= n:
            return self.output[start - n:start - n + count]
        return self.prompt[start:] + self.output[:start + count - n]

    @property
    def pending(self) -> int:
        """Tokens known and not yet in the cache."""
        return len(self.prompt) + len(self.output) - self.computed


@dataclass
class Scheduled:
    request: Request
    start: int          # first token (index into request.tokens) fed in this step
    count: int
    samples: bool       # the portion reaches the last known token: its logits choose the next


class Scheduler:
    def __init__(self, executor, choose: Callable, max_num_seqs: int = 64, max_num_batched_tokens: int = 2048,
                 chunk_size: int = 1024, decode_run_steps: int = 16, watermark: float = 0.01):
        """``executor``: ``add_request``, ``finish_request``, ``step(entries) -> logits`` and ``manager``.

        ``choose(logits, samplers) -> ids or exceptions``, one per row.
        """
        if max_num_seqs < 1 or max_num_batched_tokens < 1 or chunk_size < 1:
            raise InvalidPlan("max_num_seqs, max_num_batched_tokens and chunk_size must be positive")
        if not 0 <= watermark < 1:
            raise InvalidPlan(f"the admission watermark is a fraction of the pool in [0, 1), not {watermark}")
        self.executor = executor
        self.manager = executor.manager
        self.choose = choose
        self.max_num_seqs = max_num_seqs
        self.max_num_batched_tokens = max_num_batched_tokens
        self.chunk_size = chunk_size
        self.decode_run_steps = max(1, decode_run_steps)
        # pages per pool that an admission leaves free for the requests already running
        self.keep_free = [int(math.ceil(watermark * p.total)) for p in self.manager.pools]
        self.waiting: Deque[Request] = deque()
        self.running: List[Request] = []          # in admission order
        self.finished: List[Request] = []
        self.stats = {"steps": 0, "preemptions": 0, "prompt_tokens": 0, "decode_tokens": 0, "failed_passes": 0}

    # ------------------------------------------------------------------ requests

    def add(self, request: Request) -> Request:
        vocab = getattr(getattr(self.executor, "spec", None), "vocab", None)
        if vocab is not None:
            bad = next((t for t in request.prompt if not 0 <= t < vocab), None)
            if bad is not None:              # refused here, alone, before it could stop a step that others share
                err = InvalidPlan(f"token id {bad} outside the vocabulary of {vocab}", token=bad, vocab=vocab)
                self._finish(request, "failed", live=False, error=err)
                return request
        if request.max_new_tokens == 0:
            self._finish(request, "complete", live=False)
            return request
        self.waiting.append(request)
        return request

    def has_work(self) -> bool:
        return bool(self.waiting or self.running)

    def _finish(self, r: Request, reason: str, live: bool = True, error: Exception = None) -> None:
        if live:
            self.executor.finish_request(r.rid)
            self.running.remove(r)
        r.status, r.finish_reason, r.error = FINISHED, reason, error
        self.finished.append(r)

    def _fail_pass(self, reqs: Sequence[Request], err: StepFailed) -> None:
        """The requests of a pass that broke off end as ``failed``.  The executor has released those it names in
        ``err.detail["requests"]``; one it still holds is released here, its cache being of no use either."""
        gone = set(err.detail.get("requests", ()))
        holds = getattr(self.executor, "has_request", None)
        for r in reqs:
            if r.status != RUNNING:
                continue
            held = r.rid not in gone and (holds is None or holds(r.rid))
            if not held:
                self.running.remove(r)
            self._finish(r, "failed", live=held, error=err)
        self.stats["failed_passes"] += 1

    def _preempt(self, r: Request) -> None:
        self.executor.finish_request(r.rid)
        self.running.remove(r)
        r.status, r.computed = WAITING, 0
        r.preemptions += 1
        self.stats["preemptions"] += 1
        self.waiting.appendleft(r)

    # ------------------------------------------------------------------ one step's plan

    def _portion(self, r: Request, budget: int) -> int:
        return min(r.pending, self.chunk_size, budget)

    def _pages_short(self, plan: List[Scheduled], keep: Sequence[int] = ()) -> bool:
        """Whether the pools cannot take the plan and still have ``keep[g]`` pages left."""
        need = [0] * len(self.manager.pools)
        for s in plan:
            for g, n in enumerate(self.manager.pages_needed(s.request.rid, s.count)):
                need[g] += n
        keep = list(keep) or [0] * len(need)
        return any(n + k > pool.n_free for n, k, pool in zip(need, keep, self.manager.pools))

    def _outgrown(self, r: Request) -> Optional[ResourceLimit]:
        """The error of a request whose known tokens do not fit into the context any more, else None."""
        held = r.computed + r.pending
        if held <= self.manager.max_length:
            return None
        return ResourceLimit(f"request {r.rid!r} would hold {held} tokens, the context holds {self.manager.max_length}",
                             length=held, max_length=self.manager.max_length)

    def schedule(self) -> List[Scheduled]:
        """Decide the next step.  Admits, and preempts if pages run out; returns the plan (may be empty)."""
        # requests cancelled from outside leave first
        for r in [r for r in self.running if r.cancelled]:
            self._finish(r, "cancelled")
        for r in [r for r in self.waiting if r.cancelled]:
            self.waiting.remove(r)
            self._finish(r, "cancelled", live=False)
        # and so do requests that have outgrown the context: each fails alone
        for r in list(self.running):
            err = self._outgrown(r)
            if err is not None:
                self._finish(r, "failed", error=err)

        while True:
            budget = self.max_num_batched_tokens
            plan: List[Scheduled] = []
            decoding, prefilling = [], []
            for r in self.running:
                (decoding if r.pending == 1 and r.computed >= len(r.prompt) else prefilling).append(r)
            for r in decoding:
                if budget < 1:
                    break
                plan.append(Scheduled(r, r.computed, 1, True))
                budget -= 1
            for r in prefilling:
                n = self._portion(r, budget)
                if n < 1:
                    continue
                plan.append(Scheduled(r, r.computed, n, n == r.pending))
                budget -= n
            if self._pages_short(plan):
                victim = self.running[-1]
                if len(self.running) == 1:
                    # alone in the pool and still too large: nothing can be given back for it
                    err = ResourceLimit(f"request {victim.rid!r} does not fit into the cache on its own",
                                        tokens=victim.computed + victim.pending)
                    self._finish(victim, "failed", error=err)
                else:
                    self._preempt(victim)
                continue
            # admission, oldest first, while the step has room
            while self.waiting and len(self.running) < self.max_num_seqs and budget > 0:
                r = self.waiting[0]
                err = self._outgrown(r)
                if err is not None:
                    self.waiting.popleft()
                    self._finish(r, "failed", live=False, error=err)
                    continue
                n = self._portion(r, budget)
                if n < 1:
                    break
                if self.manager.needs_slot and self.manager.slot_pool.n_free < 1:
                    break
                try:
                    self.executor.add_request(r.rid)
                except OutOfSlots:
                    break
                trial = plan + [Scheduled(r, 0, n, n == r.pending)]
                if self._pages_short(trial, self.keep_free if self.running else ()):
                    self.executor.finish_request(r.rid)
                    if not self.running:
                        # the pool is empty and the first portion still does not fit: try a smaller one
                        fit = self._largest_fit(r, n)
                        if fit < 1:
                            self.waiting.popleft()
                            err = ResourceLimit(f"request {r.rid!r} does not fit into the cache on its own",
                                                tokens=r.pending)
                            self._finish(r, "failed", live=False, error=err)
                            continue
                        self.executor.add_request(r.rid)
                        n = fit
                        trial = plan + [Scheduled(r, 0, n, n == r.pending)]
                    else:
                        break
                self.waiting.popleft()
                r.status = RUNNING
                self.running.append(r)
                plan = trial
                budget -= n
            return plan

    def _largest_fit(self, r: Request, n: int) -> int:
        """Largest first portion of a request that the empty pool can hold."""
        ps = self.manager.page_size
        free = min((p.n_free for p in self.manager.pools), default=1 << 40)
        return min(n, free * ps)

    # ------------------------------------------------------------------ run

    def step(self) -> Optional[List[Tuple[Request, int]]]:
        """Plan, run and account one step; returns the (request, token) pairs it emitted, None if nothing ran."""
        plan = self.schedule()
        if not plan:
            return None
        run = self._decode_run(plan)
        if run is not None:
            return run
        entries = []
        for s in plan:
            toks = s.request.span(s.start, s.count)
            entries.append(StepEntry(s.request.rid, toks, [s.count - 1] if s.samples else []))
        try:
            logits = self.executor.step(entries)
        except OutOfPages:
            raise AssertionError("the plan was checked against the pools and still ran out of pages")
        except StepFailed as err:
            self._fail_pass([s.request for s in plan], err)
            return []
        self.stats["steps"] += 1
        emitted: List[Tuple[Request, int]] = []
        sampling = [s for s in plan if s.samples]
        for s in plan:
            r = s.request
            r.computed += s.count
            if s.start < len(r.prompt):
                self.stats["prompt_tokens"] += min(s.count, len(r.prompt) - s.start)
        if sampling:
            picks = self.choose(logits, [s.request.sampler for s in sampling])
            for s, tok in zip(sampling, picks):
                r = s.request
                if isinstance(tok, Exception):
                    self._finish(r, "failed", error=tok)
                    continue
                self._emit(r, int(tok), emitted)
        return emitted

    def _decode_run(self, plan: List[Scheduled]) -> Optional[List[Tuple[Request, int]]]:
        """Several decode steps at once through the executor's recorded loop, when the plan allows it."""
        ex = self.executor
        most = getattr(ex, "DECODE_MAX_BATCH", 0)
        if not hasattr(ex, "decode") or most < 1:
            return None
        if not all(s.count == 1 and s.samples for s in plan):
            return None
        reqs = [s.request for s in plan]
        if len(reqs) > most:
            most = max(most, getattr(ex, "DECODE_WIDE_MAX", 0))     # the loop for many rows, where the executor has one
        n = min(self.decode_run_steps, min(r.max_new_tokens - len(r.output) for r in reqs))
        if self.waiting:
            n = 1                     # someone waits: look at admission again after every step
        n = min(n, min(self.manager.max_length - r.computed for r in reqs))    # schedule() left each room for one
        while n > 1 and self._pages_short([Scheduled(r, r.computed, n, True) for r in reqs]):
            n -= 1
        # more requests than the recorded loop takes at once go through it in groups, one after the other (the pages
        # of all of them were counted above, so no group finds the pool short)
        emitted: List[Tuple[Request, int]] = []
        self.stats["steps"] += n
        for a in range(0, len(reqs), most):
            group = reqs[a:a + most]
            try:
                ids, bad = ex.decode([r.rid for r in group], [r.last_token for r in group], n,
                                     [r.sampler for r in group])
            except StepFailed as err:
                self._fail_pass(group, err)      # this group's requests end here; the other groups are untouched
                continue
            for i, r in enumerate(group):
                if r.computed < len(r.prompt):
                    self.stats["prompt_tokens"] += 1      # a prompt of one token decodes from its first step
                r.computed += n
                for s in range(n):
                    if bad[s][i]:
                        self._finish(r, "failed", error=NumericalInstability("non-finite logits: no token is emitted"))
                        break
                    if self._emit(r, int(ids[s][i]), emitted):
                        break
        return emitted

    def _emit(self, r: Request, tok: int, emitted: List[Tuple[Request, int]]) -> bool:
        """Account one new token of a request; True when the request has ended with it."""
        r.output.append(tok)
        self.stats["decode_tokens"] += 1
        emitted.append((r, tok))
        keep = True
        if r.on_token is not None:
            try:
                keep = r.on_token(tok) is not False
            except Exception as err:    # a failing callback ends its own request only
                self._finish(r, "failed", error=err)
                return True
        if tok in r.eos_ids or tok in r.stop_ids:
            self._finish(r, "eos")
        elif len(r.output) >= r.max_new_tokens:
            self._finish(r, "complete")
        elif not keep or r.cancelled:
            self._finish(r, "cancelled")
        else:
            return False
        return True

    def run(self) -> None:
        while self.has_work():
            if self.step() is None and self.has_work():
                raise GessoError("the scheduler found nothing to run though requests are left",
                                 waiting=len(self.waiting), running=len(self.running))
