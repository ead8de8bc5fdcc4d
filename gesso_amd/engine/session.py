"""The Python entry point: ``Session`` and ``generate``, ``run_batch`` and ``cancel``.

Names and meanings follow the reference where it has them: ``Session(...; page_size=16,
context_length, eos_token_id)`` (``src/Inference/session.jl:188-199``), ``generate(s, prompt;
max_new_tokens=8, on_token)`` returning the prompt followed by the new ids (``:1025-1060``),
``prefill`` returning every position's logits (``:681-828``), the keywords of
``reference_generate`` (``sampler``, ``eos_ids``, ``stop_ids``, ``on_token``;
``src/Inference/Inference.jl:2081-2102``), ``BatchRequest``/``run_batch``/``cancel``
(``src/Runtime/Runtime.jl:33-51``, ``:98-182``), the pass size ``GESSO_PREFILL_CHUNK`` (default 1024,
``Inference.jl:1765-1773``), the timing line of ``GESSO_PROFILE=timing`` (``:2538-2544``) and the stage table of
``GESSO_PROFILE=decode`` (``src/Inference/decode_profile.jl``; also ``Engine.profile_decode``).
Unlike the reference, one session serves many requests at once.
"""
from __future__ import annotations

import os
import time
from dataclasses import dataclass
from typing import Callable, List, Optional, Sequence

import torch

from ..errors import GessoError, InvalidPlan
from ..sampling.sampler import Sampler, choose
from .batch import StepEntry
from .engine import Engine
from .scheduler import Request, Scheduler


def _env_list(name: str):
    return {v.strip() for v in os.environ.get(name, "").split(",") if v.strip()}


def default_prefill_chunk() -> int:
    raw = os.environ.get("GESSO_PREFILL_CHUNK", "").strip()
    if not raw:
        return 1024
    try:
        n = int(raw)
    except ValueError:
        raise InvalidPlan(f"GESSO_PREFILL_CHUNK must be a positive integer, got {raw!r}") from None
    if n < 1:
        raise InvalidPlan(f"GESSO_PREFILL_CHUNK must be a positive integer, got {raw!r}")
    return n


class Session:
    def __init__(self, model, *, dtype="bfloat16", device="cuda:0", page_size: int = 16,
                 context_length: Optional[int] = None, eos_token_id: Optional[int] = None,
                 max_num_seqs: int = 64, max_num_batched_tokens: Optional[int] = None,
                 chunk_size: Optional[int] = None, num_pages: Optional[int] = None,
                 max_tokens: Optional[int] = None, random_weights_seed: Optional[int] = None,
                 random_weights_std: float = 0.02, watermark: float = 0.01, kernel_options=None,
                 poison: bool = False, memory_fraction: Optional[float] = None):
        """``model``: a folder with config.json and model.safetensors, or a typed configuration
        together with ``random_weights_seed``.  ``context_length``: most tokens one request may hold.
        The cache holds ``num_pages`` pages, or ``max_tokens`` tokens, or what fits into ``memory_fraction`` of the
        device memory left free by the weights (default: four contexts).
        ``watermark``: the fraction of the pages that an admission leaves free for those who run.
        ``kernel_options``: a :class:`~gesso_amd.parts.runtime.RuntimeOptions`; ``poison``: fill what is
        given back with NaN (a debugging aid, see :class:`Engine`)."""
        self.chunk_size = chunk_size or default_prefill_chunk()
        self.max_num_seqs = max_num_seqs
        self.max_num_batched_tokens = max_num_batched_tokens or max(self.chunk_size, max_num_seqs)
        self.watermark = watermark
        kw = dict(page_size=page_size, num_slots=max_num_seqs, options=kernel_options, poison=poison)
        if isinstance(model, (str, os.PathLike)):
            from ..config.registry import load_config
            arch, cfg = load_config(os.fspath(model))
        else:
            from ..config.registry import architecture_of
            cfg = model
            if random_weights_seed is None:
                raise InvalidPlan("a configuration without a folder needs random_weights_seed")
            arch = architecture_of(cfg.to_json())
        # the longest context the model itself allows is a fact of its description, whatever its configuration calls it
        self.context_length = int(context_length or min(arch.to_spec(cfg).max_position, 4096))
        if num_pages is None and max_tokens is None and memory_fraction is None:
            max_tokens = 4 * self.context_length
        kw.update(num_pages=num_pages, max_tokens=max_tokens, max_context=self.context_length,
                  memory_fraction=memory_fraction)
        if isinstance(model, (str, os.PathLike)):
            self.engine = Engine.from_folder(os.fspath(model), dtype=dtype, device=device, **kw)
        else:
            self.engine = Engine.from_config(cfg, random_weights_seed, dtype=dtype, device=device,
                                             std=random_weights_std, **kw)
        if "decode" in _env_list("GESSO_PROFILE"):
            self.engine.profile_decode(True)
        spec = self.engine.spec
        self.eos_ids = (int(eos_token_id),) if eos_token_id is not None else tuple(spec.eos_token_ids)
        self.last_stats = {}
        self.last_results = []
        self._next_id = 0
        self._closed = False

    # ------------------------------------------------------------------ low level

    def step(self, entries: Sequence[StepEntry]):
        return self.engine.step(entries)

    def prefill(self, prompt: Sequence[int]) -> torch.Tensor:
        """Float32 logits ``(len(prompt), vocab)`` of every position of one prompt; nothing is kept."""
        rid = ("prefill", self._next_id)
        self._next_id += 1
        self.engine.add_request(rid)
        try:
            return self.engine.step([StepEntry(rid, list(prompt), list(range(len(prompt))))])
        finally:
            self.engine.finish_request(rid)

    # ------------------------------------------------------------------ generation

    def _choose(self, logits, samplers):
        return choose(self.engine.rt.ops, logits, samplers)

    def scheduler(self) -> Scheduler:
        return Scheduler(self.engine, self._choose, self.max_num_seqs, self.max_num_batched_tokens, self.chunk_size,
                         watermark=self.watermark)

    def generate(self, prompts, max_new_tokens: int = 8, sampler=None, temperature: float = 0.0, top_p: float = 1.0,
                 seed: int = 0, eos_ids=None, stop_ids=(), on_token: Optional[Callable] = None):
        """Prompt(s) followed by up to ``max_new_tokens`` new ids.

        ``prompts``: one list of ids (one list comes back) or a list of such lists.  Greedy unless a
        ``sampler`` (one :class:`Sampler`, or one per prompt) or ``temperature > 0`` is given; with one
        sampler and several prompts, prompt ``i`` draws from seed ``seed + i``.  ``on_token(id)`` (one
        prompt) or ``on_token(i, id)`` (several) may return False to stop that request.

        A request that fails (non-finite logits, a prompt that fits no cache) stops alone; the others run to
        their end, ``last_results`` holds every request's :class:`BatchResult`, and then the first failure is
        raised, with ``detail["results"]`` = ``last_results``.
        """
        if self._closed:
            raise InvalidPlan("the session is closed")
        single = len(prompts) > 0 and not isinstance(prompts[0], (list, tuple))
        plist = [list(prompts)] if single else [list(p) for p in prompts]
        for p in plist:
            if len(p) + max_new_tokens > self.context_length:
                raise InvalidPlan(f"prompt of {len(p)} tokens plus {max_new_tokens} new ones exceed the context of "
                                  f"{self.context_length}", context_length=self.context_length)
        if sampler is None and temperature > 0:
            sampler = Sampler(temperature, top_p, seed)
        if isinstance(sampler, Sampler):
            base = sampler
            samplers = [base if single else Sampler(base.temperature, base.top_p, (base.state + i) % (1 << 64))
                        for i in range(len(plist))]
        elif sampler is None:
            samplers = [None] * len(plist)
        else:
            samplers = list(sampler)
            if len(samplers) != len(plist):
                raise InvalidPlan("one sampler per prompt")
        eos = self.eos_ids if eos_ids is None else tuple(int(t) for t in eos_ids)
        sched = self.scheduler()
        requests = []
        for i, (p, s) in enumerate(zip(plist, samplers)):
            cb = None
            if on_token is not None:
                cb = on_token if single else (lambda tok, i=i: on_token(i, tok))
            r = Request(("gen", self._next_id), p, max_new_tokens, s, eos, tuple(int(t) for t in stop_ids), cb)
            self._next_id += 1
            requests.append(sched.add(r))
        self._run(sched, requests)
        self.last_results = [BatchResult(r.tokens, r.finish_reason, r.error) for r in requests]
        for r in requests:
            if r.finish_reason == "failed":
                err = r.error
                if isinstance(err, GessoError):
                    err.detail.setdefault("results", self.last_results)
                raise err
        out = [r.tokens for r in requests]
        return out[0] if single else out

    def _run(self, sched: Scheduler, requests: List[Request]) -> None:
        dev = self.engine.device
        t0 = time.perf_counter()
        first = None
        try:
            while sched.has_work():
                out = sched.step()
                if out and first is None:
                    torch.cuda.synchronize(dev)
                    first = time.perf_counter()
                if out is None and sched.has_work():
                    raise InvalidPlan("the scheduler found nothing to run though requests are left")
        finally:
            for r in list(sched.running):       # an error above: give back what is still held
                if sched.executor.has_request(r.rid):
                    sched.executor.finish_request(r.rid)
        torch.cuda.synchronize(dev)
        t1 = time.perf_counter()
        first = first or t1
        st = dict(sched.stats)
        st.update(prefill_ms=(first - t0) * 1e3, decode_ms=(t1 - first) * 1e3,
                  new_tokens=sum(len(r.output) for r in requests), cache=self.engine.manager.stats())
        if self.engine.recorder is not None:
            st["replayed_steps"] = self.engine.recorder.replays       # since the session began
        profile = self.engine.rt.profile
        if profile is not None:
            st["decode_profile"] = profile.report()
            for line in profile.lines():
                print(line, flush=True)
            self.engine.profile_decode(True)              # a fresh one for the next call
        self.last_stats = st
        if "timing" in _env_list("GESSO_PROFILE"):
            print(f"gesso_timing prefill_ms={st['prefill_ms']:.3f} decode_ms={st['decode_ms']:.3f} "
                  f"tokens={st['new_tokens']} steps={st['steps']} preemptions={st['preemptions']}", flush=True)

    def close(self) -> None:
        self._closed = True
        self.engine = None


def generate(session: Session, prompt, **kw):
    """``generate(session, prompt; max_new_tokens=8, ...)``: the reference's spelling of :meth:`Session.generate`."""
    return session.generate(prompt, **kw)


# ---------------------------------------------------------------------- batches of requests

@dataclass
class BatchRequest:
    session: Session
    prompt: List[int]
    max_new_tokens: int = 8
    sampler: Optional[Sampler] = None
    cancelled: bool = False
    _request: Optional[Request] = None

    def __post_init__(self):
        if self.max_new_tokens < 0:
            raise InvalidPlan("BatchRequest: token budget must be nonnegative")
        self.prompt = [int(t) for t in self.prompt]


@dataclass
class BatchResult:
    ids: List[int]
    status: str                      # eos | complete | cancelled | failed
    error: Optional[Exception] = None


def cancel(request: BatchRequest) -> BatchRequest:
    request.cancelled = True
    if request._request is not None:
        request._request.cancelled = True
    return request


def run_batch(requests: Sequence[BatchRequest], on_token: Optional[Callable[[int, int], Optional[bool]]] = None
              ) -> List[BatchResult]:
    """Run requests of one session together; each ends on its own (a failure stops only itself)."""
    if not requests:
        return []
    session = requests[0].session
    if any(r.session is not session for r in requests):
        raise InvalidPlan("run_batch: all requests must belong to one session")
    if len({id(r) for r in requests}) != len(requests):
        raise InvalidPlan("run_batch: a request occurs twice")
    sched = session.scheduler()
    inner = []
    for i, br in enumerate(requests):
        cb = (lambda tok, i=i: on_token(i, tok)) if on_token is not None else None
        r = Request(("batch", session._next_id), br.prompt, br.max_new_tokens, br.sampler, session.eos_ids, (), cb)
        session._next_id += 1
        r.cancelled = br.cancelled
        br._request = r
        inner.append(sched.add(r))
    session._run(sched, inner)
    return [BatchResult(r.tokens, r.finish_reason, r.error) for r in inner]
