"""The engine: a model, its cache, and the one step function.

``step(entries)`` runs exactly the tokens it is given, as one batch, from the cache that earlier
steps left, and returns float32 logits at the wanted places, in the order of the entries and of
their ``want`` lists.  Portions of prompts may stand beside single decoded tokens, cut anywhere.
The reference runs one sequence per pass (a prefill pass of n rows, ``src/Inference/Inference.jl:2272-2530``,
or one decode row, ``:3270-3383``); a mixed batch over several requests has no counterpart there.

What happens when a pool is exhausted: ``step`` raises :class:`~gesso_amd.errors.OutOfPages`
before it has changed anything; the scheduler decides what to do then.
"""
from __future__ import annotations

from typing import Hashable, Optional, Sequence

import torch

from ..cache.manager import CacheLayout, CacheManager
from ..cache.storage import CacheStorage
from ..config.registry import load_config
from ..config.spec import ModelSpec
from ..errors import InvalidPlan, StepFailed
from ..models.model import Model, tensor_table, tied_aliases
from ..parts.runtime import Runtime, RuntimeOptions
from ..weights.loader import load_tensors, random_tensors
from .batch import StepContext, StepEntry, check_entries

_DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "fp32": torch.float32,
           torch.bfloat16: torch.bfloat16, torch.float32: torch.float32}


def parse_dtype(dtype) -> torch.dtype:
    try:
        return _DTYPES[dtype]
    except KeyError:
        raise InvalidPlan(f"dtype must be bfloat16 or float32, got {dtype!r}") from None


class Engine:
    def __init__(self, spec: ModelSpec, tensors, dtype, device="cuda:0", page_size: int = 16,
                 num_pages: Optional[int] = None, max_tokens: Optional[int] = None, num_slots: int = 8,
                 max_context: Optional[int] = None, options: Optional[RuntimeOptions] = None, poison: bool = False,
                 memory_fraction: Optional[float] = None):
        """``tensors``: ``file name -> tensor`` on the device, in the widths the loader chose.

        The page pool holds ``num_pages`` pages per group, or enough for ``max_tokens`` tokens, or as many as fit into
        ``memory_fraction`` of the device memory that is free once the weights are bound.
        ``options``: how kernels are chosen (:class:`~gesso_amd.parts.runtime.RuntimeOptions`).
        ``poison``: a debugging aid: every page and slot that is given back is filled with NaN before the next
        step runs, so that a kernel that reads a row it has no business with shows in the logits.
        """
        self.spec = spec
        self.dtype = parse_dtype(dtype)
        self.device = torch.device(device)
        self.rt = Runtime(self.device, self.dtype, options)
        self.model = Model(spec, self.rt)
        self.model.bind(tensors)
        self.page_size = int(page_size)
        self.max_context = min(spec.max_position, max_context or spec.max_position)
        needs = self.model.cache_needs()
        layout = CacheLayout.plan(needs, [c.cache for c in spec.schedule])
        if num_pages is None:
            if max_tokens is not None:
                num_pages = -(-int(max_tokens) // self.page_size)
            elif memory_fraction is not None:
                num_pages = self._pages_that_fit(layout, float(memory_fraction))
            else:
                raise InvalidPlan("give the cache a size: num_pages, max_tokens or memory_fraction")
        self.manager = CacheManager(layout, self.page_size, int(num_pages), int(num_slots), self.max_context)
        self.storage = CacheStorage(layout, self.page_size, int(num_pages), int(num_slots), self.dtype, self.device)
        self.poison = bool(poison)
        self.manager.track_released = self.poison
        if self.poison:
            self.storage.poison_all()
        self.steps = 0
        self._runners = {}
        # steps of prompt portions whose kind recurs are recorded and replayed, where the options ask for it and every
        # part can be (bfloat16: the 32-bit path has no such parts' kernels)
        self.recorder = None
        if self.rt.options.record_portions and self.dtype == torch.bfloat16 and self.model.portions_recordable:
            from .planned import StepRecorder
            self.recorder = StepRecorder(self)
        # the most requests one recorded decode step takes: as many rows as the runtime's weight-streaming products do
        # (the limit is the product kernels', asked of the runtime, not a number of the engine's own)
        self.DECODE_MAX_BATCH = self.rt.streaming_rows_max
        # More requests than that decode through a recording of the same loop in which the many-row products (the
        # vendor's, each weight read once for all rows) and the kernels of prompt steps stand for the fused
        # weight-streaming ones: up to this many at once (bfloat16; 0: no such loop).
        self.DECODE_WIDE_MAX = 512 if self.dtype == torch.bfloat16 else 0

    def _pages_that_fit(self, layout: CacheLayout, fraction: float) -> int:
        """Pages per group that ``fraction`` of the free device memory holds (every group gets as many)."""
        if not 0.0 < fraction <= 1.0:
            raise InvalidPlan(f"memory_fraction is a share of the free device memory in (0, 1], not {fraction}")
        width = torch.empty((), dtype=self.dtype).element_size()
        per_page = sum(len(g.members) * g.need.n_kv_heads * self.page_size * (g.need.head_dim + g.need.value_width) * width
                       for g in layout.paged)
        if per_page == 0:
            return 1                               # no paged layers: a page is bookkeeping only
        free, _ = torch.cuda.mem_get_info(self.device)
        pages = int(free * fraction) // per_page - 1            # (one more page per group is scratch)
        if pages < 1:
            raise InvalidPlan(f"{fraction} of the {free} free bytes hold no page of {per_page} bytes")
        # what the kernels' 32-bit offsets into one layer's pages reach (units of 16 bytes)
        reach = min((1 << 32) // max(1, g.need.n_kv_heads * self.page_size * max(1, max(g.need.head_dim, g.need.value_width) * width // 16))
                    for g in layout.paged)
        return min(pages, reach - 2)

    # ------------------------------------------------------------------ construction

    @classmethod
    def from_folder(cls, model_dir: str, dtype="bfloat16", device="cuda:0", **kw) -> "Engine":
        arch, cfg = load_config(model_dir)
        spec = arch.to_spec(cfg)
        mode = parse_dtype(dtype)
        tensors = load_tensors(model_dir, tensor_table(spec), mode, device, aliases=tied_aliases(spec),
                               ignored_suffixes=spec.ignored_tensors)
        return cls(spec, tensors, mode, device, **kw)

    @classmethod
    def from_config(cls, config, seed: int, dtype="bfloat16", device="cuda:0", std: float = 0.02, **kw) -> "Engine":
        """Random weights drawn on the device (for measurements; a folder is written by ``write_model_folder``)."""
        from ..config.registry import architecture_of
        from ..weights.loader import held_dtype

        spec = architecture_of(config.to_json()).to_spec(config)
        mode = parse_dtype(dtype)
        table = tensor_table(spec)
        drawn = random_tensors(table, seed, torch.float32 if mode == torch.float32 else torch.bfloat16, device, std)
        tensors = {name: t.to(held_dtype(t.dtype, table[name].role, mode)) for name, t in drawn.items()}
        return cls(spec, tensors, mode, device, **kw)

    # ------------------------------------------------------------------ requests

    def add_request(self, rid: Hashable) -> None:
        self.manager.admit(rid)

    def finish_request(self, rid: Hashable) -> None:
        self.manager.release(rid)

    def has_request(self, rid: Hashable) -> bool:
        return rid in self.manager.requests

    def length(self, rid: Hashable) -> int:
        return self.manager.get(rid).length

    # ------------------------------------------------------------------ the step

    def prepare_cache(self) -> None:
        """Before a step's kernels run: with poisoning on, NaN into what was given back since the last step; then the
        initial value into every slot handed out since."""
        ops = self.rt.ops
        if self.poison:
            pages, slots = self.manager.take_released()
            for g, ids in enumerate(pages):
                if ids:
                    self.storage.fill_pages(ops, g, ids, float("nan"))
            if slots:
                self.storage.fill_slots(ops, slots, None)
        fresh = self.manager.fresh_slots
        if fresh:
            self.storage.fill_slots(ops, fresh, "initial")
            fresh.clear()

    def fail_requests(self, rids, err: Exception) -> StepFailed:
        """A step broke off in the middle: the state of its requests (pages partly written, histories partly
        advanced) is worth nothing, so they are released; the reference invalidates the state of a generation that
        fails (``src/Inference/Inference.jl:2730-2736``)."""
        gone = []
        for rid in rids:
            if rid in self.manager.requests:
                self.manager.release(rid)
                gone.append(rid)
        return StepFailed(f"a step failed and its requests were released: {err}", requests=gone)

    def step(self, entries: Sequence[StepEntry]) -> Optional[torch.Tensor]:
        entries = [e if isinstance(e, StepEntry) else StepEntry(*e) for e in entries]
        if not entries:
            return None
        ids = check_entries(entries, self.manager, self.spec.vocab)
        self.manager.reserve_many([(e.rid, len(e.tokens)) for e in entries])
        # from here on the cache is written: an error leaves the requests of this step without a usable state
        try:
            self.prepare_cache()
            logits = self._step_recorded(entries, ids) if self.recorder is not None else False
            if logits is False:
                ctx = StepContext(entries, self.manager, self.storage, self.spec.vocab, self.device, token_ids=ids)
                logits = self.model.forward(ctx)
        except Exception as err:
            raise self.fail_requests([e.rid for e in entries], err) from err
        for e in entries:
            self.manager.commit(e.rid, len(e.tokens))
        self.steps += 1
        return logits

    def _step_recorded(self, entries, ids):
        """The step through a recording of its kind (:mod:`gesso_amd.engine.planned`), or False where there is none."""
        rec = self.recorder.recording_for(entries)
        if rec is None:
            return False
        n_want = rec.fill(entries, ids)
        if n_want is None:
            return False
        self.recorder.replays += 1
        return rec.launch(n_want)

    # ------------------------------------------------------------------ profiling

    def profile_decode(self, on: bool = True):
        """Switch the decode stage profiler on (returns it) or off.  While it is on, decode runs launch their step
        kernel by kernel with HIP events around every stage (:mod:`gesso_amd.engine.profile`)."""
        from .profile import StageProfile
        self.rt.profile = StageProfile() if on else None
        return self.rt.profile

    # ------------------------------------------------------------------ decoding, recorded


    def decode(self, rids: Sequence[Hashable], tokens: Sequence[int], n: int, samplers=None):
        """``n`` decode steps for requests that each bring one token, as replays of a recorded graph.

        ``tokens``: each request's next input token; the tokens chosen are fed back on the device.
        ``samplers``: per request None (greedy) or a :class:`~gesso_amd.sampling.sampler.Sampler`
        (temperature, with or without a nucleus).  Returns ``(ids, bad)`` as ``(n, batch)`` arrays; a row of
        ``bad`` marks a step whose logits were not finite.  Raises :class:`~gesso_amd.errors.OutOfPages` before changing anything.
        """
        from .decode import DecodeRunner, _capacity
        most = max(self.DECODE_MAX_BATCH, self.DECODE_WIDE_MAX)
        if not 1 <= len(rids) <= most:
            raise InvalidPlan(f"the recorded decode loop takes 1 to {most} requests, not {len(rids)}")
        if len(set(rids)) != len(rids) or len(tokens) != len(rids):
            raise InvalidPlan("one token per request, each request once")
        if not self.model.graph_safe:
            return self._decode_eager(rids, tokens, n, samplers)
        cap = _capacity(len(rids))
        runner = self._runners.get(cap)
        if runner is None:
            runner = self._runners[cap] = DecodeRunner(self, cap)
        return runner.run(rids, tokens, n, samplers)

    def choice_scratch(self, rows: int):
        """What the recorded loop's choice needs when rows draw: float64 room for the weights of ``rows`` rows of logits
        (draws from a nucleus) and for their partial sums, and the rows' maxima and flags; one set per engine, shared by
        the loops of all capacities and made anew when a loop of more rows asks (the loops recorded before keep theirs).
        Returns ``(weights, (part, amax, bad0, hist))``."""
        held = getattr(self, "_choice_scratch", None)
        if held is None or held[0] < rows:
            n, dev = rows, self.device
            self._choice_scratch = (rows, (
                torch.empty(n * self.spec.vocab, dtype=torch.float64, device=dev),
                (torch.empty(n * self.rt.ops.choice_parts(self.spec.vocab), dtype=torch.float64, device=dev),
                 torch.zeros(n, dtype=torch.int32, device=dev), torch.zeros(n, dtype=torch.int32, device=dev),
                 torch.zeros(n * self.rt.ops.choice_hist(), dtype=torch.int64, device=dev))))
        return self._choice_scratch[1]

    def _decode_eager(self, rids, tokens, n, samplers):
        """The same steps one by one through :meth:`step`, for models with parts that cannot be recorded."""
        import numpy as np
        from ..sampling.sampler import choose
        samplers = list(samplers) if samplers is not None else [None] * len(rids)
        self.manager.reserve_many([(r, n) for r in rids])
        ids = np.zeros((n, len(rids)), dtype=np.int32)
        bad = np.zeros((n, len(rids)), dtype=np.int32)
        tokens = [int(t) for t in tokens]
        for s in range(n):
            logits = self.step([StepEntry(r, [t], [0]) for r, t in zip(rids, tokens)])
            picks = choose(self.rt.ops, logits, samplers)
            for i, p in enumerate(picks):
                if isinstance(p, Exception):
                    bad[s, i] = 1
                else:
                    ids[s, i] = tokens[i] = p
        return ids, bad
