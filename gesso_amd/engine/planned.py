"""Steps of prompt portions, recorded once and replayed: the launches of such a step off the host.

A step that mixes prompt portions with decoded tokens is some 160 kernel launches, and on small models the host
needs longer to enqueue them than the device to run them.  A scheduler that fills its token budget makes step
after step with the same number of tokens; what changes is how the tokens divide into sequences.  Nearly every
launch of such a step depends on the token count alone and reads the rest (token ids, positions, sequence
starts, slots, block tables, the attention kernel's tile lists) from device memory.  So the step is recorded
once per token count as a chain of HIP graphs over buffers that every replay refills with one copy; between the
graphs stand the few calls that do depend on the step (attention over the decoded tokens at the batch's head,
whose number changes), made anew at every replay.  The final norm and the head, which take however many rows
are wanted, follow as ordinary launches.  The reference has no counterpart: it runs one sequence per pass
(``src/Inference/Inference.jl:2272-2530``).

A step of many sequences that bring one token each (more than the recorded decode loop takes) is recorded the same
way: its kind is the number of sequences, and nothing in it is left to a call.

Sequences beyond the step's own (the buffers hold ``seq_cap``) are empty: they start at the token count and own
the scratch slot and the scratch page.  Nothing in a graph clears memory with a memset node.  The kernels of a
replay are those of the same step run launch by launch, with the same arguments but for the addresses of the
buffers and the number of (empty) blocks, so the logits are the same bit for bit.
"""
from __future__ import annotations

import gc
from typing import Callable, Dict, List, Optional, Sequence

import numpy as np
import torch

from ..errors import GessoError, InvalidPlan
from ..parts.rmsnorm import ResidualStream
from .batch import BatchContext, StepEntry


class RecordedContext(BatchContext):
    """The step as the parts see it while it is recorded and while it is replayed: device fields are views of the
    recording's buffer; ``T`` is its token count, ``nseq`` its sequence capacity.  The host-side facts of the step at
    hand (``q_lens``, ``max_kv_len``, ``lead_single``) are for the calls that a replay makes anew."""

    def __init__(self, rec: "RecordedStep"):
        single = rec.single
        self._set(rec.engine.storage, T=rec.T, nseq=rec.seq_cap, n_want=0, q_lens=[1] * rec.T if single else [rec.T],
                  all_single=single, max_q_len=1 if single else rec.T, max_kv_len=None, decode_only=False,
                  token_ids=rec.field("tok"),
                  positions=rec.field("pos"), seq_of_token=rec.field("seq_of"), q_start=rec.field("q_start"),
                  kv_len=rec.field("kv_len"), slots=rec.field("slots"), want_rows=rec.field("want"),
                  block_tables=rec.tables)


class RecordedStep:
    """One recording: ``T`` tokens in up to ``seq_cap`` sequences of up to ``kv_cap`` keys, the blocks' ``key``."""

    TILE_ROOM = 1 << 16          # int32 entries for the tile lists that parts ask for
    HOST_COPIES = 4              # pinned buffers the steps are filled into in turn

    def __init__(self, engine, T: int, seq_cap: int, kv_cap: int, key, single: bool = False):
        """``single``: a step of ``T`` sequences that bring one token each (then ``seq_cap`` is ``T``)."""
        self.engine, self.T, self.seq_cap, self.kv_cap, self.key, self.single = engine, T, seq_cap, kv_cap, key, single
        storage = engine.storage
        self.max_blocks = -(-kv_cap // engine.page_size)
        self.groups = len(storage.num_pages)
        # one int32 buffer, pinned on the host and on the device, one copy a step
        self.layout: Dict[str, tuple] = {}
        at = 0
        for name, n in (("tok", T), ("pos", T), ("seq_of", T), ("q_start", seq_cap + 1), ("kv_len", seq_cap),
                        ("slots", seq_cap), ("want", T), ("tables", self.groups * seq_cap * self.max_blocks)):
            self.layout[name] = (at, n)
            at += n
        self._used = at
        # The host's side in several copies taken in turn: a step's copy to the device runs when the device gets to it,
        # which may be after the host has filled in the next step (a step that wants no logits makes the host wait for
        # nothing), so a buffer is written again only when the copy it was last the source of has been made.
        self.hosts = [torch.zeros(at + self.TILE_ROOM, dtype=torch.int32).pin_memory() for _ in range(self.HOST_COPIES)]
        self.copied = [None] * self.HOST_COPIES          # the event after each buffer's last copy
        self.turn = 0
        self.nps = [h.numpy() for h in self.hosts]
        self.host = self.hosts[0]
        self.dev = torch.zeros(at + self.TILE_ROOM, dtype=torch.int32, device=engine.device)
        self.np = self.nps[0]
        t = self.field("tables").view(self.groups, seq_cap, self.max_blocks)
        self.tables = [t[g] for g in range(self.groups)]
        self.tile_lists: Dict = {}           # what parts asked for: kind -> (offset, entries, maker)
        self.ctx = RecordedContext(self)
        self.items: List = []                # graphs and calls, in the order of a replay
        self.stream_end = None
        self._keys: Dict[int, object] = {}
        self._pool = self._graph = None

    def field(self, name: str) -> torch.Tensor:
        at, n = self.layout[name]
        return self.dev[at:at + n]

    def _host(self, name: str) -> np.ndarray:
        at, n = self.layout[name]
        return self.np[at:at + n]

    # ------------------------------------------------------------------ what parts ask of the recorder

    def key_of(self, part):
        """The entry of the recording's key (``Model.replay_key``) that ``part``'s block gave."""
        return self._keys[id(part)]

    def subtiles(self, kind, per_block: int, maker: Callable) -> torch.Tensor:
        """A tile list ``(3, blocks * per_block)`` on the device that every replay refills from ``maker(ctx)`` (host
        lists ``[sequences], [first rows], [row counts]``), filled up with tiles of no rows to as many blocks as the token
        count and the sequence capacity can make.  ``kind`` names the list: parts that ask for one kind share it."""
        if kind not in self.tile_lists:
            n = (-(-self.T // (32 * per_block)) + self.seq_cap) * per_block
            if self._used + 3 * n > self.host.numel():
                raise InvalidPlan("the recorded step's buffer has no room for another tile list")
            self.tile_lists[kind] = (self._used, n, maker)
            self._used += 3 * n
        at, n, _ = self.tile_lists[kind]
        return self.dev[at:at + 3 * n].view(3, n)

    def eager(self, call: Callable) -> None:
        """``call(ctx)`` is made at this place of every replay; the recording breaks off here and goes on after."""
        self._end_graph()
        self.items.append(call)
        self._begin_graph()

    # ------------------------------------------------------------------ recording

    def _begin_graph(self) -> None:
        self._graph = torch.cuda.CUDAGraph()
        self._graph.capture_begin(pool=self._pool)

    def _end_graph(self) -> None:
        graph, self._graph = self._graph, None
        graph.capture_end()
        self.items.append(graph)

    def record(self) -> None:
        """Record the blocks.  Nothing runs; every library product of this token count must have run before (its plan
        is made at its first call, which cannot be recorded)."""
        eng = self.engine
        model = eng.model
        for block, k in zip(model.blocks, self.key):
            for part in vars(block).values():
                self._keys[id(part)] = k
        self._pool = torch.cuda.graph_pool_handle()
        side = torch.cuda.Stream(device=eng.device)
        torch.cuda.synchronize(eng.device)
        side.wait_stream(torch.cuda.current_stream(eng.device))
        # no collection of cyclic garbage while the stream is capturing: a finalizer that frees pinned memory or a
        # graph of an engine long gone makes calls the capture forbids, and the process aborts
        collecting = gc.isenabled()
        gc.disable()
        self.ctx.recording = self
        try:
            with torch.cuda.stream(side):
                self._begin_graph()
                try:
                    stream = model.run_blocks(self.ctx)
                finally:
                    if self._graph is not None:
                        self._end_graph()
        finally:
            self.ctx.recording = None
            if collecting:
                gc.enable()
        torch.cuda.current_stream(eng.device).wait_stream(side)
        # the stream as the last block left it and what is still to be added to it: the final norm reads both
        self.stream_end = (stream.res, stream.pending)

    # ------------------------------------------------------------------ a step

    def fill(self, entries: Sequence[StepEntry], token_ids: np.ndarray) -> Optional[int]:
        """The host buffer for this step.  Returns the number of wanted rows, or None if the step does not fit the
        recording (more tiles than it holds); nothing has been launched then."""
        eng = self.engine
        manager, storage = eng.manager, eng.storage
        T, S, B = self.T, self.seq_cap, self.max_blocks
        n = len(entries)
        lens = [len(e.tokens) for e in entries]
        rcs = [manager.get(e.rid) for e in entries]
        lens_a = np.asarray(lens, dtype=np.int64)
        held = np.asarray([rc.length for rc in rcs], dtype=np.int64)
        starts = np.zeros(n + 1, dtype=np.int64)
        starts[1:] = np.cumsum(lens_a)
        ctx = self.ctx
        ctx.q_lens = lens
        ctx.max_kv_len = int((held + lens_a).max())
        ctx._tiles = None
        if sum(len(e.want) for e in entries) > T:
            return None                                       # (rows wanted more than once: more than the buffer holds)
        self.turn = (self.turn + 1) % self.HOST_COPIES
        if self.copied[self.turn] is not None:
            self.copied[self.turn].synchronize()              # (the copy of HOST_COPIES steps ago: long done, as a rule)
        self.host, self.np = self.hosts[self.turn], self.nps[self.turn]
        made = []
        for at, cnt, maker in self.tile_lists.values():
            lists = maker(ctx)
            if len(lists[0]) > cnt:
                return None
            made.append((at, cnt, lists))
        self._host("tok")[:] = token_ids
        # token t of sequence i stands at position held[i] + (t - starts[i])
        self._host("pos")[:] = np.arange(T, dtype=np.int64) + np.repeat(held - starts[:-1], lens_a)
        self._host("seq_of")[:] = np.repeat(np.arange(n, dtype=np.int32), lens_a)
        q = self._host("q_start")
        q[:n + 1] = starts
        q[n + 1:] = T
        kv = self._host("kv_len")
        kv[:n] = held + lens_a
        kv[n:] = 0
        sl = self._host("slots")
        sl[:n] = [storage.scratch_slot if rc.slot is None else rc.slot for rc in rcs]
        sl[n:] = storage.scratch_slot
        tab = self._host("tables").reshape(self.groups, S, B)
        for g in range(self.groups):
            scratch = storage.num_pages[g]
            tg = tab[g]
            tg[:] = scratch                                   # the scratch page: never read
            for i, rc in enumerate(rcs):
                t = rc.tables[g]
                m = min(len(t), B)
                tg[i, :m] = t[:m]
            tg[tg < 0] = scratch                              # pages a window has passed and given back
        for at, cnt, (seq, row, num) in made:
            # the step's tiles at the list's end, tiles of no rows before them (they name row 0 of sequence 0, which
            # exist): the kernel starts its blocks from the end of the list, so the empty ones come last
            part = self.np[at:at + 3 * cnt].reshape(3, cnt)
            m = len(seq)
            part[:, :cnt - m] = 0
            part[0, cnt - m:], part[1, cnt - m:], part[2, cnt - m:] = seq, row, num
        want = self._host("want")
        w = 0
        for i, e in enumerate(entries):
            for x in e.want:
                want[w] = int(starts[i]) + int(x)
                w += 1
        return w

    def launch(self, n_want: int) -> Optional[torch.Tensor]:
        """The filled step: one copy, the graphs and calls in order, then the final norm and the head of the wanted rows."""
        self.dev.copy_(self.host, non_blocking=True)
        done = self.copied[self.turn] = self.copied[self.turn] or torch.cuda.Event()
        done.record()
        ctx = self.ctx
        for item in self.items:
            if isinstance(item, torch.cuda.CUDAGraph):
                item.replay()
            else:
                item(ctx)
        if n_want == 0:
            return None
        res, pending = self.stream_end
        return self.engine.model.logits(ResidualStream(res, pending), self.field("want")[:n_want])


class StepRecorder:
    """Which steps an engine records, and the recordings it holds.

    A step is recorded when it is the fourth of its kind: steps of one kind share the token count, the room their
    longest sequence needs in a block table (a power of two of keys), the blocks' key and the room for sequences.  The first ones, run launch
    by launch, have made the plans of the library's products, which a recording cannot make, and a kind that comes
    once in a while (the last, shorter step of a wave of prompts) is not worth the four milliseconds of a recording."""

    SEEN_BEFORE = 3
    MAX_RECORDINGS = 4           # each holds the activations of its token count
    MAX_SEEN = 4096              # kinds whose comings are counted
    IDLE_STEPS = 256             # a recording unused for so many steps makes room when another kind wants it
    SEQ_CAP = 64                 # sequences in a recorded step with prompt portions: room for so many, or twice, ...
    MAX_SEQ_CAP = 512            # ... up to so many
    MAX_SINGLE = 1024            # sequences in a recorded step of single tokens
    MIN_KV_CAP = 4096

    def __init__(self, engine):
        self.engine = engine
        self.seen: Dict = {}
        self.recordings: Dict = {}      # kind -> RecordedStep, or None where recording was refused
        self.refused: Dict = {}         # kind -> the error that refused it
        self.replays = 0
        self.clock = 0                  # steps that could have been replayed, counted
        self.used: Dict = {}            # kind -> the clock when its recording last served

    def kind_of(self, entries: Sequence[StepEntry]):
        eng = self.engine
        lens = [len(e.tokens) for e in entries]
        if max(lens) == 1:
            # single tokens only: the recorded decode loop takes up to its own limit of them without the host; more
            # than that are one step of library products, which is worth recording
            if not getattr(eng, "DECODE_MAX_BATCH", 0) < len(entries) <= self.MAX_SINGLE:
                return None
        elif len(entries) > self.MAX_SEQ_CAP:
            return None
        longest = max(eng.manager.get(e.rid).length + n for e, n in zip(entries, lens))
        key = eng.model.replay_key(lens, longest)
        if key is None:
            return None
        kv_cap = self.MIN_KV_CAP
        while kv_cap < longest:
            kv_cap *= 2
        # room for the step's sequences: as many as it has where every one brings a single token, else 64, 128, ...
        seq_cap = len(entries)
        if max(lens) > 1:
            seq_cap = self.SEQ_CAP
            while seq_cap < len(entries):
                seq_cap *= 2
        return sum(lens), kv_cap, key, seq_cap

    def recording_for(self, entries: Sequence[StepEntry]) -> Optional[RecordedStep]:
        """The recording that takes this step, made now if the step is the fourth of its kind; None: launch by launch."""
        kind = self.kind_of(entries)
        if kind is None:
            return None
        self.clock += 1
        rec = self.recordings.get(kind)
        if rec is None and kind not in self.recordings:
            if len(self.seen) >= self.MAX_SEEN and kind not in self.seen:
                self.seen.clear()               # (a server sees a new token count in many of its steps: the tally starts over)
            n = self.seen[kind] = self.seen.get(kind, 0) + 1
            if n <= self.SEEN_BEFORE:
                return None
            held = [k for k, r in self.recordings.items() if r is not None]
            if len(held) >= self.MAX_RECORDINGS:
                # room for this kind only if a recording has lain idle for a while (sequences grow out of their block
                # tables' room, a scheduler's budget changes): the one unused longest goes, with its graphs and buffers
                oldest = min(held, key=lambda k: self.used[k])
                if self.clock - self.used[oldest] < self.IDLE_STEPS:
                    return None
                device = getattr(self.engine, "device", None)
                if device is not None and device.type == "cuda":
                    torch.cuda.synchronize(device)             # (its last replay may still be running: graphs go when idle)
                del self.recordings[oldest], self.used[oldest]
                self.seen.pop(oldest, None)
            T, kv_cap, key, seq_cap = kind
            rec = RecordedStep(self.engine, T, seq_cap, kv_cap, key, single=max(len(e.tokens) for e in entries) == 1)
            try:
                rec.record()
            except GessoError as err:
                # a part or a kernel that refuses to be recorded: steps of this kind stay with the launches
                self.refused[kind] = err
                rec = None
            self.recordings[kind] = rec
        if rec is not None:
            self.used[kind] = self.clock
        return rec
