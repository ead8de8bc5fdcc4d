"""One step's batch: entries as the caller gives them, and the flattened form the kernels read.

An entry is a request's next tokens (a portion of its prompt, or one decoded token) and the
places among them whose logits are wanted.  All entries of a step are flattened into one row of
tokens; per token its position and its sequence, per sequence its start among the rows, its
length after the step, its slot and its block tables.  Everything the device needs travels in
one int32 buffer, one copy per step.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Hashable, List, Sequence

import numpy as np
import torch

from ..errors import InvalidPlan


@dataclass
class StepEntry:
    rid: Hashable
    tokens: Sequence[int]
    want: Sequence[int] = field(default_factory=list)   # indices into ``tokens``


def check_entries(entries: List[StepEntry], manager, vocab: int) -> np.ndarray:
    """Refuse a step that cannot run, before anything is reserved or written.  Returns the step's token ids, all
    entries' in order, as one int64 array (the context takes them as they are)."""
    seen = set()
    lens = []
    for e in entries:
        manager.get(e.rid)
        if e.rid in seen:
            raise InvalidPlan(f"request {e.rid!r} occurs twice in one step")
        seen.add(e.rid)
        n = len(e.tokens)
        if n < 1:
            raise InvalidPlan(f"request {e.rid!r} brings no tokens to this step")
        lens.append(n)
        for w in e.want:
            if not 0 <= int(w) < n:
                raise InvalidPlan(f"request {e.rid!r} wants logits at place {w} of {n} tokens")
    # one array for all entries: the ids are checked at once (a bad one is then looked for entry by entry)
    ids = np.concatenate([np.asarray(e.tokens, dtype=np.int64) for e in entries]) if len(entries) > 1 \
        else np.asarray(entries[0].tokens, dtype=np.int64)
    if ids.size and (int(ids.min()) < 0 or int(ids.max()) >= vocab):
        t = int(ids[(ids < 0) | (ids >= vocab)][0])
        raise InvalidPlan(f"token id {t} outside the vocabulary of {vocab}", token=t, vocab=vocab)
    return ids


# What parts may read of a step.  Host-side facts kernels are chosen by: T (tokens), nseq, n_want, q_lens, all_single,
# max_q_len, max_kv_len (None: unknown here, kernels read kv_len on the device), decode_only (every sequence brings
# one token and wants its logits, in order).  Device tensors, int32: token_ids, positions, seq_of_token (T each),
# q_start (nseq + 1), kv_len, slots (nseq each), want_rows (n_want), block_tables (per paged group (nseq, blocks)).
CONTEXT_FIELDS = ("T", "nseq", "n_want", "q_lens", "all_single", "max_q_len", "max_kv_len", "decode_only",
                  "token_ids", "positions", "seq_of_token", "q_start", "kv_len", "slots", "want_rows", "block_tables")


class BatchContext:
    """A step as the parts see it: the fields of ``CONTEXT_FIELDS``, the cache views, the tiling of queries.

    Whoever builds a context (a step from entries, the recorded decode step from its static buffers) hands all
    fields to :meth:`_set`, which refuses a missing or an unknown one: a field added to the list must be served
    by every builder before anything runs."""

    # While a step of prompt portions is recorded for replay (engine/planned.py): the recorder.  A part whose launches
    # depend on more than the token count and device buffers asks it for tile lists that every replay refills
    # (``recording.subtiles``) and hands it what must run anew at every replay (``recording.eager``).
    recording = None

    def _set(self, storage, **fields) -> None:
        if set(fields) != set(CONTEXT_FIELDS):
            missing, unknown = set(CONTEXT_FIELDS) - set(fields), set(fields) - set(CONTEXT_FIELDS)
            raise InvalidPlan(f"{type(self).__name__} must set the context's fields exactly",
                              missing=sorted(missing), unknown=sorted(unknown))
        for k, v in fields.items():
            setattr(self, k, v)
        self._storage = storage
        self._tiles = None

    def cache_view(self, call: int):
        return self._storage.view(call, self.block_tables)

    @property
    def lead_single(self) -> int:
        """How many sequences at the batch's head bring one token each (decoded tokens come before prompt portions)."""
        n = 0
        while n < len(self.q_lens) and self.q_lens[n] == 1:
            n += 1
        return n

    def query_tiles(self, rows: int = 16, skip: int = 0) -> torch.Tensor:
        """int32 ``(3, ntiles)``: sequence, first row, row count of each tile of at most ``rows`` consecutive
        queries of one sequence, for the sequences from ``skip`` on; made once per step, on first use."""
        if self._tiles is None or self._tiles[0] != (rows, skip):
            seq, row, cnt = [], [], []
            at = 0
            for i, n in enumerate(self.q_lens):
                if i >= skip:
                    for a in range(0, n, rows):
                        seq.append(i)
                        row.append(at + a)
                        cnt.append(min(rows, n - a))
                at += n
            t = torch.tensor([seq, row, cnt], dtype=torch.int32).pin_memory().to(self.token_ids.device, non_blocking=True)
            self._tiles = ((rows, skip), t)
        return self._tiles[1]

    def subtile_lists(self, wq: int, skip: int = 0, paired: bool = True):
        """:func:`subtile_lists` of this step's sequences from ``skip`` on, on the host."""
        return subtile_lists(self.q_lens, wq, skip, paired)

    def query_subtiles(self, wq: int, skip: int = 0, paired: bool = True) -> torch.Tensor:
        """int32 ``(3, blocks * wq)`` on the device: :func:`subtile_lists` of this step's sequences from ``skip`` on."""
        key = ("sub", wq, skip, paired)
        if self._tiles is None or self._tiles[0] != key:
            t = torch.tensor(subtile_lists(self.q_lens, wq, skip, paired), dtype=torch.int32)
            self._tiles = (key, t.pin_memory().to(self.token_ids.device, non_blocking=True))
        return self._tiles[1]


def subtile_lists(q_lens: Sequence[int], wq: int, skip: int = 0, paired: bool = True):
    """``[sequence], [first row], [row count]`` of sub-tiles of at most 32 consecutive queries of one sequence, ``wq`` of
    them a block (a count of 0 fills a block up), for the sequences from ``skip`` on; rows count through all sequences.

    ``paired`` (causal attention without a window): a block gets late sub-tiles, which see many keys, together with
    early ones, which see few: the sub-tiles of a sequence are paired from both ends (last with first, ...), a block
    takes ``wq / 2`` pairs, the late ones in the first half of its entries and their partners in the second, so that
    every block has about the same number of (query, key) pairs to work through.  Otherwise blocks take neighbours."""
    seq, row, cnt = [], [], []
    at = 0
    for i, n in enumerate(q_lens):
        if i >= skip:
            subs = [(at + a, min(32, n - a)) for a in range(0, n, 32)]
            none = (at, 0)
            if paired and wq >= 2:
                pairs, lo, hi = [], 0, len(subs) - 1
                while lo < hi:
                    pairs.append((subs[hi], subs[lo]))
                    lo, hi = lo + 1, hi - 1
                if lo == hi:
                    pairs.append((subs[lo], none))
                half = wq // 2
                blocks = []
                for a in range(0, len(pairs), half):
                    group = pairs[a:a + half] + [(none, none)] * (half - len(pairs[a:a + half]))
                    blocks.append([p[0] for p in group] + [p[1] for p in group])
            else:
                blocks = [subs[a:a + wq] + [none] * (wq - len(subs[a:a + wq])) for a in range(0, len(subs), wq)]
            for b in blocks:
                for r, c in b:
                    seq.append(i)
                    row.append(r)
                    cnt.append(c)
        at += n
    return [seq, row, cnt]


class StepContext(BatchContext):
    """The flattened batch of one step on the device."""

    def __init__(self, entries: List[StepEntry], manager, storage, vocab: int, device, token_ids: np.ndarray = None):
        """``token_ids``: the entries' tokens in order as one array, where the caller has it (``check_entries``)."""
        ps = manager.page_size
        nseq = len(entries)
        lens = [len(e.tokens) for e in entries]
        T = sum(lens)
        rcs = [manager.get(e.rid) for e in entries]
        lens_a = np.asarray(lens, dtype=np.int64)
        starts = np.zeros(nseq + 1, dtype=np.int32)
        starts[1:] = np.cumsum(lens_a)
        if token_ids is None:
            token_ids = np.concatenate([np.asarray(e.tokens, dtype=np.int64) for e in entries])
        tokens = token_ids
        held = np.asarray([rc.length for rc in rcs], dtype=np.int64)
        # token t of sequence i stands at position held[i] + (t - starts[i])
        seq_of = np.repeat(np.arange(nseq, dtype=np.int32), lens_a)
        positions = (np.arange(T, dtype=np.int64) + np.repeat(held - starts[:-1], lens_a)).astype(np.int32)
        want_rows: List[int] = []
        for i, e in enumerate(entries):
            if e.want:
                a = int(starts[i])
                want_rows.extend(a + int(w) for w in e.want)
        kv_len = (held + lens_a).astype(np.int32)
        max_kv_len = int(kv_len.max()) if nseq else 0
        slots = np.asarray([storage.scratch_slot if rc.slot is None else rc.slot for rc in rcs], dtype=np.int32)
        n_groups = len(manager.pools)
        max_blocks = max(1, -(-max_kv_len // ps))
        tables = np.empty((n_groups, nseq, max_blocks), dtype=np.int32)
        for g in range(n_groups):
            scratch = storage.num_pages[g]
            tables[g, :, :] = scratch                         # the scratch page: never read
            for i, rc in enumerate(rcs):
                t = rc.tables[g]
                n = min(len(t), max_blocks)
                tables[g, i, :n] = t[:n]
            tab = tables[g]
            tab[tab < 0] = scratch                            # pages a window has passed and given back
        self.max_blocks = max_blocks

        parts = [tokens.astype(np.int32), positions, seq_of, starts, kv_len, slots,
                 np.asarray(want_rows, dtype=np.int32), tables.reshape(-1)]
        sizes = [p.size for p in parts]
        host = torch.from_numpy(np.concatenate(parts)).pin_memory() if device.type == "cuda" else torch.from_numpy(np.concatenate(parts))
        dev = host.to(device, non_blocking=True)
        views = torch.split(dev, sizes)
        token_ids, positions_d, seq_of_d, q_start, kv_len_d, slots_d, want_d, flat_tables = views
        tables_d = [flat_tables.view(n_groups, nseq, max_blocks)[g] for g in range(n_groups)] if n_groups else []
        self._set(storage, T=T, nseq=nseq, n_want=len(want_rows), q_lens=lens, all_single=all(n == 1 for n in lens),
                  max_q_len=max(lens), max_kv_len=max_kv_len, decode_only=False, token_ids=token_ids,
                  positions=positions_d, seq_of_token=seq_of_d, q_start=q_start, kv_len=kv_len_d, slots=slots_d,
                  want_rows=want_d, block_tables=tables_d)
        self._host = host          # keeps the pinned buffer alive until the copy has run
