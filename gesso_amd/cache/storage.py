"""Device memory of the cache: pages per group, state per slot.

Pages of a group: a key tensor ``(members, num_pages + 1, n_kv_heads, page_size, head_dim)`` and a value tensor
of the same shape but for its last axis (the group's value width, which may differ from the key's or be zero),
in the activation type; a page id addresses the same page in both and in every layer of the group.  A head's rows
of a page are contiguous (``page_size x width``), which is what the attention kernels stream.  Slot state: per state-keeping layer and state
name a tensor ``(num_slots + 1, *shape)`` of the type the layer asked for (float32 or bfloat16), with the value a
fresh slot starts from in ``state_init``.  The extra page and the extra slot at the end
belong to no request: padded entries of a fixed-size batch write there.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Optional

import torch

from ..errors import InvalidPlan
from .manager import CacheLayout

_DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}


@dataclass
class PagedView:
    """What an attention-like mixer sees of its cache in one step."""

    k: torch.Tensor                  # (num_pages + 1, nkv, page_size, head_dim)
    v: torch.Tensor                  # (num_pages + 1, nkv, page_size, value width)
    block_table: torch.Tensor        # int32 (nseq, max_blocks) of this step
    page_size: int
    write: bool                      # False: this call reads another call's cache


@dataclass
class SlotView:
    state: Dict[str, torch.Tensor]   # name -> (num_slots + 1, *shape)
    write: bool


class CacheStorage:
    def __init__(self, layout: CacheLayout, page_size: int, num_pages, num_slots: int, dtype, device):
        self.layout = layout
        self.page_size = page_size
        if isinstance(num_pages, int):
            num_pages = [num_pages] * len(layout.paged)
        self.num_pages = list(num_pages)
        self.num_slots = num_slots
        self.keys, self.values = [], []
        for g, n in zip(layout.paged, num_pages):
            lead = (len(g.members), n + 1, g.need.n_kv_heads, page_size)
            self.keys.append(torch.zeros(lead + (g.need.head_dim,), dtype=dtype, device=device))
            self.values.append(torch.zeros(lead + (g.need.value_width,), dtype=dtype, device=device))
        self.member_index = {c: i for g in layout.paged for i, c in enumerate(g.members)}
        # States of one shape, type and initial value share a pool (members, slots + 1, *shape), as the layers of a page
        # group share theirs: a step's fresh slots then take one fill a pool, not one a layer.  state[call][name] is
        # the member's own (slots + 1, *shape).
        self.state: Dict[int, Dict[str, torch.Tensor]] = {}
        self.state_init: Dict[int, Dict[str, float]] = {}
        alike: Dict[tuple, list] = {}
        for m in layout.slots:
            self.state[m.call], self.state_init[m.call] = {}, {}
            for name, shape, dt, init in m.need.entries():
                if dt not in _DTYPES:
                    raise InvalidPlan(f"state {name!r} of schedule entry {m.call} asks for {dt!r}; slots hold "
                                      f"{sorted(_DTYPES)}")
                alike.setdefault((tuple(shape), dt, float(init)), []).append((m.call, name))
                self.state_init[m.call][name] = init
        self.state_pools = []                      # (pool, initial value)
        for (shape, dt, init), members in alike.items():
            pool = torch.full((len(members), num_slots + 1) + shape, init, dtype=_DTYPES[dt], device=device)
            self.state_pools.append((pool, init))
            for i, (call, name) in enumerate(members):
                self.state[call][name] = pool[i]

    @property
    def scratch_page(self):
        return list(self.num_pages)

    @property
    def scratch_slot(self) -> int:
        return self.num_slots

    def view(self, call: int, block_tables) -> Optional[object]:
        """The cache of schedule position ``call`` (its own, or the one it reads)."""
        src = self.layout.source_of_call[call]
        write = src == call
        if src in self.layout.group_of_call:
            g = self.layout.group_of_call[src]
            i = self.member_index[src]
            return PagedView(self.keys[g][i], self.values[g][i], block_tables[g], self.page_size, write)
        if src in self.state:
            return SlotView(self.state[src], write)
        return None

    # ------------------------------------------------------------------ filling (initial values, debug poison)

    def fill_slots(self, ops, slots, value) -> None:
        """``value``: a number, ``"initial"`` for each state's own initial value, or None for NaN."""
        ids = None
        for pool, init in self.state_pools:
            if ids is None:
                ids = torch.tensor(list(slots), dtype=torch.int32, device=pool.device)
            v = init if value == "initial" else (float("nan") if value is None else value)
            ops.fill_rows(pool, ids, v, planes=2)

    def fill_pages(self, ops, group: int, pages, value: float) -> None:
        """Every layer's keys and values of the given pages of one group."""
        ids = torch.tensor(list(pages), dtype=torch.int32, device=self.keys[group].device)
        for pool in (self.keys[group], self.values[group]):
            if pool.numel():
                ops.fill_rows(pool, ids, value, planes=2)          # a plane of (pages + 1) rows per member

    def poison_all(self) -> None:
        """NaN everywhere but in the spare page and slot (padded rows of a recorded batch compute on those)."""
        for pool in self.keys + self.values:
            pool[:, :-1].fill_(float("nan"))
        for pool, _ in self.state_pools:
            pool[:, :-1].fill_(float("nan"))

    def bytes(self) -> int:
        n = sum(t.numel() * t.element_size() for t in self.keys + self.values)
        n += sum(pool.numel() * pool.element_size() for pool, _ in self.state_pools)
        return n
