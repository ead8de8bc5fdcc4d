"""Device memory of the cache: pages per group, state per slot.

Pages of a group: one tensor ``(members, 2, num_pages + 1, n_kv_heads, page_size, head_dim)`` in the
activation type; index 0/1 of the second axis is K/V, so that a page id addresses the same page
in every layer of the group.  A head's rows of a page are contiguous (``page_size x head_dim``),
which is what the attention kernels stream.  Slot state: per state-keeping layer and state
name a float32 tensor ``(num_slots + 1, *shape)``.  The extra page and the extra slot at the end
belong to no request: padded entries of a fixed-size batch write there.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Optional

import torch

from .manager import CacheLayout

_DTYPES = {"float32": torch.float32}


@dataclass
class PagedView:
    """What an attention-like mixer sees of its cache in one step."""

    k: torch.Tensor                  # (num_pages + 1, nkv, page_size, d)
    v: torch.Tensor
    block_table: torch.Tensor        # int32 (nseq, max_blocks) of this step
    page_size: int
    write: bool                      # False: this call reads another call's cache


@dataclass
class SlotView:
    state: Dict[str, torch.Tensor]   # name -> (num_slots + 1, *shape) float32
    write: bool


class CacheStorage:
    def __init__(self, layout: CacheLayout, page_size: int, num_pages, num_slots: int, dtype, device):
        self.layout = layout
        self.page_size = page_size
        if isinstance(num_pages, int):
            num_pages = [num_pages] * len(layout.paged)
        self.num_pages = list(num_pages)
        self.num_slots = num_slots
        self.kv = []
        for g, n in zip(layout.paged, num_pages):
            self.kv.append(torch.zeros((len(g.members), 2, n + 1, g.need.n_kv_heads, page_size, g.need.head_dim),
                                       dtype=dtype, device=device))
        self.member_index = {c: i for g in layout.paged for i, c in enumerate(g.members)}
        self.state: Dict[int, Dict[str, torch.Tensor]] = {}
        for m in layout.slots:
            self.state[m.call] = {name: torch.zeros((num_slots + 1,) + tuple(shape), dtype=_DTYPES[dt], device=device)
                                  for name, shape, dt in m.need.tensors}

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
            kv = self.kv[g][self.member_index[src]]
            return PagedView(kv[0], kv[1], block_tables[g], self.page_size, write)
        if src in self.state:
            return SlotView(self.state[src], write)
        return None

    def bytes(self) -> int:
        n = sum(t.numel() * t.element_size() for t in self.kv)
        n += sum(t.numel() * t.element_size() for d in self.state.values() for t in d.values())
        return n
