"""The cache manager: which pages and which slot each request holds.

Per-token state (keys and values) lies in pages of ``page_size`` tokens; each request has a
block table per *group*.  A group is the set of layers with the same needs: the same key/value
shape and the same reach (all keys, or a window of them); each group has pages of its own, so
that a windowed group can give back the pages its window has passed while a full group keeps
them.  Per-request state of fixed size (a convolution's history, a recurrent state) lies in one
*slot* per request, shared by all layers that keep such state, held from admission to release
and zeroed when handed out.

The reference's manager keeps one page list per (layer, K or V) per session and grows it on
append (``src/Inference/kv_manager.jl:68-95``, ``:234-291``); exhaustion is a typed error
(``:246-257``).  Here a page id addresses the same page in every layer of its group, exhaustion
of a pool raises :class:`~gesso_amd.errors.OutOfPages` before anything is changed, and what to
do then is the scheduler's decision.

This file is host-side bookkeeping only; the device memory lies in :mod:`gesso_amd.cache.storage`.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Optional, Sequence, Tuple

from ..errors import InvalidPlan, ResourceLimit
from ..parts.base import PagedKV, SlotState
from .pages import PagePool, SlotPool

RELEASED = -1   # a block-table entry whose page the window has passed


@dataclass(frozen=True)
class PagedGroup:
    index: int
    need: PagedKV
    members: Tuple[int, ...]        # positions in the schedule that keep their cache here


@dataclass(frozen=True)
class SlotMember:
    call: int                        # position in the schedule
    need: SlotState


@dataclass(frozen=True)
class CacheLayout:
    """How the schedule's caches are grouped; made once per model."""

    paged: Tuple[PagedGroup, ...]
    slots: Tuple[SlotMember, ...]
    group_of_call: Dict[int, int]    # schedule position -> paged group index (own caches only)
    source_of_call: Dict[int, int]   # schedule position -> the position whose cache it uses

    @staticmethod
    def plan(needs: Sequence[Optional[object]], cache_of: Sequence[Optional[int]]) -> "CacheLayout":
        """``needs[i]``: what call ``i`` keeps (None if nothing or if it reads ``cache_of[i]``)."""
        groups: Dict[PagedKV, List[int]] = {}
        slots: List[SlotMember] = []
        for i, need in enumerate(needs):
            if isinstance(need, PagedKV):
                groups.setdefault(need, []).append(i)
            elif isinstance(need, SlotState):
                slots.append(SlotMember(i, need))
            elif need is not None:
                raise InvalidPlan(f"schedule entry {i} asks for an unknown kind of cache: {need!r}")
        paged = tuple(PagedGroup(g, need, tuple(m)) for g, (need, m) in enumerate(groups.items()))
        group_of = {c: g.index for g in paged for c in g.members}
        source = {}
        for i, src in enumerate(cache_of):
            s = i if src is None else src
            while cache_of[s] is not None:
                s = cache_of[s]
            source[i] = s
        return CacheLayout(paged, tuple(slots), group_of, source)


@dataclass
class RequestCache:
    slot: Optional[int]
    length: int = 0                                   # tokens whose state is in the cache
    tables: List[List[int]] = field(default_factory=list)   # per paged group: page ids, RELEASED for passed ones


class CacheManager:
    def __init__(self, layout: CacheLayout, page_size: int, num_pages, num_slots: int, max_length: int):
        """``num_pages``: pages per group, an int for all groups or a sequence per group."""
        if page_size <= 0:
            raise InvalidPlan("page_size must be positive", page_size=page_size)
        self.layout = layout
        self.page_size = int(page_size)
        if isinstance(num_pages, int):
            num_pages = [num_pages] * len(layout.paged)
        if len(num_pages) != len(layout.paged):
            raise InvalidPlan("num_pages needs one count per group", groups=len(layout.paged))
        self.pools = [PagePool(n) for n in num_pages]
        self.slot_pool = SlotPool(num_slots)
        self.needs_slot = bool(layout.slots)
        self.max_length = int(max_length)
        self.requests: Dict[Hashable, RequestCache] = {}
        self.fresh_slots: List[int] = []    # slots handed out and not yet given their initial value on the device
        # debug poison: with track_released set, what comes back is listed here until the engine has overwritten it
        self.track_released = False
        self.released_pages: List[List[int]] = [[] for _ in self.pools]
        self.released_slots: List[int] = []

    # ------------------------------------------------------------------ requests

    def admit(self, rid: Hashable) -> RequestCache:
        if rid in self.requests:
            raise InvalidPlan(f"request {rid!r} is already live")
        slot = None
        if self.needs_slot:
            slot = self.slot_pool.take(1)[0]
            self.fresh_slots.append(slot)
        rc = RequestCache(slot=slot, tables=[[] for _ in self.pools])
        self.requests[rid] = rc
        return rc

    def get(self, rid: Hashable) -> RequestCache:
        try:
            return self.requests[rid]
        except KeyError:
            raise InvalidPlan(f"request {rid!r} is not live") from None

    def pages_needed(self, rid: Hashable, n_new: int) -> List[int]:
        """Per group: pages that must be taken so that ``n_new`` more tokens fit."""
        rc = self.get(rid)
        blocks = -(-(rc.length + n_new) // self.page_size)
        return [max(0, blocks - len(t)) for t in rc.tables]

    def reserve(self, rid: Hashable, n_new: int) -> None:
        """Take the pages that ``n_new`` more tokens need, in every group, or none at all."""
        rc = self.get(rid)
        if n_new < 0:
            raise InvalidPlan("cannot reserve a negative number of tokens")
        if rc.length + n_new > self.max_length:
            raise ResourceLimit(f"request {rid!r} would hold {rc.length + n_new} tokens, the context holds {self.max_length}",
                                length=rc.length + n_new, max_length=self.max_length)
        need = self.pages_needed(rid, n_new)
        for g, n in enumerate(need):
            if n > self.pools[g].n_free:
                raise self.pools[g].exhausted(
                    f"group {g}: {n} pages asked for request {rid!r}, {self.pools[g].n_free} free",
                    group=g, asked=n, free=self.pools[g].n_free, total=self.pools[g].total)
        for g, n in enumerate(need):
            rc.tables[g].extend(self.pools[g].take(n))

    def reserve_many(self, asks: Sequence[Tuple[Hashable, int]]) -> None:
        """:meth:`reserve` for several requests (each named once) as one decision: all fit or nothing is taken."""
        groups = len(self.pools)
        total = [0] * groups
        needs = []
        ps = self.page_size
        for rid, n_new in asks:
            rc = self.get(rid)
            if n_new < 0:
                raise InvalidPlan("cannot reserve a negative number of tokens")
            if rc.length + n_new > self.max_length:
                raise ResourceLimit(f"request {rid!r} would hold {rc.length + n_new} tokens, the context holds {self.max_length}",
                                    length=rc.length + n_new, max_length=self.max_length)
            blocks = -(-(rc.length + n_new) // ps)
            need = None                                    # (most decoded tokens need no page)
            for g, t in enumerate(rc.tables):
                n = blocks - len(t)
                if n > 0:
                    if need is None:
                        need = [0] * groups
                    need[g] = n
                    total[g] += n
            if need is not None:
                needs.append((rc, need))
        for g, n in enumerate(total):
            if n > self.pools[g].n_free:
                raise self.pools[g].exhausted(f"group {g}: {n} pages asked for this step, {self.pools[g].n_free} free",
                                              group=g, asked=n, free=self.pools[g].n_free, total=self.pools[g].total)
        for rc, need in needs:
            for g, n in enumerate(need):
                if n:
                    rc.tables[g].extend(self.pools[g].take(n))

    def commit(self, rid: Hashable, n_new: int) -> None:
        """``n_new`` tokens were written: advance, and give back the pages a window has passed."""
        rc = self.get(rid)
        rc.length += n_new
        if -(-rc.length // self.page_size) > min((len(t) for t in rc.tables), default=1 << 60):
            raise InvalidPlan(f"request {rid!r} advanced beyond its reserved pages")
        for g, group in enumerate(self.layout.paged):
            w = group.need.window
            if w is None:
                continue
            first_needed = rc.length - w + 1          # oldest key the next query reads
            passed = max(0, first_needed) // self.page_size
            table = rc.tables[g]
            gone = [table[b] for b in range(min(passed, len(table))) if table[b] != RELEASED]
            if gone:
                for b in range(min(passed, len(table))):
                    table[b] = RELEASED
                self.pools[g].give_back(gone)
                if self.track_released:
                    self.released_pages[g].extend(gone)

    def release(self, rid: Hashable) -> None:
        """The request is over (finished, aborted, preempted): everything it holds comes back."""
        rc = self.requests.pop(rid, None)
        if rc is None:
            raise InvalidPlan(f"request {rid!r} is not live")
        for g, table in enumerate(rc.tables):
            held = [p for p in table if p != RELEASED]
            self.pools[g].give_back(held)
            if self.track_released:
                self.released_pages[g].extend(held)
        if rc.slot is not None:
            self.slot_pool.give_back([rc.slot])
            if rc.slot in self.fresh_slots:
                self.fresh_slots.remove(rc.slot)
            if self.track_released:
                self.released_slots.append(rc.slot)

    def take_released(self):
        """``(pages per group, slots)`` given back since the last call; the lists start anew."""
        pages, slots = self.released_pages, self.released_slots
        self.released_pages, self.released_slots = [[] for _ in self.pools], []
        return pages, slots

    # ------------------------------------------------------------------ accounting

    def stats(self) -> dict:
        return {
            "pages_total": [p.total for p in self.pools], "pages_free": [p.n_free for p in self.pools],
            "slots_total": self.slot_pool.total, "slots_free": self.slot_pool.n_free,
            "requests": len(self.requests),
        }

    def check(self) -> None:
        """No page lost, none held twice; tables and pools agree."""
        for g, pool in enumerate(self.pools):
            pool.check()
            held = [p for rc in self.requests.values() for p in rc.tables[g] if p != RELEASED]
            assert len(held) == len(set(held)), f"group {g}: a page is held twice"
            assert set(held) == pool._out, f"group {g}: tables and pool disagree"
        self.slot_pool.check()
        slots = [rc.slot for rc in self.requests.values() if rc.slot is not None]
        assert len(slots) == len(set(slots)), "a slot is held twice"
        assert set(slots) == self.slot_pool._out, "slots and pool disagree"
