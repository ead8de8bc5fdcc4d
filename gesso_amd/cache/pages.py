"""Pools of numbered things handed out and taken back: cache pages and state slots.

A pool never hands out an id twice, and taking back an id that is not out is an error; both
are what the tests of the manager lean on.  Ids that come back are used again first (a stack),
so a small pool reuses its pages quickly.
"""
from __future__ import annotations

from typing import Iterable, List

from ..errors import InvalidPlan, OutOfPages, OutOfSlots


class Pool:
    exhausted = OutOfPages
    what = "page"

    def __init__(self, total: int):
        if total < 0:
            raise InvalidPlan(f"a pool cannot hold {total} {self.what}s")
        self.total = int(total)
        self._free: List[int] = list(range(self.total - 1, -1, -1))   # pop() gives 0 first
        self._out = set()

    @property
    def n_free(self) -> int:
        return len(self._free)

    @property
    def n_out(self) -> int:
        return len(self._out)

    def take(self, n: int = 1) -> List[int]:
        """``n`` ids, or :class:`OutOfPages`/:class:`OutOfSlots` with nothing taken."""
        if n > len(self._free):
            raise self.exhausted(f"{n} {self.what}s asked, {len(self._free)} free of {self.total}",
                                 asked=n, free=len(self._free), total=self.total)
        got = [self._free.pop() for _ in range(n)]
        self._out.update(got)
        return got

    def give_back(self, ids: Iterable[int]) -> None:
        for i in ids:
            if i not in self._out:
                raise InvalidPlan(f"{self.what} {i} is given back but is not out")
            self._out.remove(i)
            self._free.append(i)

    def check(self) -> None:
        """Every id is either free or out, none both, none twice."""
        free = set(self._free)
        assert len(free) == len(self._free), f"a {self.what} is free twice"
        assert not (free & self._out), f"a {self.what} is free and out"
        assert free | self._out == set(range(self.total)), f"a {self.what} is lost"


class PagePool(Pool):
    pass


class SlotPool(Pool):
    exhausted = OutOfSlots
    what = "slot"
