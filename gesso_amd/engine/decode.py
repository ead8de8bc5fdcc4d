"""The decode loop: every live request gets one token per step, the token chosen is fed back.

``DecodeLoop(engine, rids, first_tokens)`` continues requests whose prompts are in the cache;
``run(n)`` makes ``n`` steps and returns the tokens ``(n, batch)`` it chose.  Greedy choice
runs on the device; the tokens come to the host once per call, not once per step.
"""
from __future__ import annotations

from typing import Hashable, List, Sequence

import torch

from .batch import StepEntry


class DecodeLoop:
    def __init__(self, engine, rids: Sequence[Hashable], first_tokens: Sequence[int]):
        self.engine = engine
        self.rids = list(rids)
        self.tokens = [int(t) for t in first_tokens]

    def run(self, n: int) -> List[List[int]]:
        out = []
        ops = self.engine.rt.ops
        for _ in range(n):
            logits = self.engine.step([StepEntry(r, [t], [0]) for r, t in zip(self.rids, self.tokens)])
            ids, _ = ops.argmax_rows(logits)
            self.tokens = ids.tolist()
            out.append(self.tokens)
        return out

    def close(self) -> None:
        pass
