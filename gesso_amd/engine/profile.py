"""The decode stage profiler: device time per named stage of a decode step.

The reference has the same instrument behind ``GESSO_PROFILE=decode``
(``src/Inference/decode_profile.jl:1-58``): stages ``embed``, ``conv_mixer``, ``attn_mixer``, ``norm``, ``dense_ffn``,
``lm_head``, ``sample`` that are disjoint and add up to the token's time, and sub-stages nested in a stage
(``conv_in / conv_mix / conv_out``, ``attn_proj / attn_core / attn_outproj``, ``ffn_gateup / ffn_down``) that are
reported beside the table and never added to it; only decode steps are counted, never a prompt.  There a stage is
bracketed by a synchronisation of the backend; here by a pair of HIP events on the stream, read after the run, so the
device is never held up.

Off (the default) a stage site costs one attribute read.  On, the recorded decode loop runs its step eagerly
(events cannot be recorded into a graph), with the same fused kernels, so the times are those of the kernels, not
of the graph's replay: the step as a whole is slower by what the launches cost.
"""
from __future__ import annotations

from collections import OrderedDict
from typing import Dict, List, Tuple

import torch

STAGES = ("embed", "conv_mixer", "attn_mixer", "norm", "dense_ffn", "lm_head", "sample")
SUBSTAGES = ("conv_in", "conv_mix", "conv_out", "attn_proj", "attn_headnorm_rope", "attn_core", "attn_outproj",
             "ffn_gateup", "ffn_act", "ffn_down")


class _Off:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


OFF = _Off()


class _Bracket:
    __slots__ = ("profile", "name", "start")

    def __init__(self, profile, name):
        self.profile, self.name = profile, name

    def __enter__(self):
        self.start = torch.cuda.Event(enable_timing=True)
        self.start.record()
        return self

    def __exit__(self, *exc):
        end = torch.cuda.Event(enable_timing=True)
        end.record()
        self.profile._pairs.append((self.name, self.start, end))
        return False


class StageProfile:
    """Collects event pairs while a window is open; ``report()`` reads them (it waits for the device once)."""

    def __init__(self):
        self._pairs: List[Tuple[str, torch.cuda.Event, torch.cuda.Event]] = []
        self.window = False            # open only while decode steps run
        self.ms: Dict[str, float] = OrderedDict((s, 0.0) for s in STAGES + SUBSTAGES)
        self.calls: Dict[str, int] = OrderedDict((s, 0) for s in STAGES + SUBSTAGES)
        self.tokens = 0                # decode steps counted
        self.step_ms = 0.0             # their time from first to last kernel

    def bracket(self, name: str):
        if not self.window:
            return OFF
        if name not in self.ms:
            self.ms[name], self.calls[name] = 0.0, 0          # a stage of a part the framework has never seen
        return _Bracket(self, name)

    def collect(self) -> None:
        if not self._pairs:
            return
        torch.cuda.synchronize()
        for name, a, b in self._pairs:
            dt = a.elapsed_time(b)
            if name == "__step__":
                self.step_ms += dt
                self.tokens += 1
            else:
                self.ms[name] += dt
                self.calls[name] += 1
        self._pairs.clear()

    def report(self) -> dict:
        """Per decode step: milliseconds of each stage, ``other`` (the step's time that no stage covers: gaps between
        kernels), and the sub-stages beside them."""
        self.collect()
        n = max(1, self.tokens)
        stages = {s: self.ms[s] / n for s in self.ms if s not in SUBSTAGES and self.calls[s]}
        subs = {s: self.ms[s] / n for s in SUBSTAGES if self.calls[s]}
        covered = sum(stages.values())
        return {"steps": self.tokens, "step_ms": self.step_ms / n, "stages_ms": stages,
                "other_ms": max(0.0, self.step_ms / n - covered), "substages_ms": subs,
                "calls_per_step": {s: self.calls[s] / n for s in self.calls if self.calls[s]}}

    def lines(self) -> List[str]:
        r = self.report()
        out = [f"gesso_decode_profile steps={r['steps']} step_ms={r['step_ms']:.4f}"]
        for s, ms in list(r["stages_ms"].items()) + [("other", r["other_ms"])]:
            share = ms / r["step_ms"] if r["step_ms"] > 0 else 0.0
            out.append(f"gesso_decode_profile stage={s} ms={ms:.4f} share={share:.3f} "
                       f"calls={r['calls_per_step'].get(s, 0):.0f}")
        for s, ms in r["substages_ms"].items():
            out.append(f"gesso_decode_profile substage={s} ms={ms:.4f} calls={r['calls_per_step'].get(s, 0):.0f}")
        return out
