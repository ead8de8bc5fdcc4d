"""What a bfloat16 pipeline is held to: the distance the plain model itself takes when its activations are rounded.

A fixed tolerance on bfloat16 logits is either too wide to see a fault or narrower than the rounding noise of any
honest pipeline, depending on how large the weights are drawn.  So the bound is made from the model at hand: the
plain implementation with nothing but roundings to bfloat16 put in where a pipeline with bfloat16 activations stores
one (``plain_lfm2.forward(..., store=to_bfloat16)``, "the rounded model") stands at some distance from the plain
model, and the engine may stand as far, by these measures:

* each row: rms(engine - plain) <= ``row`` x rms(rounded - plain) of the same row;
* all rows together: rms <= ``all_rows`` x the rounded model's;
* the worst logit: <= ``worst`` x the rounded model's worst.

The factors for the tiny configurations were set on the CPU from two computations of the rounded model that round
alike and differ in the seventh digit before (float32 against float64 arithmetic; roundings then fall differently
here and there, and a few stages later independently): over the tiny configurations a row's ratio reached 1.56 (rows
of a few hundred logits that all hang on one hidden vector of 64 to 144 numbers scatter that much), all rows together
lay within 0.99 .. 1.01, the worst logit within 0.70 .. 1.06.  The same tests plant three faults in the rounded model
(the convolution's history lost at every seventh token, its taps reversed, one key past the causal edge seen); the
mildest of them stands 5 times, most stand 10 to 90 times further off over all rows than the rounded model, so each
breaks the bound (``tests/test_sensitivity.py`` asserts that, without a GPU).  At the layer sizes of LFM2-1.2B rows are
65,536 logits wide and scatter less; ``test_gpu_sizes.py`` keeps its narrower factors.
"""
import numpy as np

ROW, ALL_ROWS, WORST = 2.0, 1.15, 1.5


class NoiseBound:
    """Collects rows of the engine beside the plain and the rounded model's; ``failures()`` says what lies outside."""

    def __init__(self, row=ROW, all_rows=ALL_ROWS, worst=WORST):
        self.f_row, self.f_all, self.f_worst = row, all_rows, worst
        self.sq = self.nsq = 0.0
        self.n = 0
        self.worst = self.nworst = 0.0
        self.where = None
        self.row_ratio, self.row_where = 0.0, None

    def add(self, got, ref, rounded, where=None):
        got, ref, rounded = (np.asarray(x, dtype=np.float64).reshape(-1) for x in (got, ref, rounded))
        d, e = got - ref, rounded - ref
        if not np.isfinite(d).all():
            self.worst, self.where, self.row_ratio, self.row_where = float("inf"), where, float("inf"), where
            return
        self.sq += float((d * d).sum())
        self.nsq += float((e * e).sum())
        self.n += d.size
        m = float(np.abs(d).max())
        if m > self.worst:
            self.worst, self.where = m, where
        self.nworst = max(self.nworst, float(np.abs(e).max()))
        mine, theirs = float(np.sqrt((d * d).mean())), float(np.sqrt((e * e).mean()))
        ratio = mine / theirs if theirs > 0 else (0.0 if mine == 0 else float("inf"))
        if ratio > self.row_ratio:
            self.row_ratio, self.row_where = ratio, where

    @property
    def rms(self):
        return (self.sq / max(1, self.n)) ** 0.5

    @property
    def noise_rms(self):
        return (self.nsq / max(1, self.n)) ** 0.5

    def failures(self):
        out = []
        if self.n == 0 and self.worst == 0.0:
            return ["no row was compared"]
        if not self.row_ratio <= self.f_row:
            out.append(f"a row's rms is {self.row_ratio:.2f} x the rounded model's (bound {self.f_row}): first look at "
                       f"{self.row_where}")
        if not self.rms <= self.f_all * self.noise_rms:
            out.append(f"rms over all rows {self.rms:.3e} against the rounded model's {self.noise_rms:.3e} "
                       f"(bound {self.f_all} x)")
        if not self.worst <= self.f_worst * self.nworst:
            out.append(f"worst logit {self.worst:.3e} at {self.where} against the rounded model's {self.nworst:.3e} "
                       f"(bound {self.f_worst} x)")
        return out

    def summary(self):
        return (f"against the plain model rms {self.rms:.3e}, worst {self.worst:.3e} at {self.where}; the rounded plain "
                f"model: rms {self.noise_rms:.3e}, worst {self.nworst:.3e}; largest ratio of a row's rms "
                f"{self.row_ratio:.2f} at {self.row_where}")

    def check(self, label=""):
        print(f"{label} bfloat16: {self.summary()}")
        bad = self.failures()
        assert not bad, f"{label}: " + "; ".join(bad)


def supported(row_plain, token: int, slack: float) -> bool:
    """Whether ``token`` is the plain row's best, or within ``slack`` of it: a pipeline whose logits stand at most
    ``slack / 2`` from the plain ones can choose no other token."""
    row = np.asarray(row_plain, dtype=np.float64)
    return float(row.max() - row[token]) <= slack
