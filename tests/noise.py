"""What a bfloat16 pipeline is held to: the distance the plain model itself takes when its activations are rounded.

A fixed tolerance on bfloat16 logits is either too wide to see a fault or narrower than the rounding noise of any
honest pipeline, depending on how large the weights are drawn.  So the bound is made from the model at hand: the
plain implementation with nothing but roundings to bfloat16 put in where a pipeline with bfloat16 activations stores
one (``plain_lfm2.forward(..., store=to_bfloat16)``, "the rounded model") stands at some distance from the plain
model, and the engine may stand as far, by these measures:

* each row: rms(engine - plain) <= ``row`` x rms(rounded - plain) of the same row;
* all rows together: rms <= ``all_rows`` x the rounded model's;
* the worst logit: <= ``worst`` x the rounded model's worst.

How the factors for the tiny configurations were set.  The engine's roundings fall independently of the rounded
model's (it fuses, sums in other orders, rounds at a few other places), so each measure is a ratio of two independent
draws of one noise, and how far such a ratio strays is a matter of how many independent numbers a draw hangs on.  A row
of a few hundred logits hangs on one hidden vector of 64 to 144 numbers, of which a dozen carry most of the error: over
the 80 rows of a recorded decode run of the engine the ratio's median was 0.88, its 95th percentile 1.6 and its largest
value 2.06 (at the row whose rounded-model distance was the smallest of all), which is what the root of an F ratio
with 12 and 12 degrees of freedom does; two computations of the rounded model itself (float32 against float64
arithmetic) are no guide here, their roundings agree too often (ratios up to 1.56 only).  With 12 degrees of freedom a
row, and a chance of one in 100,000 that an honest pipeline is refused by a measure:

* a row: 4.0 (the ratio passes 4.15 once in 100,000 rows);
* all ``n`` rows together: ``sqrt(F(1e-5; 12 n, 12 n))``, at least 1.15: 1.76 for 5 rows, 1.22 for 40, 1.15 from 80 on;
* the worst logit, where at least 32 rows are compared (the largest of thousands of logits is steady, that of a few
  rows is one row's luck): 1.5.

The tests of ``tests/test_sensitivity.py`` plant three faults in the rounded model (the convolution's history lost at
every seventh token, its taps reversed, one key past the causal edge seen); the mildest stands 5 times, most stand 10
to 90 times further off over all rows than the rounded model, and each breaks the bound without a GPU.  At the layer
sizes of LFM2-1.2B rows are 65,536 logits wide on 2,048 numbers and scatter far less; ``test_gpu_sizes.py`` keeps its
narrower factors.
"""
import numpy as np

ROW, ALL_ROWS, WORST = 4.0, 1.15, 1.5
ROW_DOF, CHANCE, WORST_FROM_ROWS = 12, 1e-5, 32


class NoiseBound:
    """Collects rows of the engine beside the plain and the rounded model's; ``failures()`` says what lies outside."""

    def __init__(self, row=ROW, all_rows=ALL_ROWS, worst=WORST, independent=None):
        """``independent``: how many of the rows count as independent draws where that is fewer than all of them (rows
        at neighbouring positions of one long context share almost all of what their errors come from)."""
        self.f_row, self.f_all_least, self.f_worst = row, all_rows, worst
        self.rows, self.independent = 0, independent
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
        self.rows += 1
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

    @property
    def f_all(self):
        """The bound on all rows together: wider while few rows are compared."""
        from scipy import stats
        k = ROW_DOF * max(1, min(self.rows, self.independent or self.rows))
        return max(self.f_all_least, float(np.sqrt(stats.f.isf(CHANCE, k, k))))

    def failures(self):
        out = []
        if self.n == 0 and self.worst == 0.0:
            return ["no row was compared"]
        if not self.row_ratio <= self.f_row:
            out.append(f"a row's rms is {self.row_ratio:.2f} x the rounded model's (bound {self.f_row}): first look at "
                       f"{self.row_where}")
        if not self.rms <= self.f_all * self.noise_rms:
            out.append(f"rms over all rows {self.rms:.3e} against the rounded model's {self.noise_rms:.3e} "
                       f"(bound {self.f_all:.2f} x for {self.rows} rows"
                       + (f", {self.independent} of them independent)" if self.independent else ")"))
        few = min(self.rows, self.independent or self.rows) < WORST_FROM_ROWS
        if not (self.worst <= self.f_worst * self.nworst or (few and np.isfinite(self.worst))):
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
