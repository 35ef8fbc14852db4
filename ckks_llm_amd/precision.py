"""PrecisionStats / GetPrecisionStats of the reference (src/ckks/include/precision.cuh:5-249): the table of
log2(1 / |decrypted - expected|) that its test programs print (minimum, maximum, mean and median precision of the real part, the
imaginary part and the L2 norm), so that a precision claim can be stated in the reference's own unit.

Two properties of the reference's routine are kept because they show in its numbers: MinDelta starts at 1 (precision.cuh:107,
179), so the maximum precision is never reported below 0 bits; and the median of an even number n of values is the mean of the
sorted values n/2 and n/2 + 1 (counting from 0; :94-101), one place above the textbook pair, except when n/2 + 1 = n."""
import math
from dataclasses import dataclass, field

import numpy as np


@dataclass
class Stats:
    Real: float = 0.0
    Imag: float = 0.0
    L2: float = 0.0


def _prec(x):
    return math.inf if x == 0 else math.log2(1.0 / x)


def deltaToPrecision(c):
    """precision.cuh:47-49"""
    return Stats(_prec(c.Real), _prec(c.Imag), _prec(c.L2))


def _median(v):
    """calcMedian (precision.cuh:69-102) on one component."""
    v = np.sort(np.asarray(v, dtype=np.float64))
    n = len(v)
    index = n // 2
    if n % 2 == 1 or index + 1 == n:
        return float(v[index])
    return float((v[index] + v[index + 1]) / 2)


def _cdf(precs, resol):
    """calcCDF (precision.cuh:51-67): for each of `resol` thresholds between the smallest and the largest precision, how many values
    lie below it."""
    s = np.sort(np.asarray(precs, dtype=np.float64))
    s = s[np.isfinite(s)]
    if len(s) == 0:
        return []
    lo, hi = s[0], s[-1]
    out = []
    for i in range(resol):
        cur = lo + i * (hi - lo) / resol
        out.append((float(cur), int(np.searchsorted(s, cur, side="left"))))
    return out


@dataclass
class PrecisionStats:
    MaxDelta: Stats = field(default_factory=Stats)
    MinDelta: Stats = field(default_factory=Stats)
    MaxPrecision: Stats = field(default_factory=Stats)
    MinPrecision: Stats = field(default_factory=Stats)
    MeanDelta: Stats = field(default_factory=Stats)
    MeanPrecision: Stats = field(default_factory=Stats)
    MedianDelta: Stats = field(default_factory=Stats)
    MedianPrecision: Stats = field(default_factory=Stats)
    RealDist: list = field(default_factory=list)
    ImagDist: list = field(default_factory=list)
    L2Dist: list = field(default_factory=list)
    cdfResol: int = 500

    def String(self):
        """The table of PrecisionStats::String (precision.cuh:29-44), character for character."""
        rows = [("MIN Prec", self.MinPrecision), ("MAX Prec", self.MaxPrecision), ("AVG Prec", self.MeanPrecision),
                ("MED Prec", self.MedianPrecision)]
        out = "\n _________________________________\n|    Log2 | REAL  | IMAG  | L2    |\n"
        for name, s in rows:
            out += "|%s | %.2f | %.2f | %.2f |\n" % (name, s.Real, s.Imag, s.L2)
        return out + "===================================\n"

    __str__ = String


def GetPrecisionStats(valuesTest, valuesWant):
    """precision.cuh:104-174 for complex vectors, :178-249 for real ones (imaginary deltas are zero there, so the IMAG column reads
    inf, as the reference prints it)."""
    t = np.asarray(valuesTest)
    w = np.asarray(valuesWant)
    if t.shape != w.shape or t.ndim != 1 or len(w) == 0:
        raise ValueError("GetPrecisionStats: two vectors of the same positive length")
    if np.iscomplexobj(t) or np.iscomplexobj(w):
        d_re = np.abs(t.real - w.real).astype(np.float64)
        d_im = np.abs(t.imag - w.imag).astype(np.float64)
        d_l2 = np.sqrt(d_re * d_re + d_im * d_im)
    else:
        d_re = np.abs(t.astype(np.float64) - w.astype(np.float64))
        d_im = np.zeros_like(d_re)
        d_l2 = np.sqrt(d_re * d_re)
    p = PrecisionStats()
    p.MaxDelta = Stats(max(0.0, float(d_re.max())), max(0.0, float(d_im.max())), max(0.0, float(d_l2.max())))
    p.MinDelta = Stats(min(1.0, float(d_re.min())), min(1.0, float(d_im.min())), min(1.0, float(d_l2.min())))
    p.MeanDelta = Stats(float(d_re.sum() / len(w)), float(d_im.sum() / len(w)), float(d_l2.sum() / len(w)))
    with np.errstate(divide="ignore"):
        p.RealDist = _cdf(np.log2(1.0 / d_re), p.cdfResol)
        p.ImagDist = _cdf(np.log2(1.0 / d_im), p.cdfResol)
        p.L2Dist = _cdf(np.log2(1.0 / d_l2), p.cdfResol)
    p.MinPrecision = deltaToPrecision(p.MaxDelta)
    p.MaxPrecision = deltaToPrecision(p.MinDelta)
    p.MeanPrecision = deltaToPrecision(p.MeanDelta)
    p.MedianDelta = Stats(_median(d_re), _median(d_im), _median(d_l2))
    p.MedianPrecision = deltaToPrecision(p.MedianDelta)
    return p
