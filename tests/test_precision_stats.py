"""GetPrecisionStats (the reference's precision.cuh:104-249) restated in the host mirror: hand-worked values, including the two
properties of the reference's routine that show in its numbers (the minimum delta starts at 1; the median of an even count is
taken one place above the textbook pair)."""
import math

import numpy as np
import pytest

from ckks_llm_amd.precision import GetPrecisionStats


def test_real_vectors_hand_worked():
    want = np.array([1.0, 2.0, 3.0, 4.0, 5.0])
    got = want + np.array([2.0 ** -10, -2.0 ** -12, 2.0 ** -8, 2.0 ** -20, -2.0 ** -16])
    p = GetPrecisionStats(got, want)
    assert p.MinPrecision.Real == 8 and p.MaxPrecision.Real == 20          # worst and best coefficient
    assert p.MedianPrecision.Real == 12                                     # sorted deltas 2^-20, -16, -12, -10, -8: the middle one
    mean = (2.0 ** -10 + 2.0 ** -12 + 2.0 ** -8 + 2.0 ** -20 + 2.0 ** -16) / 5
    assert p.MeanPrecision.Real == pytest.approx(math.log2(1 / mean), abs=1e-12)
    assert p.MinPrecision.L2 == 8 and math.isinf(p.MinPrecision.Imag)       # real input: no imaginary error (precision.cuh:196)
    text = p.String()
    assert "|MIN Prec | 8.00 | inf | 8.00 |" in text and "|MAX Prec | 20.00 | inf | 20.00 |" in text
    assert text.startswith("\n _________________________________\n|    Log2 | REAL  | IMAG  | L2    |\n")


def test_even_count_median_follows_the_reference():
    want = np.zeros(4)
    got = np.array([2.0 ** -4, 2.0 ** -3, 2.0 ** -2, 2.0 ** -1])
    p = GetPrecisionStats(got, want)
    # precision.cuh:94-101: index = n/2 = 2; mean of sorted[2] and sorted[3], not of sorted[1] and sorted[2]
    assert p.MedianDelta.Real == (2.0 ** -2 + 2.0 ** -1) / 2
    p2 = GetPrecisionStats(np.array([0.25, 0.5]), np.zeros(2))              # n = 2: index + 1 == n, the upper value alone
    assert p2.MedianDelta.Real == 0.5


def test_max_precision_is_capped_by_the_initial_minimum():
    p = GetPrecisionStats(np.array([3.0, 5.0]), np.array([0.0, 0.0]))      # every delta above 1
    assert p.MinDelta.Real == 1.0 and p.MaxPrecision.Real == 0.0           # precision.cuh:107: MinDelta starts at {1, 1, 1}
    assert p.MinPrecision.Real == pytest.approx(-math.log2(5.0))


def test_complex_vectors():
    want = np.array([1 + 1j, 2 - 1j, -3 + 0.5j])
    got = want + np.array([2.0 ** -9 + 2.0 ** -11 * 1j, -2.0 ** -13, 2.0 ** -7 * 1j])
    p = GetPrecisionStats(got, want)
    assert p.MinPrecision.Real == 9 and p.MinPrecision.Imag == 7
    assert p.MinPrecision.L2 == 7
    l2 = math.hypot(2.0 ** -9, 2.0 ** -11)
    assert p.MedianDelta.L2 == pytest.approx(sorted([l2, 2.0 ** -13, 2.0 ** -7])[1])
    assert len(p.RealDist) == 500 and p.RealDist[0][1] == 0
    with pytest.raises(ValueError):
        GetPrecisionStats(np.zeros(3), np.zeros(4))
