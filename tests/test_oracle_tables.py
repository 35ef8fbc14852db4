"""Pins root selection and twiddle-table generation by closed forms and an independent library (sympy)."""
import numpy as np
import pytest
import sympy

from oracle import oracle_py as O
from tests.helpers import bitrev
from tests.params import CFG1_Q, CFG2_Q, CFG3_P, REF_PARAMS


def ref_rule_primitive_root(q):
    """The reference's rule (Utils.cuh:63-96) restated independently with sympy's factorisation, INCLUDING its
    quirk: trial division stops at i < sqrt(n) on the shrinking cofactor, so a leftover prime square p^2 is kept
    as one 'factor'."""
    n = q - 1
    s = set()
    while n % 2 == 0:
        s.add(2)
        n //= 2
    i = 3
    while float(i) < float(n) ** 0.5:
        while n % i == 0:
            s.add(i)
            n //= i
        i += 1
    if n > 2:
        s.add(n)
    r = 2
    while any(pow(r, (q - 1) // f, q) == 1 for f in s):
        r += 1
    return r


@pytest.mark.parametrize("q", CFG1_Q + CFG2_Q[:6] + CFG3_P[:2] + [65537, 998244353])
def test_primitive_root_small_factor_primes(q):
    # q-1 of these primes has only small odd factors besides 2^k, so the loop is cheap in pure Python
    L = O.lib()
    g = L.orc_find_primitive_root(q)
    assert g == ref_rule_primitive_root(q)
    # for these moduli the quirk does not bite: the result is a true primitive root, and the smallest one
    assert sympy.is_primitive_root(g, q)
    assert g == sympy.primitive_root(q)


@pytest.mark.parametrize("logN,q", [(12, CFG1_Q[0]), (16, CFG2_Q[0]), (16, CFG3_P[0]), (16, REF_PARAMS[16]["q"][0]),
                                    (16, REF_PARAMS[16]["t"][0]), (13, REF_PARAMS[13]["p"][0])])
def test_psi_is_primitive_2Nth_root(logN, q):
    L = O.lib()
    N = 1 << logN
    psi = L.orc_find_mth_root(2 * N, q)
    assert pow(psi, N, q) == q - 1 and pow(psi, 2 * N, q) == 1
    g = L.orc_find_primitive_root(q)
    assert psi == pow(g, (q - 1) // (2 * N), q)


@pytest.mark.parametrize("logN,q", [(5, 65537), (10, CFG2_Q[3]), (12, CFG1_Q[1]), (12, REF_PARAMS[16]["t"][1])])
def test_psi_tables_closed_form(logN, q):
    L = O.lib()
    N = 1 << logN
    psi = L.orc_find_mth_root(2 * N, q)
    tabs = [np.zeros(N, dtype=np.uint64) for _ in range(4)]
    L.orc_fill_psi_tables(psi, q, N, *[O._ptr(t) for t in tabs])
    ps, pi, pss, pis = tabs
    ninv = pow(N, -1, q)
    for i in range(N):
        r = bitrev(i, logN)
        assert int(ps[r]) == pow(psi, i, q)
        want_inv = pow(psi, -i, q)
        if r == 1:
            want_inv = want_inv * ninv % q           # the N^-1 fold of Utils.cuh:200
        assert int(pi[r]) == want_inv
        assert int(pss[r]) == (int(ps[r]) << 64) // q
        assert int(pis[r]) == (int(pi[r]) << 64) // q
