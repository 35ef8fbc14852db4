"""Pins the oracle's NTT / iNTT: closed form, convolution theorem vs schoolbook, the reference notebook's KAT."""
import numpy as np
import pytest

from oracle import oracle_py as O
from tests.helpers import bitrev, negacyclic_mul, limbs_uniform
from tests.params import CFG1_Q, CFG2_Q, REF_PARAMS


def tables(q, logN):
    L = O.lib()
    N = 1 << logN
    psi = L.orc_find_mth_root(2 * N, q)
    tabs = [np.zeros(N, dtype=np.uint64) for _ in range(4)]
    L.orc_fill_psi_tables(psi, q, N, *[O._ptr(t) for t in tabs])
    return psi, tabs


def fwd(a, q, logN, tabs):
    a = np.array(a, dtype=np.uint64)
    O.lib().orc_ntt_limb(O._ptr(a), 1 << logN, q, O._ptr(tabs[0]))
    return a


def inv(a, q, logN, tabs):
    a = np.array(a, dtype=np.uint64)
    O.lib().orc_intt_limb(O._ptr(a), 1 << logN, q, O._ptr(tabs[1]), pow(1 << logN, -1, q))
    return a


@pytest.mark.parametrize("logN,q", [(5, 65537), (8, 65537), (10, CFG2_Q[0]), (12, CFG1_Q[0]), (10, REF_PARAMS[16]["t"][0])])
def test_closed_form_monomials(logN, q):
    """NTT(X^k) at output position j is psi^(k*(2*bitrev(j)+1)): fixes output order, root and sign conventions."""
    N = 1 << logN
    psi, tabs = tables(q, logN)
    for k in [0, 1, 2, N // 2, N - 1]:
        a = [0] * N
        a[k] = 1
        out = fwd(a, q, logN, tabs)
        want = [pow(psi, k * (2 * bitrev(j, logN) + 1), q) for j in range(N)]
        assert [int(v) for v in out] == want


@pytest.mark.parametrize("logN,q", [(5, 65537), (9, CFG2_Q[1]), (9, REF_PARAMS[15]["q"][0]), (8, REF_PARAMS[16]["t"][2])])
def test_convolution_vs_schoolbook(logN, q):
    N = 1 << logN
    rng = np.random.default_rng(logN)
    a = rng.integers(0, q, N, dtype=np.uint64)
    b = rng.integers(0, q, N, dtype=np.uint64)
    psi, tabs = tables(q, logN)
    fa, fb = fwd(a, q, logN, tabs), fwd(b, q, logN, tabs)
    prod = np.array([int(x) * int(y) % q for x, y in zip(fa, fb)], dtype=np.uint64)
    c = inv(prod, q, logN, tabs)
    want = negacyclic_mul([int(v) for v in a], [int(v) for v in b], q)
    assert [int(v) for v in c] == want
    # the oracle's own schoolbook routine (Utils.cuh:255-285) agrees with the Python one
    cc = np.zeros(N, dtype=np.uint64)
    O.lib().orc_negacyclic_mul(O._ptr(a), O._ptr(b), O._ptr(cc), N, q)
    assert [int(v) for v in cc] == want
    # round trip and linearity
    assert np.array_equal(inv(fa, q, logN, tabs), a)
    s = np.array([(int(x) + int(y)) % q for x, y in zip(a, b)], dtype=np.uint64)
    fs = fwd(s, q, logN, tabs)
    assert [int(v) for v in fs] == [(int(x) + int(y)) % q for x, y in zip(fa, fb)]


def test_notebook_kat_square(golden_nb):
    """ring_packing.ipynb cell 6: (sum i x^i)^2 in Z_65537[x]/(x^32+1) and embedded in Z_65537[x]/(x^256+1)."""
    q = golden_nb["q"]
    for logN, key, a in [(5, "cell6_square_N32", list(range(32))),
                         (8, "cell6_square_N256", [(i // 8) if i % 8 == 0 else 0 for i in range(256)])]:
        psi, tabs = tables(q, logN)
        fa = fwd(a, q, logN, tabs)
        sq = np.array([int(x) * int(x) % q for x in fa], dtype=np.uint64)
        assert [int(v) for v in inv(sq, q, logN, tabs)] == golden_nb[key]


def test_batched_entry_points_match_plain_loops():
    """The Shoup-table transforms behind orc_ntt_fwd/inv equal the plain 128-bit-remainder loops, with the
    reference's (start_poly_idx, start_mod_idx, poly_num, mod_num, poly_mod_len) addressing."""
    logN = 10
    p, q, t = [REF_PARAMS[13]["p"][0]], CFG2_Q[:4], REF_PARAMS[13]["t"][:2]
    # all of these primes are 1 mod 2^17 >= 2N
    ctx = O.OracleContext(logN, p, q, t, gamma=2)
    N = 1 << logN
    primes = p + q + t
    data = limbs_uniform(7, q, 3, N)              # 3 polys x 4 Q limbs
    buf = np.zeros((3, 6, N), dtype=np.uint64)    # poly_mod_len = 6, data at limb offset 1
    buf[:, 1:5, :] = data
    work = buf.copy()
    ctx.ToNTTInplace(work.reshape(-1), 1, 1, 3, 4, 6)     # start_poly_idx = 1 limb, start_mod_idx = K = 1
    for y in range(3):
        for j in range(4):
            psi, tabs = tables(q[j], logN)
            assert np.array_equal(work[y, 1 + j], fwd(data[y, j], q[j], logN, tabs))
    assert np.array_equal(work[:, 0], buf[:, 0]) and np.array_equal(work[:, 5], buf[:, 5])
    ctx.FromNTTInplace(work.reshape(-1), 1, 1, 3, 4, 6)
    assert np.array_equal(work, buf)
    # tables held by the context are the stand-alone ones
    pt = ctx.table("psi_table").reshape(len(primes), N)
    for i, m in enumerate(primes):
        psi, tabs = tables(m, logN)
        assert np.array_equal(pt[i], tabs[0])
    # ext variant: batch stride
    ext = limbs_uniform(9, t, 2 * 3, N).reshape(2, 3 * 2, N)      # batch 2, 3 polys x 2 T limbs
    w2 = ext.copy()
    ctx.ToNTTInplace_for_externalProduct(w2.reshape(-1), 0, 5, 3, 2, 2, 6, 2)
    for z in range(2):
        for y in range(3):
            for j in range(2):
                psi, tabs = tables(t[j], logN)
                assert np.array_equal(w2[z, y * 2 + j], fwd(ext[z, y * 2 + j], t[j], logN, tabs))
    ctx.FromNTTInplace_for_externalProduct(w2.reshape(-1), 0, 5, 3, 2, 2, 6, 2)
    assert np.array_equal(w2, ext)
