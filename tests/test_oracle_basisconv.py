"""Pins the oracle's RNS basis conversions, ModDown, external/inner products, rescale and both key-switch chains
against exact big-integer arithmetic (Python ints) and the decryption identity."""
import numpy as np
import pytest

from oracle import oracle_py as O
from tests.helpers import crt, limbs_uniform
from tests.params import CFG2_Q, CFG3_P, REF_PARAMS

LOGN = 6
N = 1 << LOGN


def ref_ctx(logN_params=14, logN=LOGN):
    P = REF_PARAMS[logN_params]
    return O.OracleContext(logN, P["p"], P["q"], P["t"], P["gamma"])


def prod(v):
    r = 1
    for x in v:
        r *= int(x)
    return r


@pytest.mark.parametrize("params", [13, 14, 15])
def test_modup_pq_to_t_exact(params):
    ctx = ref_ctx(params)
    K, Q, T, g, RB = ctx.p_num, ctx.q_num, ctx.t_num, ctx.gamma, ctx.Ri_blockNum
    pq = ctx.p + ctx.q
    for l in {ctx.L, max(ctx.L - 2, 0)}:
        batch = 2
        inp = limbs_uniform(11 + l, pq, batch, N)                      # [batch][K+Q][N]
        out = np.zeros((batch, RB * T, N), dtype=np.uint64)
        ctx.modUpPQtoT_23(out.reshape(-1), inp.reshape(-1), l, batch)
        nblk = -(-(K + l + 1) // g)
        for b in range(batch):
            for blk in range(nblk):
                idx = [i for i in range(blk * g, blk * g + g) if i < K + l + 1]
                if len(idx) != min(g, K + Q - blk * g):
                    # The tables (Context_23.cuh:232-283) are built for whole gamma-blocks of [P | Q_L]; a
                    # block cut short by l < L is not a CRT basis for them (reference behaviour: the key
                    # generator only calls this map at l = L).  Nothing exact to compare with.
                    continue
                for x in range(0, N, 7):
                    val, R = crt([inp[b, i, x] for i in idx], [pq[i] for i in idx])
                    for k in range(T):
                        assert int(out[b, blk * T + k, x]) == val % ctx.t[k]


@pytest.mark.parametrize("params", [13, 14, 15])
def test_modup_qj_to_t_exact_and_corner(params):
    ctx = ref_ctx(params)
    K, Q, T, B = ctx.p_num, ctx.q_num, ctx.t_num, ctx.Qj_blockNum
    for l in {ctx.L, ctx.L - 1}:
        inp = limbs_uniform(21 + l, ctx.q, 1, N)
        # corner columns: value 0, 1, D-1 of every digit
        nblk = -(-(l + 1) // K)
        for blk in range(nblk):
            idx = [i for i in range(blk * K, blk * K + K) if i <= l]
            D = prod(ctx.q[i] for i in idx)
            for col, v in enumerate([0, 1, D - 1, D // 2]):
                for i in idx:
                    inp[0, i, col] = v % ctx.q[i]
        out = np.zeros((1, B * T, N), dtype=np.uint64)
        ctx.modUpQjtoT_23(out.reshape(-1), inp.reshape(-1), l, 1)
        for blk in range(nblk):
            idx = [i for i in range(blk * K, blk * K + K) if i <= l]
            for x in range(N):
                val, D = crt([inp[0, i, x] for i in idx], [ctx.q[i] for i in idx])
                for k in range(T):
                    got = int(out[0, blk * T + k, x])
                    if x < 4:   # corners: the float estimate of v may be off by one at the very ends of [0, D)
                        assert got in {(val + e * D) % ctx.t[k] for e in (-1, 0, 1)}
                    else:
                        assert got == val % ctx.t[k]


@pytest.mark.parametrize("params", [13, 14, 15])
def test_modup_t_to_pql_centred(params):
    ctx = ref_ctx(params)
    K, Q, T, g, RB = ctx.p_num, ctx.q_num, ctx.t_num, ctx.gamma, ctx.Ri_blockNum
    pq = ctx.p + ctx.q
    Tprod = prod(ctx.t)
    half = Tprod // 2
    l, batch = ctx.L - 1, 2
    nblk = -(-(K + l + 1) // g)
    # inputs: small signed integers and full-range values, written in the T basis
    rng = np.random.default_rng(5)
    vals = [[[int(rng.integers(-2 ** 62, 2 ** 62)) * (1 if x % 3 else pq[0] * pq[1]) for x in range(N)]
             for _ in range(nblk)] for _ in range(batch)]
    inp = np.zeros((batch, RB * T, N), dtype=np.uint64)
    for b in range(batch):
        for blk in range(nblk):
            for x in range(N):
                for i in range(T):
                    inp[b, blk * T + i, x] = vals[b][blk][x] % ctx.t[i]
    buf = np.zeros((batch, RB * T, N), dtype=np.uint64)
    ctx.modUpTtoPQl_23(buf.reshape(-1), inp.reshape(-1), l, batch)
    for b in range(batch):
        for blk in range(nblk):
            for j in range(g):
                ipq = blk * g + j
                if ipq >= K + l + 1:
                    continue
                for x in range(N):
                    v = vals[b][blk][x] % Tprod
                    centred = ((v + half) % Tprod) - half
                    assert centred == vals[b][blk][x]          # inputs were chosen inside (-T/2, T/2)
                    assert int(buf[b, ipq, x]) == centred % pq[ipq]


@pytest.mark.parametrize("params", [13, 14, 15])
def test_moddown_closed_form(params):
    ctx = ref_ctx(params)
    K, Q, T, RB = ctx.p_num, ctx.q_num, ctx.t_num, ctx.Ri_blockNum
    P = prod(ctx.p)
    l, batch = ctx.L, 2
    rng = np.random.default_rng(3)
    buf = np.zeros((batch, RB * T, N), dtype=np.uint64)
    m = [[int(rng.integers(0, 2 ** 62)) * int(rng.integers(0, 2 ** 62)) for _ in range(N)] for _ in range(batch)]
    e = [[int(rng.integers(0, 2 ** 62)) % P for _ in range(N)] for _ in range(batch)]
    for b in range(batch):
        for x in range(N):
            c = P * m[b][x] + e[b][x]
            for i in range(K):
                buf[b, i, x] = c % ctx.p[i]
            for i in range(l + 1):
                buf[b, K + i, x] = c % ctx.q[i]
    out = np.zeros((batch, Q, N), dtype=np.uint64)
    ctx.modDownPQltoQl_23(out.reshape(-1), buf.reshape(-1), l, batch)
    for b in range(batch):
        for x in range(N):
            # fast conversion without the v term returns e + v*P for one v in [0, K) shared by all q_i
            if K == 1:
                cands = [0]
            else:
                y = [e[b][x] % ctx.p[j] * pow(P // ctx.p[j], -1, ctx.p[j]) % ctx.p[j] for j in range(K)]
                conv = sum(y[j] * (P // ctx.p[j]) for j in range(K))
                assert (conv - e[b][x]) % P == 0
                cands = [(conv - e[b][x]) // P]
                assert 0 <= cands[0] < K
            for i in range(l + 1):
                assert int(out[b, i, x]) == (m[b][x] - cands[0]) % ctx.q[i]


def test_external_product_bruteforce():
    ctx = ref_ctx(14)
    K, Q, T, g, RB, dnum = ctx.p_num, ctx.q_num, ctx.t_num, ctx.gamma, ctx.Ri_blockNum, ctx.dnum
    l = ctx.L - 1
    cb = -(-(l + 1) // K)
    nblk = -(-(K + l + 1) // g)
    cT = limbs_uniform(1, ctx.t, ctx.Qj_blockNum, N)                    # [digit][T][N]
    swk = limbs_uniform(2, ctx.t, 2 * dnum * RB, N).reshape(2, dnum, RB, T, N)
    out = np.zeros((2, RB, T, N), dtype=np.uint64)
    ctx.external_product_T(out.reshape(-1), cT.reshape(-1), swk.reshape(-1), l)
    for z in range(2):
        for blk in range(nblk):
            for k in range(T):
                for x in range(0, N, 5):
                    want = sum(int(cT[i, k, x]) * int(swk[z, i, blk, k, x]) for i in range(cb)) % ctx.t[k]
                    assert int(out[z, blk, k, x]) == want


def test_external_product_swk_reuse_bruteforce():
    """One key against several digit sets (ExternalProduct.cuh:103-162): every output word against Python integers, with the
    reference's addressing (set stride t_num * Qj_blockNum limbs, result pair of set i at polynomials 2i, 2i + 1), and equal to
    the single-set product set by set."""
    ctx = ref_ctx(14)
    K, T, g, RB, QB, dnum = ctx.p_num, ctx.t_num, ctx.gamma, ctx.Ri_blockNum, ctx.Qj_blockNum, ctx.dnum
    for l, batch in ((ctx.L - 1, 3), (1, 8), (ctx.L, 1)):
        cb = -(-(l + 1) // K)
        nblk = -(-(K + l + 1) // g)
        cT = limbs_uniform(31 + l, ctx.t, batch * QB, N).reshape(batch, QB, T, N)
        swk = limbs_uniform(32 + l, ctx.t, 2 * dnum * RB, N).reshape(2, dnum, RB, T, N)
        out = np.zeros((batch, 2, RB, T, N), dtype=np.uint64)
        ctx.external_product_T_swk_reuse(out.reshape(-1), cT.reshape(-1), swk.reshape(-1), l, batch)
        for it in range(batch):
            one = np.zeros((2, RB, T, N), dtype=np.uint64)
            ctx.external_product_T(one.reshape(-1), np.ascontiguousarray(cT[it]).reshape(-1), swk.reshape(-1), l)
            assert np.array_equal(out[it, :, :nblk], one[:, :nblk]), (l, it)
            for z in range(2):
                for blk in range(0, nblk, 2):
                    for k in range(T):
                        for x in range(0, N, 11):
                            want = sum(int(cT[it, i, k, x]) * int(swk[z, i, blk, k, x]) for i in range(cb)) % ctx.t[k]
                            assert int(out[it, z, blk, k, x]) == want
    with pytest.raises(Exception):
        ctx.external_product_T_swk_reuse(out.reshape(-1), cT.reshape(-1), swk.reshape(-1), 1, 9)


def test_rescale_closed_form():
    ctx = ref_ctx(14, logN=5)
    n = 1 << 5
    K, L = ctx.K, ctx.L
    l = L - 1
    c = limbs_uniform(4, ctx.q, 2, n)                                    # [2][L+1][N], NTT domain
    work = c.copy().reshape(-1)
    ctx.rescaleAndEqual(work, l)
    work = work.reshape(2, L + 1, n)
    # closed form: (c_i - NTT_i([c_l]_coeff mod q_i)) * q_l^-1 mod q_i, non-centred lift of the dropped limb
    last = c[:, l:l + 1, :].copy()
    ctx.FromNTTInplace(last.reshape(-1), 0, K + l, 2, 1, 1)
    for i in range(l):
        red = np.array([[int(v) % ctx.q[i] for v in last[z, 0]] for z in range(2)], dtype=np.uint64)
        ctx.ToNTTInplace(red.reshape(-1), 0, K + i, 2, 1, 1)
        inv = pow(ctx.q[l], -1, ctx.q[i])
        for z in range(2):
            want = [(int(a) - int(b)) * inv % ctx.q[i] for a, b in zip(c[z, i], red[z])]
            assert [int(v) for v in work[z, i]] == want
    assert np.array_equal(work[:, l + 1:], c[:, l + 1:])                 # limbs above l untouched
    assert np.array_equal(work[:, l], last[:, 0])                        # dropped limb is left in coefficient form (Scheme_23.cuh:372)


# ---------------------------------------------------------------------------------------------------------
# key-switch chains: decryption identity (m = a*s + b, Scheme_23.cuh:125-126)
# ---------------------------------------------------------------------------------------------------------
def ternary(rng, n, h):
    s = np.zeros(n, dtype=np.int64)
    pos = rng.choice(n, size=h, replace=False)
    s[pos] = rng.choice([-1, 1], size=h)
    return s


def to_rns_ntt(ctx, poly_int, prime_idx_list):
    """signed integer coefficients -> NTT-domain limbs for the listed prime indices (pqt order)."""
    n = len(poly_int)
    pqt = ctx.p + ctx.q + ctx.t
    out = np.zeros((len(prime_idx_list), n), dtype=np.uint64)
    for r, pi in enumerate(prime_idx_list):
        out[r] = np.array([int(v) % pqt[pi] for v in poly_int], dtype=np.uint64)
        ctx.ToNTTInplace(out[r], 0, pi, 1, 1, 1)
    return out


def mulmod_vec(a, b, q):
    return np.array([int(x) * int(y) % q for x, y in zip(a, b)], dtype=np.uint64)


def addmod_vec(a, b, q):
    return np.array([(int(x) + int(y)) % q for x, y in zip(a, b)], dtype=np.uint64)


def centred_crt(limbs_coeff, primes):
    M = prod(primes)
    out = []
    for x in range(limbs_coeff.shape[1]):
        v, _ = crt([limbs_coeff[i, x] for i in range(len(primes))], primes)
        out.append(v - M if v > M // 2 else v)
    return out, M


def test_hybrid_keyswitch_decrypts():
    """Textbook hybrid switch over [P | Q]: KS(d) decrypts under s to d*s' + small noise."""
    logN, n = 6, 64
    q, p = CFG2_Q[:6], CFG3_P[:2]
    ctx = O.OracleContext(logN, p, q)
    K, Q = 2, 6
    W = K + Q
    dnum = Q // K
    rng = np.random.default_rng(42)
    s, s2 = ternary(rng, n, 16), ternary(rng, n, 16)
    all_idx = list(range(W))
    pq = p + q
    s_ntt, s2_ntt = to_rns_ntt(ctx, s, all_idx), to_rns_ntt(ctx, s2, all_idx)
    P = prod(p)
    evk = np.zeros((2, dnum, W, n), dtype=np.uint64)
    for d in range(dnum):
        e_ntt = to_rns_ntt(ctx, rng.integers(-8, 9, n), all_idx)
        for r in range(W):
            m = pq[r]
            a = rng.integers(0, m, n, dtype=np.uint64)
            evk[0, d, r] = a
            b = [(-int(x) * int(y)) % m for x, y in zip(a, s_ntt[r])]
            b = addmod_vec(b, e_ntt[r], m)
            if K + d * K <= r < K + (d + 1) * K:                         # P * s' on the digit's own primes
                b = addmod_vec(b, mulmod_vec(s2_ntt[r], [P % m] * n, m), m)
            evk[1, d, r] = b
    for l in (Q - 1, Q - 2):
        d_in = limbs_uniform(9 + l, q, 1, n)[0]                          # NTT-domain input polynomial
        out = np.zeros((2, Q, n), dtype=np.uint64)
        ctx.hybrid_keyswitch(out.reshape(-1), d_in.reshape(-1), evk.reshape(-1), l)
        lhs = np.zeros((l + 1, n), dtype=np.uint64)
        rhs = np.zeros((l + 1, n), dtype=np.uint64)
        for i in range(l + 1):
            m = q[i]
            lhs[i] = addmod_vec(mulmod_vec(out[0, i], s_ntt[K + i], m), out[1, i], m)
            rhs[i] = mulmod_vec(d_in[i], s2_ntt[K + i], m)
            diff = np.array([(int(a) - int(b)) % m for a, b in zip(lhs[i], rhs[i])], dtype=np.uint64)
            ctx.FromNTTInplace(diff, 0, K + i, 1, 1, 1)
            lhs[i] = diff
        noise, M = centred_crt(lhs, q[:l + 1])
        assert max(abs(v) for v in noise) < 2 ** 20, max(abs(v) for v in noise)


@pytest.mark.parametrize("params", [14, 15])
def test_keyswitch_23_decrypts(params):
    """The reference's T-basis switch (KeySwitch_23.cuh:216-231) with a key built as addMultKey_23 does
    (KeySwitch_23.cuh:37-64): KS(d) decrypts under s to d*s' + small noise."""
    logN, n = 5, 32
    ctx = ref_ctx(params, logN)
    K, Q, T, g, RB, dnum, L = ctx.p_num, ctx.q_num, ctx.t_num, ctx.gamma, ctx.Ri_blockNum, ctx.dnum, ctx.L
    W = K + Q
    pq = ctx.p + ctx.q
    rng = np.random.default_rng(params)
    s, s2 = ternary(rng, n, 8), ternary(rng, n, 8)
    all_idx = list(range(W))
    s_ntt, s2_ntt = to_rns_ntt(ctx, s, all_idx), to_rns_ntt(ctx, s2, all_idx)
    P = prod(ctx.p)
    swk = np.zeros((2, dnum, RB * T, n), dtype=np.uint64)
    for d in range(dnum):
        e_ntt = to_rns_ntt(ctx, rng.integers(-8, 9, n), all_idx)
        key_pq = np.zeros((2, W, n), dtype=np.uint64)
        for r in range(W):
            m = pq[r]
            a = rng.integers(0, m, n, dtype=np.uint64)
            b = [(-int(x) * int(y)) % m for x, y in zip(a, s_ntt[r])]
            b = addmod_vec(b, e_ntt[r], m)
            if K + d * K <= r < K + (d + 1) * K:
                b = addmod_vec(b, mulmod_vec(s2_ntt[r], [P % m] * n, m), m)
            key_pq[0, r], key_pq[1, r] = a, b
        for z in range(2):
            coeff = key_pq[z].copy()
            ctx.FromNTTInplace(coeff.reshape(-1), 0, 0, 1, W, W)
            lifted = np.zeros((RB * T, n), dtype=np.uint64)
            ctx.modUpPQtoT_23(lifted.reshape(-1), coeff.reshape(-1), L, 1)
            ctx.ToNTTInplace(lifted.reshape(-1), 0, W, RB, T, T)
            swk[z, d] = lifted
    for l in (L, L - 1, 1):
        d_in = np.zeros((Q, n), dtype=np.uint64)
        d_in[:l + 1] = limbs_uniform(l, ctx.q[:l + 1], 1, n)[0]
        out = np.zeros((2, Q, n), dtype=np.uint64)
        ctx.keyswitch_23(out.reshape(-1), d_in.reshape(-1), swk.reshape(-1), l)
        res = np.zeros((l + 1, n), dtype=np.uint64)
        for i in range(l + 1):
            m = ctx.q[i]
            lhs = addmod_vec(mulmod_vec(out[0, i], s_ntt[K + i], m), out[1, i], m)
            rhs = mulmod_vec(d_in[i], s2_ntt[K + i], m)
            diff = np.array([(int(a) - int(b)) % m for a, b in zip(lhs, rhs)], dtype=np.uint64)
            ctx.FromNTTInplace(diff, 0, K + i, 1, 1, 1)
            res[i] = diff
        noise, M = centred_crt(res, ctx.q[:l + 1])
        assert max(abs(v) for v in noise) < 2 ** 24, max(abs(v) for v in noise)


def test_hybrid_modup_exact_and_ip_bruteforce():
    logN, n = 5, 32
    q, p = CFG2_Q[:7], CFG3_P[:3]
    ctx = O.OracleContext(logN, p, q)
    K, Q = 3, 7
    W = K + Q
    pq = p + q
    for l in (6, 4):
        dn = -(-(l + 1) // K)
        inp = limbs_uniform(l, q, 1, n)[0]
        dig = np.zeros((dn, W, n), dtype=np.uint64)
        ctx.hybrid_modup(dig.reshape(-1), inp.reshape(-1), l)
        for d in range(dn):
            idx = [j for j in range(d * K, d * K + K) if j <= l]
            for x in range(n):
                val, D = crt([inp[j, x] for j in idx], [q[j] for j in idx])
                for r in range(K + l + 1):
                    assert int(dig[d, r, x]) == val % pq[r]
        dnum = -(-Q // K)
        evk = limbs_uniform(77, pq, 2 * dnum, n).reshape(2, dnum, W, n)
        out = np.zeros((2, W, n), dtype=np.uint64)
        ctx.hybrid_inner_product(out.reshape(-1), dig.reshape(-1), evk.reshape(-1), l)
        for z in range(2):
            for r in range(K + l + 1):
                for x in range(0, n, 3):
                    want = sum(int(dig[d, r, x]) * int(evk[z, d, r, x]) for d in range(dn)) % pq[r]
                    assert int(out[z, r, x]) == want
