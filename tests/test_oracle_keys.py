"""Pins of the oracle's NTT-domain automorphisms, its switching keys in the T basis and its homomorphic multiply / rotate /
conjugate: substitution X -> X^g in the coefficient domain, and decrypt identities with Python integer algebra.  No GPU."""
import numpy as np
import pytest

from oracle import oracle_py as O
from tests.helpers import crt, negacyclic_mul
from tests.params import REF_PARAMS

LOGN = 5
N = 1 << LOGN
KEY = bytes(range(32))


def ref_ctx(params):
    P = REF_PARAMS[params]
    return O.OracleContext(LOGN, P["p"], P["q"], P["t"], P["gamma"])


def substitute(a, g, q):
    """a(X^g) in Z_q[X]/(X^N + 1), g odd."""
    n = len(a)
    out = [0] * n
    for i, v in enumerate(a):
        e = i * g % (2 * n)
        if e < n:
            out[e] = (out[e] + v) % q
        else:
            out[e - n] = (out[e - n] - v) % q
    return out


def test_automorphisms_are_substitutions():
    ctx = ref_ctx(14)
    K = ctx.K
    q = ctx.q[:2]
    rng = np.random.default_rng(0)
    a = np.stack([rng.integers(0, m, N, dtype=np.uint64) for m in q])
    a_ntt = np.zeros((ctx.L + 1, N), dtype=np.uint64)
    a_ntt[:2] = a
    ctx.ToNTTInplace(a_ntt.reshape(-1), 0, K, 1, 2, ctx.L + 1)
    assert ctx.rot_group(0) == 1 and ctx.rot_group(3) == 125 % (2 * N) and ctx.rot_group(N // 2) == 1       # 5 has order N/2 mod 2N
    for pow_ in (ctx.rot_group(1), ctx.rot_group(N // 2 - 3), 2 * N - 1):
        out = np.zeros((3, N), dtype=np.uint64)
        ctx.automorph_ntt(out.reshape(-1), a_ntt.reshape(-1), pow_, 1, 0, 2)
        assert not out[0].any()
        back = np.zeros((ctx.L + 1, N), dtype=np.uint64)
        back[:2] = out[1:3]
        ctx.FromNTTInplace(back.reshape(-1), 0, K, 1, 2, ctx.L + 1)
        inv = pow(pow_, -1, 2 * N)
        for j, m in enumerate(q):
            assert [int(v) for v in back[j]] == substitute([int(v) for v in a[j]], inv, m)      # out(Y^pow) = in(Y)
    out = np.zeros((2, N), dtype=np.uint64)
    ctx.conjugate_ntt(out.reshape(-1), a_ntt.reshape(-1), 0, 0, 2)
    back = np.zeros((ctx.L + 1, N), dtype=np.uint64)
    back[:2] = out
    ctx.FromNTTInplace(back.reshape(-1), 0, K, 1, 2, ctx.L + 1)
    for j, m in enumerate(q):
        assert [int(v) for v in back[j]] == substitute([int(v) for v in a[j]], 2 * N - 1, m)    # X -> X^-1


class Party:
    """Keys of one user from the oracle's own generators, and exact decryption to centred integers."""

    def __init__(self, ctx, h=8, seed=1):
        self.ctx = ctx
        K, L1 = ctx.K, ctx.L + 1
        self.K, self.L1 = K, L1
        KL = K + L1
        self.stream = O.salsa20_stream(1 << 20, KEY, seed)
        self.pos = 0
        self.sx = np.zeros((KL, N), dtype=np.uint64)
        ctx.keygen_secret(self.sx.reshape(-1), self.take(5 * h), h)
        sc = self.sx.copy()
        ctx.FromNTTInplace(sc.reshape(-1), 0, 0, 1, KL, KL)
        pq = ctx.p + ctx.q
        self.s = [int(v) if v <= 1 else int(v) - pq[0] for v in sc[0]]
        self.pk = np.zeros((2, L1, N), dtype=np.uint64)
        ctx.keygen_public(self.pk.reshape(-1), self.sx.reshape(-1), self.take(8 * N * L1), self.take(4 * N))

    def take(self, n):
        n64 = (n + 63) // 64 * 64
        out = np.ascontiguousarray(self.stream[self.pos:self.pos + n])
        self.pos += n64
        return out

    def switch_key(self, s_to, s_from):
        c = self.ctx
        swk = np.zeros((2, c.dnum, c.Ri_blockNum * c.t_num, N), dtype=np.uint64)
        KL = self.K + self.L1
        c.keygen_switch_23(swk.reshape(-1), np.ascontiguousarray(s_to).reshape(-1), np.ascontiguousarray(s_from).reshape(-1),
                           self.take(c.dnum * 8 * N * KL), self.take(c.dnum * 4 * N))
        return swk

    def encrypt(self, m, l):
        c = self.ctx
        mx = np.zeros((self.L1, N), dtype=np.uint64)
        for j in range(l + 1):
            mx[j] = [v % c.q[j] for v in m]
        c.ToNTTInplace(mx.reshape(-1), 0, self.K, 1, l + 1, self.L1)
        ct = np.zeros((2, self.L1, N), dtype=np.uint64)
        c.encrypt(ct.reshape(-1), mx.reshape(-1), self.pk.reshape(-1), self.take(9 * N), l)
        return ct

    def decrypt(self, ct, l):
        c = self.ctx
        mx = np.zeros((self.L1, N), dtype=np.uint64)
        c.decrypt(mx.reshape(-1), ct.reshape(-1), self.sx.reshape(-1), l)
        c.FromNTTInplace(mx.reshape(-1), 0, self.K, 1, l + 1, self.L1)
        out = []
        M = 1
        for x in c.q[:l + 1]:
            M *= x
        for i in range(N):
            v, _ = crt([mx[j, i] for j in range(l + 1)], c.q[:l + 1])
            out.append(v - M if v > M // 2 else v)
        return out


def int_negacyclic(a, b):
    n = len(a)
    out = [0] * n
    for i, x in enumerate(a):
        for j, y in enumerate(b):
            k = i + j
            if k < n:
                out[k] += x * y
            else:
                out[k - n] -= x * y
    return out


def int_substitute(a, g):
    n = len(a)
    out = [0] * n
    for i, v in enumerate(a):
        e = i * g % (2 * n)
        if e < n:
            out[e] += v
        else:
            out[e - n] -= v
    return out


@pytest.mark.parametrize("params", [14, 15])
def test_mult_rotate_conjugate_decrypt_to_the_right_messages(params):
    ctx = ref_ctx(params)
    K, L1 = ctx.K, ctx.L + 1
    u = Party(ctx, seed=params)
    rng = np.random.default_rng(params)
    m1 = [int(v) for v in rng.integers(-(1 << 24), 1 << 24, N)]
    m2 = [int(v) for v in rng.integers(-(1 << 24), 1 << 24, N)]
    # relinearisation key: switches s^2 to s (KeySwitch_23.cuh:34)
    sxsx = np.zeros((L1, N), dtype=np.uint64)
    ctx.poly_op(0, sxsx.reshape(-1), u.sx.reshape(-1), u.sx.reshape(-1), 0, K, K, K, L1)
    rlk = u.switch_key(u.sx, sxsx)
    for l in (ctx.L, 2):
        c1, c2 = u.encrypt(m1, l), u.encrypt(m2, l)
        out = np.zeros((2, L1, N), dtype=np.uint64)
        ctx.mult_23(out.reshape(-1), c1.reshape(-1), c2.reshape(-1), rlk.reshape(-1), l)
        got = u.decrypt(out, l)
        want = int_negacyclic(m1, m2)
        assert max(abs(v) for v in want) > 1 << 48
        assert max(abs(g - w) for g, w in zip(got, want)) < 1 << 40
    with pytest.raises(ValueError):
        ctx.mult_23(out.reshape(-1), c1.reshape(-1), c2.reshape(-1), rlk.reshape(-1), 0)
    # rotation by r slots: the key switches s to s(X^(5^-r)) (KeySwitch_23.cuh:133-134, 141, 150); result decrypts to m(X^(5^r))
    for r in (1, 5):
        s_rot = np.zeros((K + L1, N), dtype=np.uint64)
        ctx.automorph_ntt(s_rot.reshape(-1), u.sx.reshape(-1), ctx.rot_group(r), 0, 0, K + L1)
        rk = u.switch_key(s_rot, u.sx[K:])
        for l in (ctx.L, 1):
            c1 = u.encrypt(m1, l)
            out = np.zeros((2, L1, N), dtype=np.uint64)
            ctx.leftRotate_23(out.reshape(-1), c1.reshape(-1), rk.reshape(-1), r, l)
            got = u.decrypt(out, l)
            want = int_substitute(m1, pow(5, r, 2 * N))
            assert max(abs(g - w) for g, w in zip(got, want)) < 1 << 16
    # conjugation: the key switches the reversed secret to s (KeySwitch_23.cuh:83); result decrypts to m(X^-1)
    s_conj = np.zeros((L1, N), dtype=np.uint64)
    ctx.conjugate_ntt(s_conj.reshape(-1), u.sx.reshape(-1), 0, K, L1)
    ck = u.switch_key(u.sx, s_conj)
    c1 = u.encrypt(m1, ctx.L)
    out = np.zeros((2, L1, N), dtype=np.uint64)
    ctx.conjugate_23(out.reshape(-1), c1.reshape(-1), ck.reshape(-1), ctx.L)
    got = u.decrypt(out, ctx.L)
    want = int_substitute(m1, 2 * N - 1)
    assert max(abs(g - w) for g, w in zip(got, want)) < 1 << 16
