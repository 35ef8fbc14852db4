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


def plaintext_T(ctx, poly):
    """A small integer polynomial as a PlaintextT: its residues modulo the T primes, NTT domain, t_num limbs."""
    T = ctx.t_num
    buf = np.zeros((T, N), dtype=np.uint64)
    for k, t in enumerate(ctx.t):
        buf[k] = [v % t for v in poly]
    ctx.ToNTTInplace(buf.reshape(-1), 0, ctx.K + ctx.L + 1, 1, T, T)
    return buf


def rotation_key(ctx, u, r):
    s_rot = np.zeros((ctx.K + ctx.L + 1, N), dtype=np.uint64)
    ctx.automorph_ntt(s_rot.reshape(-1), u.sx.reshape(-1), ctx.rot_group(r), 0, 0, ctx.K + ctx.L + 1)
    return u.switch_key(s_rot, u.sx[ctx.K:])


def t_basis_inputs(ctx, ct_coeff, l):
    """What a level of the slot <-> coefficient transforms feeds its hoisted kernels (Bootstrapping_C2S_S2C_impl.cuh:262-272):
    the digits of a in T (NTT) and P * (a, b) in T (NTT)."""
    K, L, T, RB = ctx.K, ctx.L, ctx.t_num, ctx.Ri_blockNum
    up = np.zeros((ctx.Qj_blockNum, T, N), dtype=np.uint64)
    ctx.modUpQjtoT_23(up.reshape(-1), ct_coeff.reshape(-1), l, 1)
    ctx.ToNTTInplace(up.reshape(-1), 0, K + L + 1, -(-(l + 1) // K), T, T)
    pq = np.zeros((2, K + L + 1, N), dtype=np.uint64)
    ctx.cipher_mul_P(pq.reshape(-1), ct_coeff.reshape(-1), l)
    pqT = np.zeros((2, RB, T, N), dtype=np.uint64)
    ctx.modUpPQtoT_23(pqT.reshape(-1), pq.reshape(-1), l, 2)
    ctx.ToNTTInplace_for_externalProduct(pqT.reshape(-1), 0, K + L + 1, -(-(K + l + 1) // ctx.gamma), T, T, RB * T, 2)
    return up, pq, pqT


@pytest.mark.parametrize("params,l", [(14, None), (15, 2)])
def test_hoisted_rotation_kernels_equal_their_pinned_parts(params, l):
    """Giant_Rotate_And_Mult_PlaintT and Baby_Rotate against a composition of functions pinned elsewhere: external product, the
    NTT-domain automorphism in its scatter form with the inverse exponent, pointwise products and sums modulo the T primes."""
    ctx = ref_ctx(params)
    l = ctx.L if l is None else l
    K, L, T, RB = ctx.K, ctx.L, ctx.t_num, ctx.Ri_blockNum
    blockNum = -(-(K + l + 1) // ctx.gamma)
    u = Party(ctx, seed=40 + params)
    rng = np.random.default_rng(params)
    ct = u.encrypt([int(v) for v in rng.integers(-(1 << 20), 1 << 20, N)], l)
    ctx.FromNTTInplace(ct.reshape(-1), 0, K, 2, l + 1, L + 1)
    up, pq, pqT = t_basis_inputs(ctx, ct, l)
    # cipher_mul_P: special limbs zero, limb K + i = c_i * P mod q_i
    Pprod = 1
    for p in ctx.p:
        Pprod *= p
    assert not pq[:, :K].any()
    for z in range(2):
        for i in range(l + 1):
            assert [int(v) for v in pq[z, K + i]] == [int(v) * Pprod % ctx.q[i] for v in ct[z, i]]
    gs, bs = 3, 2
    slots = [0, 1, 5]
    keys = [None, rotation_key(ctx, u, 1), rotation_key(ctx, u, 5)]
    plains = [[plaintext_T(ctx, [int(v) for v in rng.integers(-3, 4, N)]) for _ in range(gs)] for _ in range(bs)]
    accNum = [3, 2]                                                  # the second baby step has no third plaintext
    flat = [plains[i][j] if j < accNum[i] else None for i in range(bs) for j in range(gs)]
    got = np.full((bs, 2, RB, T, N), 7, dtype=np.uint64)
    ctx.Giant_Rotate_And_Mult_PlaintT(got.reshape(-1), pqT.reshape(-1), up.reshape(-1), [k.reshape(-1) if k is not None else None for k in keys],
                                      [s if s else -1 for s in slots], [p.reshape(-1) if p is not None else None for p in flat], accNum, bs, gs, l)
    tq = ctx.t

    def rotated_pair(j):
        if keys[j] is None:
            return pqT.copy()
        ext = np.zeros((2, RB, T, N), dtype=np.uint64)
        ctx.external_product_T(ext.reshape(-1), up.reshape(-1), keys[j].reshape(-1), l)
        for blk in range(blockNum):
            for k in range(T):
                ext[1, blk, k] = (ext[1, blk, k] + pqT[1, blk, k]) % np.uint64(tq[k])
        out = np.zeros_like(ext)
        inv = ctx.rot_group(N // 2 - slots[j])                      # gather with 5^r = scatter with 5^-r
        for z in range(2):
            for blk in range(blockNum):
                ctx.automorph_ntt(out[z, blk].reshape(-1), ext[z, blk].reshape(-1), inv, 0, 0, T)
        return out

    pairs = [rotated_pair(j) for j in range(gs)]
    for i in range(bs):
        for z in range(2):
            for blk in range(RB):
                for k in range(T):
                    if blk >= blockNum:
                        assert (got[i, z, blk, k] == 7).all()       # blocks beyond the level's are left alone
                        continue
                    want = [sum(int(pairs[j][z, blk, k, x]) * int(plains[i][j][k, x]) for j in range(accNum[i])) % tq[k] for x in range(N)]
                    assert [int(v) for v in got[i, z, blk, k]] == want
    # Baby_Rotate adds the rotated pair (with a plaintext of all ones the giant step yields exactly that pair)
    acc = got[0].copy()
    before = acc.copy()
    ctx.Baby_Rotate(acc.reshape(-1), up.reshape(-1), pqT.reshape(-1), [keys[2].reshape(-1), None], [5, -1], l)
    for z in range(2):
        for blk in range(blockNum):
            for k in range(T):
                want = (before[z, blk, k].astype(object) + pairs[2][z, blk, k].astype(object)) % tq[k]
                assert [int(v) for v in acc[z, blk, k]] == [int(v) for v in want]
    # cipher_add_T and the coefficient-domain rescale
    a, b = got[0].copy(), got[1].copy()
    ctx.cipher_add_T(a.reshape(-1), b.reshape(-1), 2 * RB)
    for k in range(T):
        assert ((got[0][:, :, k].astype(object) + got[1][:, :, k].astype(object)) % tq[k] == a[:, :, k].astype(object)).all()
    res = ct.copy()
    ctx.rescaleAndEqual_noNTT(res.reshape(-1), l)
    for z in range(2):
        for i in range(l):
            ql_inv = pow(ctx.q[l], -1, ctx.q[i])
            assert [int(v) for v in res[z, i]] == [(int(x) - int(y)) * ql_inv % ctx.q[i] for x, y in zip(ct[z, i], ct[z, l])]
        assert (res[z, l] == ct[z, l]).all()


@pytest.mark.parametrize("params,l", [(14, None), (15, 1)])
def test_bsgs_level_decrypts_to_the_transformed_message(params, l):
    """One level of EvalCoeffsToSlots / EvalSlotsToCoeffs: the result decrypts to sum_i rho_i( sum_j p_ij * sigma_j(m) ), with
    sigma_j, rho_i the substitutions X -> X^(5^r) of the inner and outer rotations, in exact integer algebra."""
    ctx = ref_ctx(params)
    l = ctx.L if l is None else l
    K, L = ctx.K, ctx.L
    u = Party(ctx, seed=60 + params)
    rng = np.random.default_rng(100 + params)
    m = [int(v) for v in rng.integers(-(1 << 20), 1 << 20, N)]
    gs, bs = 3, 3
    rot_in, rot_out = [0, 1, 2], [0, 3, 0]                           # rot_out[0] is never used; the third baby step is added unrotated
    keyring = {r: rotation_key(ctx, u, r) for r in (1, 2, 3)}
    polys = [[[int(v) for v in rng.integers(-2, 3, N)] for _ in range(gs)] for _ in range(bs)]
    accNum = [3, 3, 2]
    flat = [plaintext_T(ctx, polys[i][j]).reshape(-1) if j < accNum[i] else None for i in range(bs) for j in range(gs)]
    ct = u.encrypt(m, l)
    m_in = u.decrypt(ct, l)                                          # message plus the encryption noise: what the transform acts on
    ctx.FromNTTInplace(ct.reshape(-1), 0, K, 2, l + 1, L + 1)
    ctx.bsgs_level_23(ct.reshape(-1), l, flat, accNum, rot_in, [keyring[r].reshape(-1) if r else None for r in rot_in], rot_out,
                      [keyring[r].reshape(-1) if r else None for r in rot_out], bs, gs)
    ctx.ToNTTInplace(ct.reshape(-1), 0, K, 2, l + 1, L + 1)
    got = u.decrypt(ct, l)
    want = [0] * N
    for i in range(bs):
        inner = [0] * N
        for j in range(accNum[i]):
            term = int_negacyclic(polys[i][j], int_substitute(m_in, pow(5, rot_in[j], 2 * N)))
            inner = [a + b for a, b in zip(inner, term)]
        if i and rot_out[i]:
            inner = int_substitute(inner, pow(5, rot_out[i], 2 * N))
        want = [a + b for a, b in zip(want, inner)]
    assert max(abs(v) for v in want) > 1 << 22
    assert max(abs(g - w) for g, w in zip(got, want)) < 1 << 16
