"""Pins of the oracle's client-side functions (random stream, samplers, pointwise arithmetic, keys, encryption, coefficient
encoding) against known answers and against what the mathematics fixes.  No GPU."""
from fractions import Fraction

import numpy as np
import pytest

from oracle import oracle_py as O
from tests.helpers import negacyclic_mul
from tests.params import CFG2_Q, CFG3_P, REF_PARAMS

Q3 = CFG2_Q[:3]
P1 = CFG3_P[:1]


# ---- Salsa20/20 stream (RNG.cuh:18-56, RNG_impl.cuh:72-176) ----
def test_salsa20_ecrypt_vectors():
    """ECRYPT stream-cipher project, Salsa20 verified.test-vectors, 256-bit keys: set 1 vector 0 (key 80 00.., IV 0) at stream offsets
    0, 192, 256, 448 (block counters 0, 3, 4, 7) and set 5 vector 0 (key 0, IV 80 00..) at offset 0 (nonce in words 6-7, low byte first)."""
    s = bytes(O.salsa20_stream(512, bytes([0x80] + [0] * 31), 0)).hex().upper()
    assert s[0:128] == ("E3BE8FDD8BECA2E3EA8EF9475B29A6E7003951E1097A5C38D23B7A5FAD9F6844"
                        "B22C97559E2723C7CBBD3FE4FC8D9A0744652A83E72A9C461876AF4D7EF1A117")
    assert s[384:512] == ("57BE81F47B17D9AE7C4FF15429A73E10ACF250ED3A90A93C711308A74C6216A9"
                          "ED84CD126DA7F28E8ABF8BB63517E1CA98E712F4FB2E1A6AED9FDC73291FAA17")
    assert s[512:640] == ("958211C4BA2EBD5838C635EDB81F513A91A294E194F1C039AEEC657DCE40AA7E"
                          "7C0AF57CACEFA40C9F14B71A4B3456A63E162EC7D8D10B8FFB1810D71001B618")
    assert s[896:1024] == ("696AFCFD0CDDCC83C7E77F11A649D79ACDC3354E9635FF137E929933A0BD6F53"
                           "77EFA105A3A4266B7C0D089D08F1E855CC32B15B93784A36E56A76CC64BC8477")
    t = bytes(O.salsa20_stream(64, bytes(32), 0x80)).hex().upper()
    assert t[:64] == "2ABA3DC45B4947007B14C851CD694456B303AD59A465662803006705673D6C3E"
    # a partial last block is the prefix of the full one
    assert bytes(O.salsa20_stream(100, bytes([0x80] + [0] * 31), 0)).hex().upper() == s[:200]


# ---- discrete Gaussian (Sampler_impl.cuh:27-70) ----
def test_gaussian_steps_against_scipy_normal_tail():
    from scipy.stats import norm
    thr = [int(v) for v in O.gauss_thresholds()]
    assert thr == sorted(thr) and len(set(thr)) == 19
    for k in range(1, 20):
        # value >= k  <=>  (u + 0.5) / 2^32 >= Phi(k / 3.2): the threshold is the first word on or above the step
        step = 2 ** 32 * (1 - norm.sf(k / 3.2)) - 0.5
        assert abs(thr[k - 1] - step) <= 1.0 and thr[k - 1] >= step - 1e-3, (k, thr[k - 1], step)
        # the same in the tail, where 1 - Phi loses nothing: 2^32 - thr = round(2^32 * Q(k / 3.2))
        assert abs((2 ** 32 - thr[k - 1]) - 2 ** 32 * norm.sf(k / 3.2)) <= 0.5 + 1e-6


def test_gaussian_sampler_words_symmetry_and_moments():
    ctx = O.OracleContext(8, P1, Q3)
    N = ctx.N
    thr = [int(v) for v in O.gauss_thresholds()]
    words = np.zeros(N, dtype=np.uint32)
    special = [0, 2 ** 32 - 1, 2 ** 31, 2 ** 31 - 1, thr[0], thr[0] - 1, thr[4], thr[4] - 1, 2 ** 32 - 1 - thr[0], 2 ** 32 - thr[0]]
    expect = [-19, 19, 0, 0, 1, 0, 5, 4, -1, 0]
    words[: len(special)] = special
    rng = np.random.default_rng(5)
    words[len(special):] = rng.integers(0, 2 ** 32, N - len(special), dtype=np.uint32)
    out = np.zeros((4, N), dtype=np.uint64)
    ctx.gaussianSampler_xq(words.view(np.uint8), out.reshape(-1), 1, 1, 3)              # limbs 1..3 <- primes q0..q2
    assert not out[0].any()
    signed = []
    for t, q in enumerate(Q3):
        v = out[1 + t].astype(object)
        signed.append([int(x) if x <= q // 2 else int(x) - q for x in v])
    assert signed[0] == signed[1] == signed[2]                                          # one noise value, reduced per prime
    assert signed[0][: len(special)] == expect
    # mirror words give mirrored values
    out2 = np.zeros((1, N), dtype=np.uint64)
    ctx.gaussianSampler_xq((~words).view(np.uint8), out2.reshape(-1), 0, 1, 1)
    s2 = [int(x) if x <= Q3[0] // 2 else int(x) - Q3[0] for x in out2[0].astype(object)]
    assert s2 == [-x for x in signed[0]]
    # moments on a long stream: trunc(3.2 * Z) has mean 0 and variance sum k^2 P(k)
    from scipy.stats import norm
    var = 2 * sum(k * k * (norm.sf(k / 3.2) - norm.sf((k + 1) / 3.2)) for k in range(1, 19))
    big = O.OracleContext(14, P1, Q3[:1])
    stream = O.salsa20_stream(4 * big.N, bytes(range(32)), 7)
    o = np.zeros(big.N, dtype=np.uint64)
    big.gaussianSampler_xq(stream, o, 0, 1, 1)
    x = np.where(o > Q3[0] // 2, o.astype(np.int64) - Q3[0], o.astype(np.int64)).astype(np.float64)
    assert abs(x.mean()) < 4 * np.sqrt(var / big.N)
    assert abs(x.var() - var) < 0.08 * var
    assert np.abs(x).max() <= 19


# ---- uniform, ZO, HWT (Sampler_impl.cuh:13-24, 74-113) ----
def test_uniform_sampler_is_the_reference_float_map():
    ctx = O.OracleContext(8, P1, Q3)
    N = ctx.N
    rng = np.random.default_rng(11)
    w = rng.integers(0, 2 ** 64, (2, N), dtype=np.uint64)
    w[0, :4] = [0, 2 ** 64 - 1, 2 ** 63, 1]
    out = np.zeros((3, N), dtype=np.uint64)
    ctx.uniformSampler_xq(w.view(np.uint8).reshape(-1), out.reshape(-1), 1, 2, 2)       # primes 2, 3 = q1, q2 -> limbs 1, 2
    for t, q in enumerate(Q3[1:3]):
        want = [int(float(int(x)) / 2.0 ** 64 * float(q - 1)) for x in w[t]]
        assert [int(v) for v in out[1 + t]] == want
        assert int(out[1 + t].max()) < q
    assert [int(v) for v in out[1, :4]] == [0, Q3[1] - 1, (Q3[1] - 1) // 2, 0]
    assert not out[0].any()


def test_zo_and_hwt_samplers():
    ctx = O.OracleContext(8, P1, Q3)
    N = ctx.N
    b = np.arange(N, dtype=np.uint8)                                                    # N = 256: every byte value once
    out = np.zeros((2, N), dtype=np.uint64)
    ctx.ZOSampler(b, out.reshape(-1), 0.5, 0, 1, 2)
    for t, q in enumerate(Q3[:2]):
        assert not out[t, :128].any() and (out[t, 128:192] == 1).all() and (out[t, 192:] == q - 1).all()
    # HWT: h words then h bytes; positions from the low logN bits, sign 1 for bytes >= 128; the later word wins a collision
    h = 6
    pos = np.array([5, 300, 17, 5 + 256, 255, 17 + 512], dtype=np.uint32)               # -> 5, 44, 17, 5, 255, 17
    sign = np.array([200, 3, 128, 127, 255, 0], dtype=np.uint8)
    rnd = np.concatenate([pos.view(np.uint8), sign])
    out = np.full((5, N), 7, dtype=np.uint64)
    ctx.HWTSampler(rnd, out.reshape(-1), h, 1, 1, 2)                                    # limbs idx_out + idx_mod + t = 2, 3
    assert (out[0] == 7).all() and (out[1] == 7).all() and (out[4] == 7).all()
    for t, q in enumerate(Q3[:2]):
        want = np.zeros(N, dtype=np.uint64)
        want[44] = q - 1
        want[5] = q - 1          # word 3 (byte 127) after word 0 (byte 200)
        want[255] = 1
        want[17] = q - 1         # word 5 (byte 0) after word 2 (byte 128)
        assert np.array_equal(out[2 + t], want)


# ---- pointwise arithmetic (poly_arithmetic.cuh) ----
def test_poly_ops_against_python_integers():
    ctx = O.OracleContext(8, P1, Q3)
    N = ctx.N
    pq = P1 + Q3
    rng = np.random.default_rng(3)
    a = np.stack([rng.integers(0, q, N, dtype=np.uint64) for q in pq])
    b = np.stack([rng.integers(0, q, N, dtype=np.uint64) for q in pq])
    a[1, :3] = [0, Q3[0] - 1, Q3[0] - 1]
    b[1, :3] = [0, Q3[0] - 1, 1]
    for op, f in ((0, lambda x, y, q: x * y % q), (1, lambda x, y, q: (x + y) % q), (2, lambda x, y, q: (x - y) % q)):
        c = np.zeros((4, N), dtype=np.uint64)
        ctx.poly_op(op, c.reshape(-1), a.reshape(-1), b.reshape(-1), 2, 1, 1, 1, 2)     # limbs 1, 2 (primes q0, q1) -> limbs 2, 3
        for t in range(2):
            q = pq[1 + t]
            assert [int(v) for v in c[2 + t]] == [f(int(x), int(y), q) for x, y in zip(a[1 + t], b[1 + t])]
        assert not c[:2].any()


# ---- keys, encryption, decryption (SecretKey.cuh:18-31, Scheme_23.cuh:54-127) ----
def centred(v, q):
    v = int(v) % q
    return v - q if v > q // 2 else v


def test_keys_and_encryption_decrypt_identities():
    ctx = O.OracleContext(8, P1, Q3)
    N, K, L1 = ctx.N, ctx.K, ctx.L + 1
    h = 32
    stream = O.salsa20_stream(5 * h + 8 * N * L1 + 4 * N + 9 * N + 64, bytes(range(32)), 1)
    sx = np.zeros((K + L1, N), dtype=np.uint64)
    ctx.keygen_secret(sx.reshape(-1), stream[: 5 * h], h)
    s_coeff = sx.copy()
    ctx.FromNTTInplace(s_coeff.reshape(-1), 0, 0, 1, K + L1, K + L1)
    pq = P1 + Q3
    s = [centred(v, pq[0]) for v in s_coeff[0]]
    assert set(s) <= {-1, 0, 1} and 0 < sum(abs(v) for v in s) <= h
    for j, q in enumerate(pq):
        assert [centred(v, q) for v in s_coeff[j]] == s                                 # one secret, reduced per prime
    # public key: a*s + b = e, a small polynomial
    ra = stream[5 * h: 5 * h + 8 * N * L1]
    re = stream[5 * h + 8 * N * L1: 5 * h + 8 * N * L1 + 4 * N]
    pk = np.zeros((2, L1, N), dtype=np.uint64)
    ctx.keygen_public(pk.reshape(-1), sx.reshape(-1), np.ascontiguousarray(ra), np.ascontiguousarray(re))
    pkc = pk.copy()
    ctx.FromNTTInplace(pkc.reshape(-1), 0, K, 2, L1, L1)
    noise = None
    for j, q in enumerate(Q3):
        a_s = negacyclic_mul([int(v) for v in pkc[0, j]], [v % q for v in s], q)
        e = [centred(x + int(y), q) for x, y in zip(a_s, pkc[1, j])]
        assert max(abs(v) for v in e) <= 19
        assert noise is None or e == noise
        noise = e
    assert any(noise)
    # encryption of a message at level 1, decryption, noise bound; limbs above the level untouched / zeroed
    l = 1
    m = [int(v) for v in np.random.default_rng(2).integers(-(1 << 20), 1 << 20, N)]
    mx = np.zeros((L1, N), dtype=np.uint64)
    for j in range(l + 1):
        mx[j] = [v % Q3[j] for v in m]
    ctx.ToNTTInplace(mx.reshape(-1), 0, K, 1, l + 1, L1)
    renc = np.ascontiguousarray(stream[5 * h + 8 * N * L1 + 4 * N: 5 * h + 8 * N * L1 + 4 * N + 9 * N])
    ct = np.full((2, L1, N), 5, dtype=np.uint64)
    ctx.encrypt(ct.reshape(-1), mx.reshape(-1), pk.reshape(-1), renc, l)
    assert (ct[:, l + 1:] == 5).all()
    dec = np.full((L1, N), 9, dtype=np.uint64)
    ctx.decrypt(dec.reshape(-1), ct.reshape(-1), sx.reshape(-1), l)
    assert not dec[l + 1:].any()
    ctx.FromNTTInplace(dec.reshape(-1), 0, K, 1, l + 1, L1)
    err0 = [centred(int(v) - mm, Q3[0]) for v, mm in zip(dec[0], m)]
    err1 = [centred(int(v) - mm, Q3[1]) for v, mm in zip(dec[1], m)]
    assert err0 == err1                                                                  # the same small integer modulo both primes
    assert 0 < max(abs(v) for v in err0) <= 19 * (N + h + 1)                             # v*e + e1 + e0*s
    # the decryption is exactly a*s + b in the coefficient domain
    ctc = ct.copy()
    ctx.FromNTTInplace(ctc.reshape(-1), 0, K, 2, l + 1, L1)
    a_s = negacyclic_mul([int(v) for v in ctc[0, 0]], [v % Q3[0] for v in s], Q3[0])
    assert [int(v) for v in dec[0]] == [(x + int(y)) % Q3[0] for x, y in zip(a_s, ctc[1, 0])]
    # encryptZero = the same call without a message: the difference is the message
    ct0 = np.zeros((2, L1, N), dtype=np.uint64)
    ctx.encrypt(ct0.reshape(-1), None, pk.reshape(-1), renc, l)
    assert np.array_equal(ct0[0], np.where(np.arange(L1)[:, None] <= l, ct[0], 0))
    for j in range(l + 1):
        assert [int(v) for v in ct[1, j]] == [(int(x) + int(y)) % Q3[j] for x, y in zip(ct0[1, j], mx[j])]


# ---- coefficient encoding (Encoder.cuh:67-186) ----
def test_encode_and_decode_coeffs_against_exact_integers():
    ctx = O.OracleContext(8, P1, Q3)
    N, K, L1 = ctx.N, ctx.K, ctx.L + 1
    rng = np.random.default_rng(9)
    vals = rng.normal(0, 3.0, N)
    vals[:4] = [0.0, -1.0, 1.0 - 2 ** -30, -7.999]
    scale = 1 << 30
    l = 2
    mx = np.zeros((L1, N), dtype=np.uint64)
    ctx.encode_coeffs(mx.reshape(-1), vals, scale, l)
    coeff = mx.copy()
    ctx.FromNTTInplace(coeff.reshape(-1), 0, K, 1, l + 1, L1)
    ints = [int(v * scale) for v in vals]                                               # truncation toward zero (:75)
    for j in range(l + 1):
        assert [int(v) for v in coeff[j]] == [c % Q3[j] for c in ints]
    # values beyond one prime still reduce to the residue
    big = np.zeros(N)
    big[0], big[1] = 2.0 ** 40, -2.0 ** 40
    ctx.encode_coeffs(mx.reshape(-1), big, 1 << 10, 0)
    c0 = mx.copy()
    ctx.FromNTTInplace(c0.reshape(-1), 0, K, 1, 1, L1)
    assert int(c0[0, 0]) == (1 << 50) % Q3[0] and int(c0[0, 1]) == (-(1 << 50)) % Q3[0]
    # decode: chosen centred integers, including the ends of the range, come back as the nearest double of c / scale
    for l, slots, sc in ((2, N // 2, float(1 << 30)), (1, N // 8, 3.0 * 2 ** 20), (0, N // 2, 1.0)):
        Q = 1
        for q in Q3[: l + 1]:
            Q *= q
        cs = [int(rng.integers(-(1 << 62), 1 << 62)) * int(rng.integers(1, 1 << 40)) % Q for _ in range(N)]
        cs = [c - Q if c > Q // 2 else c for c in cs]
        cs[0], cs[N // 2] = Q // 2, -(Q // 2)
        gap = (N // 2) // slots
        if gap < N // 2:
            cs[gap] = (1 << 53) + 1 if Q > (1 << 55) else 5                              # needs the sticky bit to round correctly
        res = np.zeros((L1, N), dtype=np.uint64)
        for j in range(l + 1):
            res[j] = [c % Q3[j] for c in cs]
        ctx.ToNTTInplace(res.reshape(-1), 0, K, 1, l + 1, L1)
        got = ctx.decode_coeffs(res.reshape(-1), sc, slots, l)
        want = np.zeros(N)
        for j in range(slots):
            for idx in (j * gap, N // 2 + j * gap):
                want[idx] = float(Fraction(cs[idx]) / Fraction(sc))
        assert np.array_equal(got, want)
        gotr = ctx.decode_coeffs(res.reshape(-1), sc, slots, l, is_bitrev=True)
        for idx in range(N):
            r = int(format(idx, "08b")[::-1], 2)
            assert gotr[r] == want[idx] * 256
    # round trip of the encoder
    mx = np.zeros((L1, N), dtype=np.uint64)
    ctx.encode_coeffs(mx.reshape(-1), vals, scale, 2)
    back = ctx.decode_coeffs(mx.reshape(-1), float(scale), N // 2, 2)
    assert np.abs(back - vals).max() <= 1.0 / scale
