"""GPU parity of the switching-key generation in the T basis, the NTT-domain automorphisms and the homomorphic multiply / rotate /
conjugate through the C ABI against the CPU oracle on the same random bytes: bit-exact on every word; plus the reference's flow
through the mirror classes with a decrypt check."""
import numpy as np
import pytest

from ckks_llm_amd import CkksError, Ciphertext, Context_23, DeviceBuffer, Plaintext, Scheme_23, SecretKey
from oracle import oracle_py as O
from tests.gpu_common import Pair, to_dev, from_dev
from tests.params import REF_PARAMS

pytestmark = pytest.mark.gpu

KEY = bytes(range(7, 39))


def ref_pair(params, logN):
    P = REF_PARAMS[params]
    return Pair(logN, P["p"], P["q"], P["t"], P["gamma"])


def test_automorphisms_match_oracle():
    pair = ref_pair(14, 10)
    N, K, L1 = pair.N, pair.orc.K, pair.orc.L + 1
    pq = pair.orc.p + pair.orc.q
    rng = np.random.default_rng(0)
    a = np.stack([rng.integers(0, m, N, dtype=np.uint64) for m in pq[:5]])
    d_a = to_dev(a)
    for idx in (1, 7, N // 2 - 3, N // 2):
        pow_ = pair.orc.rot_group(idx)
        assert pair.dev.rotGroups(idx) == pow_
        want = np.full((6, N), 4, dtype=np.uint64)
        pair.orc.automorph_ntt(want.reshape(-1), a.reshape(-1), pow_, 2, 1, 4)
        d = to_dev(np.full((6, N), 4, dtype=np.uint64))
        assert pair.dev.L_.ckks_poly_automorph_ntt(pair.dev.h, d.ptr, d_a.ptr, pow_, 2, 1, 4) == 0
        assert np.array_equal(from_dev(d, want.shape), want)
    # the mirror's two named forms are each other's inverse
    d1, d2 = to_dev(np.zeros((5, N), dtype=np.uint64)), to_dev(np.zeros((5, N), dtype=np.uint64))
    pair.dev.sk_and_poly_LeftRot_ntt(d1, d_a, 9, 0, 0, 5)
    pair.dev.sk_and_poly_LeftRot_inv(d2, d1, 9, 0, 0, 5)
    assert np.array_equal(from_dev(d2, a.shape), a)
    want = np.zeros((5, N), dtype=np.uint64)
    pair.orc.conjugate_ntt(want.reshape(-1), a.reshape(-1), 1, 0, 4)
    d = to_dev(np.zeros((5, N), dtype=np.uint64))
    pair.dev.sk_and_poly_conjugate(d, d_a, 1, 0, 4)
    assert np.array_equal(from_dev(d, want.shape), want)
    assert pair.dev.L_.ckks_poly_automorph_ntt(pair.dev.h, d.ptr, d_a.ptr, 4, 0, 0, 1) != 0        # even exponent
    assert pair.dev.L_.ckks_poly_automorph_ntt(pair.dev.h, d.ptr, d.ptr, 5, 0, 0, 1) != 0          # in place


@pytest.mark.parametrize("params,logN", [(14, 10), (15, 8), (13, 12)])
def test_switch_keys_and_operations_match_oracle(params, logN):
    pair = ref_pair(params, logN)
    orc, dev = pair.orc, pair.dev
    N, K, L, T, RB, dnum = pair.N, orc.K, orc.L, orc.t_num, orc.Ri_blockNum, orc.dnum
    L1, KL = L + 1, K + L + 1
    L_ = dev.L_
    h = 64
    na, ne = dnum * 8 * N * KL, dnum * 4 * N
    rnd = O.salsa20_stream(5 * h + 8 * N * L1 + 4 * N + 3 * (na + ne) + 2 * 9 * N, KEY, params)
    d_rnd = DeviceBuffer.from_numpy(rnd)
    off = [0]

    def take(n):
        o = off[0]
        off[0] += n
        return o

    o_sk, o_pa, o_pe = take(5 * h), take(8 * N * L1), take(4 * N)
    sx = np.zeros((KL, N), dtype=np.uint64)
    orc.keygen_secret(sx.reshape(-1), np.ascontiguousarray(rnd[o_sk:o_sk + 5 * h]), h)
    pk = np.zeros((2, L1, N), dtype=np.uint64)
    orc.keygen_public(pk.reshape(-1), sx.reshape(-1), np.ascontiguousarray(rnd[o_pa:o_pa + 8 * N * L1]), np.ascontiguousarray(rnd[o_pe:o_pe + 4 * N]))
    d_sx, d_pk = to_dev(sx), to_dev(pk)
    scratch = DeviceBuffer(8 * N * KL)
    # three kinds of keys: s^2 -> s, reversed s -> s, s -> permuted s
    sxsx = np.zeros((L1, N), dtype=np.uint64)
    orc.poly_op(0, sxsx.reshape(-1), sx.reshape(-1), sx.reshape(-1), 0, K, K, K, L1)
    s_conj = np.zeros((L1, N), dtype=np.uint64)
    orc.conjugate_ntt(s_conj.reshape(-1), sx.reshape(-1), 0, K, L1)
    rot = 3
    s_rot = np.zeros((KL, N), dtype=np.uint64)
    orc.automorph_ntt(s_rot.reshape(-1), sx.reshape(-1), orc.rot_group(rot), 0, 0, KL)
    keys = {}
    for name, s_to, s_from in (("mult", sx, sxsx), ("conj", sx, s_conj), ("rot", s_rot, np.ascontiguousarray(sx[K:]))):
        oa, oe = take(na), take(ne)
        want = np.zeros((2, dnum, RB * T, N), dtype=np.uint64)
        orc.keygen_switch_23(want.reshape(-1), np.ascontiguousarray(s_to).reshape(-1), s_from.reshape(-1),
                             np.ascontiguousarray(rnd[oa:oa + na]), np.ascontiguousarray(rnd[oe:oe + ne]))
        d_key = to_dev(np.zeros(want.shape, dtype=np.uint64))
        assert L_.ckks_keygen_switch_23(dev.h, d_key.ptr, to_dev(s_to).ptr, to_dev(s_from).ptr, d_rnd.ptr + oa, d_rnd.ptr + oe, scratch.ptr) == 0
        assert np.array_equal(from_dev(d_key, want.shape), want), name
        keys[name] = (want, d_key)
    # ciphertexts of two messages
    rng = np.random.default_rng(params)
    cts = []
    for k in range(2):
        mx = np.zeros((L1, N), dtype=np.uint64)
        for j in range(L1):
            mx[j] = rng.integers(0, 1 << 20, N, dtype=np.uint64)
        orc.ToNTTInplace(mx.reshape(-1), 0, K, 1, L1, L1)
        ct = np.zeros((2, L1, N), dtype=np.uint64)
        oe = take(9 * N)
        orc.encrypt(ct.reshape(-1), mx.reshape(-1), pk.reshape(-1), np.ascontiguousarray(rnd[oe:oe + 9 * N]), L)
        cts.append(ct)
    d_c1, d_c2 = to_dev(cts[0]), to_dev(cts[1])
    work = DeviceBuffer(8 * N * L1 * 3)
    up, ext, buf = DeviceBuffer(8 * N * T * orc.Qj_blockNum), DeviceBuffer(8 * N * T * RB * 2), DeviceBuffer(8 * N * T * RB * 2)
    for l in sorted({L, max(1, L // 2), 1}):
        want = np.full((2, L1, N), 6, dtype=np.uint64)
        orc.mult_23(want.reshape(-1), cts[0].reshape(-1), cts[1].reshape(-1), keys["mult"][0].reshape(-1), l)
        d_out = to_dev(np.full((2, L1, N), 6, dtype=np.uint64))
        assert L_.ckks_mult_23(dev.h, d_out.ptr, d_c1.ptr, d_c2.ptr, keys["mult"][1].ptr, l, work.ptr, up.ptr, ext.ptr, buf.ptr) == 0
        got = from_dev(d_out, want.shape)
        assert np.array_equal(got[:, :l + 1], want[:, :l + 1]), ("mult", l)
        want = np.zeros((2, L1, N), dtype=np.uint64)
        orc.leftRotate_23(want.reshape(-1), cts[0].reshape(-1), keys["rot"][0].reshape(-1), rot, l)
        assert L_.ckks_rotate_23(dev.h, d_out.ptr, d_c1.ptr, keys["rot"][1].ptr, rot, l, work.ptr, up.ptr, ext.ptr, buf.ptr) == 0
        got = from_dev(d_out, want.shape)
        assert np.array_equal(got[:, :l + 1], want[:, :l + 1]), ("rot", l)
        want = np.zeros((2, L1, N), dtype=np.uint64)
        orc.conjugate_23(want.reshape(-1), cts[0].reshape(-1), keys["conj"][0].reshape(-1), l)
        assert L_.ckks_conjugate_23(dev.h, d_out.ptr, d_c1.ptr, keys["conj"][1].ptr, l, work.ptr, up.ptr, ext.ptr, buf.ptr) == 0
        got = from_dev(d_out, want.shape)
        assert np.array_equal(got[:, :l + 1], want[:, :l + 1]), ("conj", l)
        assert np.array_equal(from_dev(d_c1, cts[0].shape), cts[0])                       # operands are left as they were
    # errors: level 0 and a missing key are the reference's std::invalid_argument (CKKS_E_STATE = -4)
    assert L_.ckks_mult_23(dev.h, d_out.ptr, d_c1.ptr, d_c2.ptr, keys["mult"][1].ptr, 0, work.ptr, up.ptr, ext.ptr, buf.ptr) == -4
    assert L_.ckks_mult_23(dev.h, d_out.ptr, d_c1.ptr, d_c2.ptr, None, L, work.ptr, up.ptr, ext.ptr, buf.ptr) == -4
    assert L_.ckks_rotate_23(dev.h, d_out.ptr, d_c1.ptr, None, rot, L, work.ptr, up.ptr, ext.ptr, buf.ptr) == -4
    assert L_.ckks_conjugate_23(dev.h, d_out.ptr, d_c1.ptr, None, L, work.ptr, up.ptr, ext.ptr, buf.ptr) == -4
    assert L_.ckks_rotate_23(dev.h, d_c1.ptr, d_c1.ptr, keys["rot"][1].ptr, rot, L, work.ptr, up.ptr, ext.ptr, buf.ptr) not in (0, -4)


def negacyclic_fp(a, b):
    n = len(a)
    full = np.convolve(a, b)
    out = full[:n].copy()
    out[: n - 1] -= full[n:]
    return out


def substitute_fp(a, g):
    n = len(a)
    out = np.zeros(n)
    for i, v in enumerate(a):
        e = i * g % (2 * n)
        if e < n:
            out[e] += v
        else:
            out[e - n] -= v
    return out


def test_mirror_classes_multiply_rotate_conjugate():
    """The reference's flow with its class names on its logN = 14 parameter set (at N = 2^12): keys, encode_coeffs, encryptMsg, mult_23 +
    rescaleAndEqual, leftRotate_23, conjugate_23, decryptMsg, decode_coeffs; the results are the polynomial product, m(X^(5^r)) and m(X^-1)."""
    P = REF_PARAMS[14]
    ctx = Context_23(12, P["p"], P["q"], P["t"], P["gamma"])
    N, L = ctx.N, ctx.L
    sk = SecretKey(ctx, h=64, key=KEY, nonce=11)
    scheme = Scheme_23(ctx, key=KEY)
    scheme.addEncKey(sk)
    rng = np.random.default_rng(1)
    v1, v2 = rng.uniform(-1, 1, N), rng.uniform(-1, 1, N)
    scale = float(1 << 30)
    c = []
    for v in (v1, v2):
        msg = Plaintext(N, L, L, N // 2, int(scale))
        ctx.encode_coeffs(DeviceBuffer.from_numpy(v), msg)
        ct = Ciphertext(N, L, L, N // 2, int(scale))
        scheme.encryptMsg(ct, msg)
        c.append(ct)
    res = Ciphertext(N, L, L, N // 2, 1)
    with pytest.raises(ValueError):
        scheme.mult_23(res, c[0], c[1])                                     # no relinearisation key yet
    with pytest.raises(ValueError):
        scheme.leftRotate_23(res, c[0], 5)
    with pytest.raises(ValueError):
        scheme.conjugate_23(res, c[0])
    scheme.addMultKey_23(sk)
    scheme.addConjKey_23(sk)
    scheme.addLeftRotKey_23(sk, 5)
    out = Plaintext(N, L, L, N // 2, 1)
    d_vals = DeviceBuffer(8 * N)

    def decoded(ct):
        scheme.decryptMsg(out, sk, ct)
        ctx.decode_coeffs(out, d_vals)
        return d_vals.download(np.float64)

    scheme.mult_23(res, c[0], c[1])
    assert res.l == L and res.scale == scale * scale
    want = negacyclic_fp(v1, v2)
    got = decoded(res)
    assert np.abs(got - want).max() < 1e-3 and np.abs(want).max() > 10
    scheme.rescaleAndEqual(res)
    assert res.l == L - 1
    got = decoded(res)
    assert np.abs(got - want).max() < 1e-3
    scheme.leftRotate_23(res, c[0], 5)
    got = decoded(res)
    assert np.abs(got - substitute_fp(v1, pow(5, 5, 2 * N))).max() < 1e-4
    scheme.conjugate_23(res, c[0])
    got = decoded(res)
    assert np.abs(got - substitute_fp(v1, 2 * N - 1)).max() < 1e-4
    zero = Ciphertext(N, L, 0, N // 2, 1)
    with pytest.raises(ValueError):
        scheme.mult_23(res, c[0], zero)                                     # level 0 (KeySwitch_23.cuh:194-197)


def test_in_place_and_derived_members_leave_the_same_words():
    """multAndEqual_23, square, squareAndEqual, conjugateAndEqual_23, leftRotateAndEqual_23, rightRotateAndEqual_23,
    leftRotateAddSelf_23, add / sub and their in-place forms, rescaleToAndEqual: each against the separate-result member (parity-
    tested against the oracle above) or against the oracle / numpy directly, word for word."""
    P = REF_PARAMS[14]
    logN = 10
    pair = Pair(logN, P["p"], P["q"], P["t"], P["gamma"])
    ctx, orc = pair.dev, pair.orc
    N, L, K = ctx.N, ctx.L, ctx.K
    sk = SecretKey(ctx, h=32, key=KEY, nonce=21)
    scheme = Scheme_23(ctx, key=KEY)
    scheme.addEncKey(sk)
    scheme.addMultKey_23(sk)
    scheme.addConjKey_23(sk)
    r_right = N // 2 - (1 << 3)
    for r in (3, r_right):
        scheme.addLeftRotKey_23(sk, r)
    rng = np.random.default_rng(5)
    scale = float(1 << 30)

    def fresh(l=None):
        msg = Plaintext(N, L, L, N // 2, int(scale))
        ctx.encode_coeffs(DeviceBuffer.from_numpy(rng.uniform(-1, 1, N)), msg)
        ct = Ciphertext(N, L, L, N // 2, int(scale))
        scheme.encryptMsg(ct, msg)
        if l is not None:
            ct.l = l
        return ct

    def words(ct, l=None):
        l = ct.l if l is None else l
        return ct.cipher_device.download(np.uint64).reshape(2, L + 1, N)[:, : l + 1].copy()

    def clone(ct):
        c2 = Ciphertext(N, L, ct.l, ct.slots, ct.scale)
        c2.cipher_device.upload(ct.cipher_device.download(np.uint64))
        return c2

    a, b = fresh(), fresh(L - 2)
    res = Ciphertext(N, L, L, N // 2, 1)
    # multAndEqual_23 (levels differ: the lower one wins)
    scheme.mult_23(res, a, b)
    a2 = clone(a)
    scheme.multAndEqual_23(a2, b)
    assert a2.l == L - 2 and a2.scale == a.scale * b.scale and np.array_equal(words(a2), words(res))
    # square / squareAndEqual = the product of a ciphertext with itself
    scheme.mult_23(res, a, a)
    sq = Ciphertext(N, L, L, N // 2, 1)
    scheme.square(sq, a)
    assert sq.l == a.l and np.array_equal(words(sq), words(res))
    a2 = clone(a)
    scheme.squareAndEqual(a2)
    assert a2.scale == a.scale * a.scale and np.array_equal(words(a2), words(res))
    # conjugate / rotations in place
    scheme.conjugate_23(res, a)
    a2 = clone(a)
    scheme.conjugateAndEqual_23(a2)
    assert np.array_equal(words(a2), words(res))
    scheme.leftRotate_23(res, a, 3)
    a2 = clone(a)
    scheme.leftRotateAndEqual_23(a2, 3)
    assert np.array_equal(words(a2), words(res))
    rot3 = words(res)
    scheme.leftRotate_23(res, a, r_right)
    a2 = clone(a)
    scheme.rightRotateAndEqual_23(a2, 3)                                     # right by 2^3 slots
    assert np.array_equal(words(a2), words(res))
    # leftRotateAddSelf_23, add, sub against numpy on the residues
    q = np.array(ctx.qVec, dtype=object)[None, :, None]
    a2 = clone(a)
    scheme.leftRotateAddSelf_23(a2, 3)
    assert np.array_equal(words(a2).astype(object), (words(a).astype(object) + rot3.astype(object)) % q[:, : L + 1])
    lo = L - 2
    scheme.add(res, a, b)
    assert res.l == lo and np.array_equal(words(res).astype(object), (words(a, lo).astype(object) + words(b).astype(object)) % q[:, : lo + 1])
    scheme.sub(res, a, b)
    assert res.l == a.l and np.array_equal(words(res, lo).astype(object), (words(a, lo).astype(object) - words(b).astype(object)) % q[:, : lo + 1])
    a2 = clone(a)
    scheme.addAndEqual(a2, b)
    assert a2.l == lo and a2.scale == a.scale and np.array_equal(words(a2).astype(object), (words(a, lo).astype(object) + words(b).astype(object)) % q[:, : lo + 1])
    a2 = clone(a)
    scheme.subAndEqual(a2, b)
    assert a2.l == lo and np.array_equal(words(a2).astype(object), (words(a, lo).astype(object) - words(b).astype(object)) % q[:, : lo + 1])
    # rescaleToAndEqual against the oracle's steps
    a2 = clone(a)
    want = a.cipher_device.download(np.uint64).copy()
    orc.FromNTTInplace(want, 0, K, 2, L + 1, L + 1)
    for l in range(L, L - 3, -1):
        orc.rescaleAndEqual_noNTT(want, l)
    orc.ToNTTInplace(want, 0, K, 2, L - 2, L + 1)
    scheme.rescaleToAndEqual(a2, L - 3)
    assert a2.l == L - 3 and np.array_equal(words(a2), want.reshape(2, L + 1, N)[:, : L - 2])
    prod = float(np.prod([float(x) for x in ctx.qVec[L - 2:]]))
    assert abs(a2.scale * prod / a.scale - 1) < 1e-9
