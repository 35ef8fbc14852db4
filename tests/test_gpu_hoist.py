"""GPU parity of the hoisted rotations of the slot <-> coefficient transforms (Giant_Rotate_And_Mult_PlaintT, Baby_Rotate,
cipher_mul_P, cipher_add_T, rescaleAndEqual_noNTT and one whole baby-step / giant-step level) through the C ABI against the CPU
oracle on the same seeded inputs: bit-exact on every word; plus the level through the mirror classes with generated keys and a
decrypt check."""
import ctypes as C

import numpy as np
import pytest

from ckks_llm_amd import Ciphertext, DeviceBuffer, EncodingMatrix, Plaintext, PlaintextT, Scheme_23, SecretKey
from tests.gpu_common import Pair, to_dev, from_dev
from tests.params import REF_PARAMS

pytestmark = pytest.mark.gpu


def ref_pair(params, logN):
    P = REF_PARAMS[params]
    return Pair(logN, P["p"], P["q"], P["t"], P["gamma"])


def ptr_table(bufs):
    T = C.c_void_p * max(len(bufs), 1)
    return T(*[(b.ptr if b is not None else None) for b in bufs])


def int_table(vals):
    T = C.c_int * max(len(vals), 1)
    return T(*[int(v) for v in vals])


def uniform_T(rng, orc, shape):
    """Uniform residues modulo the T primes; the T index is the second-to-last axis."""
    out = np.empty(shape, dtype=np.uint64)
    for k, t in enumerate(orc.t):
        out[..., k, :] = rng.integers(0, t, shape[:-2] + shape[-1:], dtype=np.uint64)
    return out


@pytest.mark.parametrize("params,logN,l,bs,gs,generic", [(14, 10, None, 2, 8, False), (15, 9, 2, 4, 16, False), (13, 11, 3, 3, 5, False),
                                                         (14, 8, 0, 1, 1, False), (15, 10, None, 8, 16, False), (13, 16, 3, 2, 4, False),
                                                         (15, 9, None, 4, 16, True), (14, 10, 3, 2, 3, True)])
def test_giant_and_baby_rotations_match_oracle(params, logN, l, bs, gs, generic):
    """generic: the integer back end is forced, which takes the kernels' 128-bit multiply-add path instead of the carry-free sums
    that primes below 2^60 allow."""
    pair = ref_pair(params, logN)
    orc, dev = pair.orc, pair.dev
    if generic:
        assert dev.L_.ckks_ctx_set_arith_mode(dev.h, 1) == 0
    l = orc.L if l is None else l
    N, K, L, T, RB, dnum = pair.N, orc.K, orc.L, orc.t_num, orc.Ri_blockNum, orc.dnum
    rng = np.random.default_rng(1000 * params + logN)
    up = uniform_T(rng, orc, (orc.Qj_blockNum, T, N))
    pqT = uniform_T(rng, orc, (2, RB, T, N))
    nkeys = min(gs, 3)                                               # distinct key buffers, reused over the rotations
    keybufs = [uniform_T(rng, orc, (2, dnum, RB, T, N)) for _ in range(nkeys)]
    slots = [int(v) for v in rng.integers(1, N // 2, gs)]
    keys = [keybufs[j % nkeys] for j in range(gs)]
    if gs > 1:
        keys[0], slots[0] = None, -1                                 # "no rotation"
    if gs > 4:
        keys[3], slots[3] = None, -1
    nplain = min(bs * gs, 5)
    plainbufs = [uniform_T(rng, orc, (T, N)) for _ in range(nplain)]
    accNum = [gs] * bs
    if bs > 1:
        accNum[-1] = max(gs - 1, 0)
    if bs > 2:
        accNum[1] = gs // 2
    plains = [plainbufs[(i * gs + j) % nplain] if j < accNum[i] else None for i in range(bs) for j in range(gs)]
    want = np.full((bs, 2, RB, T, N), 5, dtype=np.uint64)
    orc.Giant_Rotate_And_Mult_PlaintT(want.reshape(-1), pqT.reshape(-1), up.reshape(-1), [k.reshape(-1) if k is not None else None for k in keys],
                                      slots, [p.reshape(-1) if p is not None else None for p in plains], accNum, bs, gs, l)
    d_up, d_pqT = to_dev(up), to_dev(pqT)
    d_keybufs, d_plainbufs = [to_dev(k) for k in keybufs], [to_dev(p) for p in plainbufs]
    d_keys = [d_keybufs[j % nkeys] if keys[j] is not None else None for j in range(gs)]
    d_plains = [d_plainbufs[(i * gs + j) % nplain] if j < accNum[i] else None for i in range(bs) for j in range(gs)]
    d_out = to_dev(np.full(want.shape, 5, dtype=np.uint64))
    L_ = dev.L_
    print("giant", params, logN, l, bs, gs, flush=True)
    assert L_.ckks_giant_rotate_mult_plain_t(dev.h, d_out.ptr, d_pqT.ptr, d_up.ptr, ptr_table(d_keys), int_table(slots), ptr_table(d_plains),
                                             int_table(accNum), bs, gs, l) == 0
    got = from_dev(d_out, want.shape)
    assert np.array_equal(got, want)
    # Baby_Rotate: accumulate up to three rotations of the pair pqT into the first baby step's pair
    rot = [(d_keys[j], keys[j], slots[j]) for j in range(gs)][:3]
    want_b = want[0].copy()
    orc.Baby_Rotate(want_b.reshape(-1), up.reshape(-1), pqT.reshape(-1), [k.reshape(-1) if k is not None else None for _, k, _ in rot],
                    [s for _, _, s in rot], l)
    d_acc = to_dev(want[0])
    print("baby", len(rot), flush=True)
    assert L_.ckks_baby_rotate(dev.h, d_acc.ptr, d_up.ptr, d_pqT.ptr, len(rot), ptr_table([d for d, _, _ in rot]), int_table([s for _, _, s in rot]), l) == 0
    assert np.array_equal(from_dev(d_acc, want_b.shape), want_b)
    # error paths
    assert L_.ckks_giant_rotate_mult_plain_t(dev.h, d_out.ptr, d_pqT.ptr, d_up.ptr, ptr_table(d_keys), int_table(slots), ptr_table(d_plains),
                                             int_table(accNum), 9, gs, l) != 0
    assert L_.ckks_giant_rotate_mult_plain_t(dev.h, d_out.ptr, d_pqT.ptr, d_up.ptr, ptr_table(d_keys), int_table(slots), ptr_table(d_plains),
                                             int_table(accNum), bs, 17, l) != 0
    assert L_.ckks_baby_rotate(dev.h, d_acc.ptr, d_up.ptr, d_acc.ptr, 1, ptr_table(d_keys[-1:]), int_table(slots[-1:]), l) != 0      # in place


@pytest.mark.parametrize("params,logN", [(14, 10), (13, 12)])
def test_pointwise_helpers_match_oracle(params, logN):
    pair = ref_pair(params, logN)
    orc, dev = pair.orc, pair.dev
    N, K, L, T, RB = pair.N, orc.K, orc.L, orc.t_num, orc.Ri_blockNum
    rng = np.random.default_rng(params)
    L_ = dev.L_
    ct = np.stack([np.stack([rng.integers(0, q, N, dtype=np.uint64) for q in orc.q]) for _ in range(2)])
    for l in (L, 1, 0):
        want = np.full((2, K + L + 1, N), 9, dtype=np.uint64)
        orc.cipher_mul_P(want.reshape(-1), ct.reshape(-1), l)
        d = to_dev(np.full(want.shape, 9, dtype=np.uint64))
        assert L_.ckks_cipher_mul_p(dev.h, d.ptr, to_dev(ct).ptr, l) == 0
        assert np.array_equal(from_dev(d, want.shape), want)
        if l:
            want = ct.copy()
            orc.rescaleAndEqual_noNTT(want.reshape(-1), l)
            d = to_dev(ct)
            assert L_.ckks_rescale_coeff(dev.h, d.ptr, l) == 0
            assert np.array_equal(from_dev(d, want.shape), want)
    assert L_.ckks_rescale_coeff(dev.h, d.ptr, 0) != 0
    a, b = uniform_T(rng, orc, (2 * RB, T, N)), uniform_T(rng, orc, (2 * RB, T, N))
    want = a.copy()
    orc.cipher_add_T(want.reshape(-1), b.reshape(-1), 2 * RB)
    d = to_dev(a)
    assert L_.ckks_cipher_add_t(dev.h, d.ptr, to_dev(b).ptr, 2 * RB) == 0
    assert np.array_equal(from_dev(d, want.shape), want)


@pytest.mark.parametrize("params,logN,l", [(14, 10, None), (15, 9, 2), (13, 12, 4)])
def test_bsgs_level_matches_oracle(params, logN, l):
    """The whole level on a random coefficient-domain pair with random keys and plaintexts: every word of the result."""
    pair = ref_pair(params, logN)
    orc, dev = pair.orc, pair.dev
    l = orc.L if l is None else l
    N, K, L, T, RB, dnum = pair.N, orc.K, orc.L, orc.t_num, orc.Ri_blockNum, orc.dnum
    rng = np.random.default_rng(7 * params + logN)
    ct = np.zeros((2, L + 1, N), dtype=np.uint64)
    for i in range(l + 1):
        ct[:, i] = rng.integers(0, orc.q[i], (2, N), dtype=np.uint64)
    bs, gs = 3, 4
    rot_in, rot_out = [0, 1, 2, 3], [0, 4, 0]
    keyring = {r: uniform_T(rng, orc, (2, dnum, RB, T, N)) for r in (1, 2, 3, 4)}
    accNum = [4, 4, 3]
    plainbufs = [uniform_T(rng, orc, (T, N)) for _ in range(bs * gs)]
    plains = [plainbufs[i * gs + j] if j < accNum[i] else None for i in range(bs) for j in range(gs)]
    want = ct.copy()
    orc.bsgs_level_23(want.reshape(-1), l, [p.reshape(-1) if p is not None else None for p in plains], accNum, rot_in,
                      [keyring[r].reshape(-1) if r else None for r in rot_in], rot_out, [keyring[r].reshape(-1) if r else None for r in rot_out], bs, gs)
    d_ct = to_dev(ct)
    d_ring = {r: to_dev(k) for r, k in keyring.items()}
    d_plains = [to_dev(p) if p is not None else None for p in plains]
    words = C.c_size_t(0)
    L_ = dev.L_
    assert L_.ckks_bsgs_scratch_words(dev.h, bs, C.byref(words)) == 0
    scratch = DeviceBuffer(8 * words.value)
    print("bsgs level", params, logN, l, flush=True)
    rc = L_.ckks_bsgs_level_23(dev.h, d_ct.ptr, l, ptr_table(d_plains), int_table(accNum), int_table(rot_in), ptr_table([d_ring.get(r) for r in rot_in]),
                               int_table(rot_out), ptr_table([d_ring.get(r) for r in rot_out]), bs, gs, scratch.ptr)
    assert rc == 0
    got = from_dev(d_ct, ct.shape)
    assert np.array_equal(got[:, : l + 1], want[:, : l + 1])
    # a rotation without its key is the reference's "rotKey_23 not exists"
    rc = L_.ckks_bsgs_level_23(dev.h, d_ct.ptr, l, ptr_table(d_plains), int_table(accNum), int_table(rot_in), ptr_table([None] * gs),
                               int_table(rot_out), ptr_table([d_ring.get(r) for r in rot_out]), bs, gs, scratch.ptr)
    assert rc == -4


def test_level_through_the_mirror_decrypts_to_the_transformed_message():
    """EncodingMatrix.EvalLevel with keys from addLeftRotKey_23 on an encrypted message: the result decrypts to
    sum_i rho_i( sum_j p_ij * sigma_j(m) ), sigma / rho the substitutions X -> X^(5^r), and the level drops by one."""
    P = REF_PARAMS[14]
    logN = 10
    from ckks_llm_amd import Context_23
    ctx = Context_23(logN, P["p"], P["q"], P["t"], P["gamma"])
    N, L, T = ctx.N, ctx.L, ctx.t_num
    scheme = Scheme_23(ctx, key=bytes(range(32)))
    sk = SecretKey(ctx, h=32, key=bytes(range(32)), nonce=3)
    scheme.addEncKey(sk)
    for r in (1, 2, 7):
        scheme.addLeftRotKey_23(sk, r)
    rng = np.random.default_rng(2)
    scale = float(1 << 58)
    m = rng.integers(-1000, 1000, N).astype(np.float64) / 1000.0
    msg = Plaintext(N, L, L, N // 2, scale)
    ctx.encode_coeffs(DeviceBuffer.from_numpy(m), msg)
    ct = Ciphertext(N, L, L, N // 2, scale)
    scheme.encryptMsg(ct, msg)
    b, g = 2, 3
    rot_in, rot_out = [0, 1, 2], [0, 7]
    polys = rng.integers(-2, 3, (b * g, N))
    polys[b * g - 1] = 0
    numRotations = b * g - 1                                          # the last slot of the table has no plaintext
    tq = ctx.tVec
    A = []
    for i in range(b * g):
        pt = PlaintextT(N, T, 1.0)
        res = np.stack([np.mod(polys[i], t).astype(np.uint64) for t in tq])
        pt.mx_device.upload(res)
        ctx.ToNTTInplace(pt.mx_device, 0, ctx.K + L + 1, 1, T, T)
        A.append(pt)
    ctx.FromNTTInplace(ct.cipher_device, 0, ctx.K, 2, ct.l + 1, L + 1)            # the transforms work on the coefficient domain (:252)
    em = EncodingMatrix(scheme)
    em.EvalLevel(A, ct, rot_in, rot_out, b, g, numRotations, rescale=False)
    assert ct.l == L

    def decrypted(ct):
        tmp = Ciphertext(N, L, ct.l, N // 2, ct.scale)
        tmp.cipher_device.upload(ct.cipher_device.download(np.uint64))
        ctx.ToNTTInplace(tmp.cipher_device, 0, ctx.K, 2, ct.l + 1, L + 1)
        dec = Plaintext(N, L, ct.l, N // 2, ct.scale)
        scheme.decryptMsg(dec, sk, tmp)
        vals = DeviceBuffer(8 * N)
        ctx.decode_coeffs(dec, vals)
        return vals.download(np.float64)

    got = decrypted(ct)
    scheme.rescaleAndEqual_noNTT(ct)                                              # what EvalLevel does by default (:381)
    assert ct.l == L - 1 and abs(ct.scale * ctx.qVec[L] / scale - 1) < 1e-12
    got_rescaled = decrypted(ct)

    def substitute(a, e):
        out = np.zeros(N)
        for i in range(N):
            k = i * e % (2 * N)
            if k < N:
                out[k] += a[i]
            else:
                out[k - N] -= a[i]
        return out

    def negacyclic(p, a):
        full = np.convolve(p.astype(np.float64), a)
        out = full[:N].copy()
        out[: N - 1] -= full[N:]
        return out

    want = np.zeros(N)
    for i in range(b):
        inner = np.zeros(N)
        for j in range(g):
            if i * g + j != numRotations:
                inner += negacyclic(polys[i * g + j], substitute(m, pow(5, rot_in[j], 2 * N)))
        want += substitute(inner, pow(5, rot_out[i], 2 * N)) if i and rot_out[i] else inner
    assert np.abs(want).max() > 10
    assert np.abs(got - want).max() < 1e-6
    assert np.abs(got_rescaled - want).max() < 64.0 / ct.scale                   # the rescale's own rounding, at the lower scale
