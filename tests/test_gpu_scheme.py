"""GPU parity of the client-side entry points (random stream, samplers, pointwise arithmetic, keys, encryption, decryption,
coefficient encode / decode) through the C ABI against the CPU oracle: bit-exact on every integer word; the decoder's doubles
exact for power-of-two scales and within one unit in the last place otherwise."""
import numpy as np
import pytest

from ckks_llm_amd import CkksError, Ciphertext, Context_23, DeviceBuffer, Plaintext, Scheme_23, SecretKey
from oracle import oracle_py as O
from tests.gpu_common import Pair, to_dev, from_dev
from tests.params import CFG2_Q, CFG3_P

pytestmark = pytest.mark.gpu

KEY = bytes(range(1, 33))


def dev_bytes(a):
    return DeviceBuffer.from_numpy(np.ascontiguousarray(a, dtype=np.uint8))


@pytest.mark.parametrize("n", [64, 100, 4096 + 17, 9 * 65536, 0])
def test_random_stream_is_salsa20(n):
    pair = Pair(8, [], CFG2_Q[:1])
    buf = DeviceBuffer(n + 64)
    buf.upload(np.full(n + 64, 0xAB, dtype=np.uint8))
    pair.dev.generateRandom_device(buf, n, KEY, 0x0123456789ABCDEF)
    got = buf.download(np.uint8)
    assert np.array_equal(got[:n], O.salsa20_stream(n, KEY, 0x0123456789ABCDEF))
    assert (got[n:] == 0xAB).all()                                       # nothing written past the requested length
    if n == 64:
        # unaligned destination: the byte-wise store path
        pair.dev.generateRandom_device(buf.ptr + 3, 61, KEY, 5)
        assert np.array_equal(buf.download(np.uint8)[3:64], O.salsa20_stream(61, KEY, 5))
        with pytest.raises(ValueError):
            pair.dev.generateRandom_device(buf, 8, b"short", 0)


@pytest.mark.parametrize("logN", [8, 12])
def test_samplers_match_oracle(logN):
    p, q = CFG3_P[:1], CFG2_Q[:3]
    pair = Pair(logN, p, q)
    N = pair.N
    h = 64
    rnd = O.salsa20_stream(8 * N * 3 + 64, KEY, logN)
    rnd[:8] = 0
    rnd[8:16] = 255
    rnd[16:20] = 255                                                      # gaussian word 4 = 2^32 - 1 -> +19
    d_rnd = dev_bytes(rnd)
    L4 = 5                                                                # buffer of 5 limbs
    for name, args_o, args_d in (
        ("uniform", lambda o: pair.orc.uniformSampler_xq(rnd, o, 1, 1, 3), lambda d: pair.dev.uniformSampler_xq(d_rnd, d, 1, 1, 3)),
        ("gauss", lambda o: pair.orc.gaussianSampler_xq(rnd, o, 1, 0, 4), lambda d: pair.dev.gaussianSampler_xq(d_rnd, d, 1, 0, 4)),
        ("zo", lambda o: pair.orc.ZOSampler(rnd, o, 0.5, 2, 1, 2), lambda d: pair.dev.ZOSampler(d_rnd, d, 0.5, 2, 1, 2)),
        ("zo25", lambda o: pair.orc.ZOSampler(rnd, o, 0.25, 0, 0, 4), lambda d: pair.dev.ZOSampler(d_rnd, d, 0.25, 0, 0, 4)),
        ("hwt", lambda o: pair.orc.HWTSampler(rnd, o, h, 1, 1, 3), lambda d: pair.dev.HWTSampler(d_rnd, d, h, 1, 1, 3)),
    ):
        want = np.full((L4, N), 3, dtype=np.uint64)
        args_o(want.reshape(-1))
        d = to_dev(np.full((L4, N), 3, dtype=np.uint64))
        args_d(d)
        assert np.array_equal(from_dev(d, want.shape), want), name
    # colliding positions in the sparse sampler: the later word wins
    pos = np.zeros(h, dtype=np.uint32)
    pos[:] = np.arange(h) % 7 + N * 3
    sign = (np.arange(h) * 37 % 256).astype(np.uint8)
    r2 = np.concatenate([pos.view(np.uint8), sign])
    want = np.zeros((2, N), dtype=np.uint64)
    pair.orc.HWTSampler(r2, want.reshape(-1), h, 0, 0, 2)
    d = to_dev(np.full((2, N), 9, dtype=np.uint64))
    pair.dev.HWTSampler(dev_bytes(r2), d, h, 0, 0, 2)
    assert np.array_equal(from_dev(d, want.shape), want)
    assert np.count_nonzero(want[0]) == 7
    with pytest.raises(CkksError):
        pair.dev.uniformSampler_xq(d_rnd, d, 0, 3, 2)                     # primes 3, 4 of four
    with pytest.raises(CkksError):
        pair.dev.gaussianSampler_xq(d_rnd.ptr + 1, d, 0, 0, 1)            # misaligned words


def test_pointwise_ops_match_oracle():
    p, q = CFG3_P[:1], CFG2_Q[:3]
    pair = Pair(10, p, q)
    N = pair.N
    pq = p + q
    rng = np.random.default_rng(1)
    a = np.stack([rng.integers(0, m, N, dtype=np.uint64) for m in pq])
    b = np.stack([rng.integers(0, m, N, dtype=np.uint64) for m in pq])
    a[:, 0], b[:, 0] = 0, 0
    for j, m in enumerate(pq):
        a[j, 1], b[j, 1] = m - 1, m - 1
        a[j, 2], b[j, 2] = 0, m - 1
    da, db = to_dev(a), to_dev(b)
    ops = (pair.dev.barrett_batch_3param_device, pair.dev.poly_add_3param_batch_device, pair.dev.poly_sub_3param_batch_device)
    for op in range(3):
        want = np.full((4, N), 11, dtype=np.uint64)
        pair.orc.poly_op(op, want.reshape(-1), a.reshape(-1), b.reshape(-1), 1, 0, 1, 1, 3)   # c[1+t] = a[t] (op) b[1+t] mod prime 1+t
        dc = to_dev(np.full((4, N), 11, dtype=np.uint64))
        ops[op](dc, da, db, 1, 0, 1, 1, 3)
        assert np.array_equal(from_dev(dc, want.shape), want), op
    # in place: b = a - b (poly_sub2_batch_device, poly_arithmetic.cuh:474-478)
    want = b.copy()
    pair.orc.poly_op(2, want.reshape(-1), a.reshape(-1), b.reshape(-1), 0, 0, 0, 0, 4)
    pair.dev.poly_sub_3param_batch_device(db, da, db, 0, 0, 0, 0, 4)
    assert np.array_equal(from_dev(db, want.shape), want)
    with pytest.raises(CkksError):
        pair.dev.barrett_batch_3param_device(db, da, db, 0, 0, 0, 2, 3)


@pytest.mark.parametrize("logN,nq,l", [(8, 3, 1), (12, 4, 3), (16, 2, 1)])
def test_keys_encrypt_decrypt_match_oracle(logN, nq, l):
    p, q = CFG3_P[:1], CFG2_Q[:nq]
    pair = Pair(logN, p, q)
    N, K, L1 = pair.N, 1, nq
    h = 64
    rnd = O.salsa20_stream(5 * h + 8 * N * L1 + 4 * N + 9 * N, KEY, 100 + logN)
    o_sk, o_pk, o_enc = 0, 5 * h, 5 * h + 8 * N * L1 + 4 * N
    # the device draws the same bytes itself
    d_rnd = DeviceBuffer(rnd.size)
    pair.dev.generateRandom_device(d_rnd, rnd.size, KEY, 100 + logN)
    assert np.array_equal(d_rnd.download(np.uint8), rnd)
    L_ = pair.dev.L_
    sx = np.zeros((K + L1, N), dtype=np.uint64)
    pair.orc.keygen_secret(sx.reshape(-1), np.ascontiguousarray(rnd[:5 * h]), h)
    d_sx = to_dev(np.full(sx.shape, 1, dtype=np.uint64))
    assert L_.ckks_keygen_secret(pair.dev.h, d_sx.ptr, d_rnd.ptr + o_sk, h) == 0
    assert np.array_equal(from_dev(d_sx, sx.shape), sx)
    pk = np.zeros((2, L1, N), dtype=np.uint64)
    pair.orc.keygen_public(pk.reshape(-1), sx.reshape(-1), np.ascontiguousarray(rnd[o_pk:o_pk + 8 * N * L1]),
                           np.ascontiguousarray(rnd[o_pk + 8 * N * L1:o_enc]))
    d_pk = to_dev(np.zeros(pk.shape, dtype=np.uint64))
    assert L_.ckks_keygen_public(pair.dev.h, d_pk.ptr, d_sx.ptr, d_rnd.ptr + o_pk, d_rnd.ptr + o_pk + 8 * N * L1) == 0
    assert np.array_equal(from_dev(d_pk, pk.shape), pk)
    # message limbs (NTT domain), encryption at level l with and without a message
    mx = np.zeros((L1, N), dtype=np.uint64)
    rng = np.random.default_rng(logN)
    for j in range(l + 1):
        mx[j] = rng.integers(0, q[j], N, dtype=np.uint64)
    d_mx = to_dev(mx)
    scratch = DeviceBuffer(8 * N * (l + 1))
    for msg, d_msg in ((mx, d_mx.ptr), (None, None)):
        ct = np.full((2, L1, N), 5, dtype=np.uint64)
        pair.orc.encrypt(ct.reshape(-1), None if msg is None else msg.reshape(-1), pk.reshape(-1), np.ascontiguousarray(rnd[o_enc:]), l)
        d_ct = to_dev(np.full(ct.shape, 5, dtype=np.uint64))
        assert L_.ckks_encrypt(pair.dev.h, d_ct.ptr, d_msg, d_pk.ptr, d_rnd.ptr + o_enc, scratch.ptr, l) == 0
        assert np.array_equal(from_dev(d_ct, ct.shape), ct)
        dec = np.full((L1, N), 9, dtype=np.uint64)
        pair.orc.decrypt(dec.reshape(-1), ct.reshape(-1), sx.reshape(-1), l)
        d_dec = to_dev(np.full(dec.shape, 9, dtype=np.uint64))
        assert L_.ckks_decrypt(pair.dev.h, d_dec.ptr, d_ct.ptr, d_sx.ptr, l) == 0
        assert np.array_equal(from_dev(d_dec, dec.shape), dec)
    assert L_.ckks_encrypt(pair.dev.h, d_ct.ptr, None, d_pk.ptr, d_rnd.ptr + o_enc, scratch.ptr, L1) != 0          # level above L
    assert L_.ckks_decrypt(pair.dev.h, d_dec.ptr, d_ct.ptr, d_sx.ptr, -1) != 0


def ulp_close(a, b):
    return np.all((a == b) | (np.abs(a - b) <= np.spacing(np.maximum(np.abs(a), np.abs(b)))))


@pytest.mark.parametrize("logN,nq", [(8, 3), (12, 24), (12, 1)])
def test_encode_decode_coeffs_match_oracle(logN, nq):
    """nq = 24 primes of 36 bits: an 864-bit modulus, 16 machine words in the decoder."""
    p, q = CFG3_P[:1], CFG2_Q[:nq]
    pair = Pair(logN, p, q)
    N, K, L1 = pair.N, 1, nq
    L_ = pair.dev.L_
    rng = np.random.default_rng(nq)
    vals = rng.normal(0, 2.0, N)
    vals[:4] = [0.0, -1.0, 1.0 - 2.0 ** -30, -7.999]
    d_vals = DeviceBuffer.from_numpy(vals)
    scale = 1 << 30
    for l in sorted({0, nq // 2, nq - 1}):
        mx = np.zeros((L1, N), dtype=np.uint64)
        pair.orc.encode_coeffs(mx.reshape(-1), vals, scale, l)
        d_mx = to_dev(np.zeros(mx.shape, dtype=np.uint64))
        assert L_.ckks_encode_coeffs(pair.dev.h, d_mx.ptr, d_vals.ptr, scale, l) == 0
        assert np.array_equal(from_dev(d_mx, mx.shape), mx)
        # decoding: random residues (a uniformly random integer modulo Q), several slot counts, both orders, two kinds of scale
        res = np.zeros((L1, N), dtype=np.uint64)
        for j in range(l + 1):
            res[j] = rng.integers(0, q[j], N, dtype=np.uint64)
        res[: l + 1, 0] = 0
        res[: l + 1, 1] = 1
        for j in range(l + 1):
            res[j, 2] = q[j] - 1                                          # the integer -1
        pair.orc.ToNTTInplace(res.reshape(-1), 0, K, 1, l + 1, L1)
        d_res = to_dev(res)
        scratch = DeviceBuffer(8 * N * (l + 1))
        d_out = DeviceBuffer(8 * N)
        for slots, sc, bitrev in ((N // 2, float(1 << 30), 0), (N // 8, 2.0 ** -3, 1), (1, 12345.678, 0), (N // 2, 3.0e9, 0)):
            want = pair.orc.decode_coeffs(res.reshape(-1), sc, slots, l, is_bitrev=bool(bitrev))
            d_out.upload(np.full(N, 77.0))
            assert L_.ckks_decode_coeffs(pair.dev.h, d_out.ptr, d_res.ptr, scratch.ptr, sc, slots, bitrev, l) == 0
            got = d_out.download(np.float64)
            if sc == float(1 << 30) or sc == 2.0 ** -3:
                assert np.array_equal(got, want), (l, slots)
            else:
                assert ulp_close(got, want), (l, slots)
            assert np.count_nonzero(got) <= 2 * slots
        assert np.array_equal(from_dev(d_res, res.shape), res)            # the plaintext itself is not modified
        # encoder -> decoder round trip on the device
        assert L_.ckks_decode_coeffs(pair.dev.h, d_out.ptr, d_mx.ptr, scratch.ptr, float(scale), N // 2, 0, l) == 0
        assert np.abs(d_out.download(np.float64) - vals).max() <= 1.0 / scale
        assert L_.ckks_decode_coeffs(pair.dev.h, d_out.ptr, d_mx.ptr, scratch.ptr, float(scale), 3, 0, l) != 0       # 3 does not divide N/2
        assert L_.ckks_decode_coeffs(pair.dev.h, d_out.ptr, d_mx.ptr, scratch.ptr, 0.0, 1, 0, l) != 0


def test_decoder_rounds_to_nearest_with_sticky_bits():
    """Integers that sit exactly between two doubles, and just beside such a point with the deciding bit far below the top 64."""
    p, q = CFG3_P[:1], CFG2_Q[:6]
    pair = Pair(8, p, q)
    N, K, L1 = pair.N, 1, 6
    Q = 1
    for m in q:
        Q *= m
    cs = [0] * N
    cs[0] = (1 << 53) + 1                       # tie: rounds to even 2^53
    cs[1] = (1 << 53) + 3                       # tie: rounds to even 2^53 + 4
    cs[2] = (1 << 120) + (1 << 67)              # tie at bit 67 of a 121-bit number
    cs[3] = (1 << 120) + (1 << 67) + 1          # just above the tie: the last bit decides
    cs[4] = -((1 << 200) + (1 << 147) + 1)
    cs[5] = Q // 2
    cs[6] = -(Q // 2)
    cs[7] = (1 << 64) - 1
    cs[8] = 1 << 64
    cs[9] = (1 << 128) - 1
    res = np.zeros((L1, N), dtype=np.uint64)
    for j in range(L1):
        res[j] = [c % q[j] for c in cs]
    pair.orc.ToNTTInplace(res.reshape(-1), 0, K, 1, L1, L1)
    d_out = DeviceBuffer(8 * N)
    scratch = DeviceBuffer(8 * N * L1)
    assert pair.dev.L_.ckks_decode_coeffs(pair.dev.h, d_out.ptr, to_dev(res).ptr, scratch.ptr, 1.0, N // 2, 0, L1 - 1) == 0
    got = d_out.download(np.float64)
    assert [float(c) for c in cs[:10]] == list(got[:10])                 # Python's int -> float is correctly rounded
    assert not got[10:].any()


def test_mirror_classes_encrypt_decrypt_decode():
    """The reference's flow with its class names: encode_coeffs, encryptMsg, decryptMsg, decode_coeffs gives the message back up to
    the encryption noise; a rescale divides it by the last prime."""
    from ckks_llm_amd import Context_23
    p, q = CFG3_P[:1], CFG2_Q[:3]
    ctx = Context_23(12, p, q)
    N, L = ctx.N, ctx.L
    sk = SecretKey(ctx, h=64, key=KEY, nonce=3)
    scheme = Scheme_23(ctx, key=KEY)
    with pytest.raises(ValueError):
        scheme.encryptZero(Ciphertext(N, L, L, N // 2, 1 << 30), L, N // 2)
    scheme.addEncKey(sk)
    rng = np.random.default_rng(0)
    vals = rng.uniform(-4, 4, N)
    scale = float(q[2]) * 2.0 ** 20                                       # so that the rescale leaves 2^20
    msg = Plaintext(N, L, L, N // 2, int(scale))
    ctx.encode_coeffs(DeviceBuffer.from_numpy(vals), msg)
    ct = Ciphertext(N, L, L, N // 2, int(scale))
    scheme.encryptMsg(ct, msg)
    assert (ct.l, ct.scale) == (L, int(scale))
    out = Plaintext(N, L, L, N // 2, 1)
    scheme.decryptMsg(out, sk, ct)
    d_vals = DeviceBuffer(8 * N)
    ctx.decode_coeffs(out, d_vals)
    got = d_vals.download(np.float64)
    noise = 19 * (N + 64 + 1)
    assert np.abs(got - vals).max() <= (noise + 1) / scale
    assert np.abs(got - vals).max() > 0                                   # there is noise
    # two encryptions of one message differ (fresh nonce), both decrypt
    ct2 = Ciphertext(N, L, L, N // 2, int(scale))
    scheme.encryptMsg(ct2, msg)
    assert not np.array_equal(ct2.cipher_device.download(), ct.cipher_device.download())
    scheme.rescaleAndEqual(ct)
    assert ct.l == L - 1
    scheme.decryptMsg(out, sk, ct)
    out.scale = 2.0 ** 20
    ctx.decode_coeffs(out, d_vals)
    got = d_vals.download(np.float64)
    assert np.abs(got - vals).max() <= (noise / q[2] + N + 2) / 2.0 ** 20


def test_reference_constructor_selects_the_compiled_in_sets():
    """Context_23(logN, logslots, h, sigma), the reference's own constructor (Context_23.h:21): prime sets, gamma and precision of
    Params.cuh:11-170, the derived counts of Context_23.cuh:24-35, and one transform over all of [P | Q | T] against the oracle."""
    from ckks_llm_amd.params import REF_PARAMS
    for logN, counts in ((13, (1, 5, 3, 3)), (14, (2, 10, 4, 3)), (15, (4, 12, 7, 4)), (16, (4, 28, 8, 4))):
        ctx = Context_23(logN, logN - 1)
        assert (ctx.p_num, ctx.q_num, ctx.t_num, ctx.gamma) == counts
        assert ctx.slots == 1 << (logN - 1) and ctx.precision == (1 << 36 if logN < 15 else 1 << 49)
        assert ctx.dnum == ctx.q_num // ctx.p_num and ctx.Ri_blockNum == -(-(ctx.p_num + ctx.q_num) // ctx.gamma)
        assert ctx.Qj_blockNum == -(-ctx.q_num // ctx.p_num)
        if logN > 14:
            continue
        r = REF_PARAMS[logN]
        primes = r["p"] + r["q"] + r["t"]
        rng = np.random.default_rng(logN)
        x = np.stack([rng.integers(0, q, ctx.N, dtype=np.uint64) for q in primes])
        d = DeviceBuffer.from_numpy(x)
        ctx.ToNTTInplace(d, 0, 0, 1, len(primes), len(primes))
        orc = O.OracleContext(logN, r["p"], r["q"], r["t"], r["gamma"])
        want = x.copy()
        orc.ToNTTInplace(want, 0, 0, 1, len(primes), len(primes))
        assert np.array_equal(d.download(np.uint64).reshape(x.shape), want)
    with pytest.raises(ValueError, match="hamming weight error"):
        Context_23(13, 12, 100)
    with pytest.raises(ValueError):
        Context_23(12, 11)
    ctx = Context_23(13, 12, 192)
    sk = SecretKey(ctx)                                                      # the context's Hamming weight
    ctx.FromNTTInplace(sk.sx_device, 0, 0, 1, 1, ctx.K + ctx.L + 1)
    s0 = sk.sx_device.download(np.uint64, ctx.N)
    assert ctx.h_weight == 192 and 150 < np.count_nonzero(s0) <= 192 and set(np.unique(s0)) <= {0, 1, ctx.pVec[0] - 1}
