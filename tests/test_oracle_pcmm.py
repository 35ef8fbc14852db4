"""Pins the oracle's RLWE->MLWE gather and PPMM: notebook vectors, ring identity, big-int brute force."""
import numpy as np
import pytest

from oracle import oracle_py as O
from tests.helpers import negacyclic_mul, limbs_uniform
from tests.params import CFG2_Q, REF_PARAMS


def ring_down(poly, N, N1):
    """ring_packing.ipynb cell 1 `ringDown`: sub-ring i takes coefficients i, i+k, i+2k, ..."""
    k = N // N1
    return [[poly[i + g * k] for g in range(N1)] for i in range(k)]


def test_notebook_algebra_is_consistent(golden_nb):
    """The test's own negacyclic algebra reproduces the numbers the notebook printed (cell 1): per-sub-ring
    products, their sum ('inner product') and the extraction target."""
    q = golden_nb["q"]
    a, s = golden_nb["cell1_ax_big_ring"], golden_nb["cell0_sx_big_ring"]
    a_down, s_down = ring_down(a, 32, 8), ring_down(s, 32, 8)
    assert a_down == golden_nb["cell1_ax_down"]
    prods = [negacyclic_mul(x, y, q) for x, y in zip(a_down, s_down)]
    assert prods == golden_nb["cell1_products"]
    ip = [sum(p[i] for p in prods) % q for i in range(8)]
    assert ip == golden_nb["cell1_inner_product"] == golden_nb["cell1_target"]
    tw_s = negacyclic_mul(golden_nb["cell1_twist"], s, q)
    assert tw_s == golden_nb["cell1_twist_times_sx"]
    assert ring_down(tw_s, 32, 8)[0] == golden_nb["cell1_target"]


def make_small_ctx(q_list, logN=5, p=None):
    # N = 32; every modulus must be 1 mod 64
    return O.OracleContext(logN, p or [], q_list)


def test_decompose_notebook_kat(golden_nb):
    """Extract(twist(a)) returns the sub-rings of a (ring_packing.ipynb cells 1,3): the gather kernel applied to the
    printed 'twist' polynomial must give the printed 'ax down' rows."""
    q = golden_nb["q"]
    ctx = make_small_ctx([q])
    pc = O.OraclePCMM(ctx, 8, 4, [], [q])
    rlwe = np.zeros((2, 1, 32), dtype=np.uint64)
    rlwe[0, 0] = golden_nb["cell1_twist"]
    rlwe[1, 0] = np.arange(32) * 2                      # cell 0: bx = [2i]
    mlwe = [np.zeros((1, 5, 8), dtype=np.uint64)]
    pc.rlweCipherDecompose(rlwe.reshape(-1), [m.reshape(-1) for m in mlwe], 0)
    assert [[int(v) for v in row] for row in mlwe[0][0, :4]] == golden_nb["cell1_ax_down"]
    assert [int(v) for v in mlwe[0][0, 4]] == [2 * (g * 4) for g in range(8)]


@pytest.mark.parametrize("mlwe_num", [4, 2, 1])
def test_decompose_ring_identity(mlwe_num):
    """b_m + sum_i a_{m,i} * s_i  ==  ringDown(a*s + b)[m*gap]  for every extracted MLWE sample m
    (decryption convention m = a*s + b, Scheme_23.cuh:125-126; PCMM_Scheme.cuh:546-552)."""
    N, N1, k = 32, 8, 4
    qs = [65537, 0xfff9c0001]
    ctx = make_small_ctx(qs)
    pc = O.OraclePCMM(ctx, N1, k, [], qs)
    rng = np.random.default_rng(mlwe_num)
    rlwe = limbs_uniform(3, qs, 2, N)                     # [2][L+1][N] coefficient domain
    s = [int(v) for v in rng.integers(-1, 2, N)]
    mlwe = [np.zeros((2, k + 1, N1), dtype=np.uint64) for _ in range(mlwe_num)]
    pc.rlweCipherDecompose(rlwe.reshape(-1), [m.reshape(-1) for m in mlwe], 1)
    gap = k // mlwe_num
    for im, q in enumerate(qs):
        a = [int(v) for v in rlwe[0, im]]
        b = [int(v) for v in rlwe[1, im]]
        big = negacyclic_mul(a, [v % q for v in s], q)
        big = [(x + y) % q for x, y in zip(big, b)]
        s_down = ring_down([v % q for v in s], N, N1)
        for m in range(mlwe_num):
            acc = [int(v) for v in mlwe[m][im, k]]
            for i in range(k):
                pr = negacyclic_mul([int(v) for v in mlwe[m][im, i]], s_down[i], q)
                acc = [(x + y) % q for x, y in zip(acc, pr)]
            assert acc == ring_down(big, N, N1)[m * gap]


@pytest.mark.parametrize("mod_num", [2, 3, 1])
def test_ppmm_bruteforce(mod_num):
    N1, k, M, Kin = 4, 3, 5, 6
    qs = CFG2_Q[:mod_num]
    ctx = make_small_ctx(qs, logN=5)
    pc = O.OraclePCMM(ctx, N1, k, [CFG2_Q[5]], qs)
    C = (k + 1) * N1
    rng = np.random.default_rng(mod_num)
    W = rng.normal(0, 0.02, (M, Kin)).astype(np.float32)
    W[0, 0] = 0.0                                           # exercises the A == 0 -> q mapping (PPMM_kernel.cuh:25)
    scaler = float(2 ** 26)
    mlwe = [limbs_uniform(10 + n, qs, 1, C)[0] for n in range(Kin)]      # [mod][C]
    out = np.zeros((M, mod_num, C), dtype=np.uint64)
    pc.PPMM(W, [m.reshape(-1) for m in mlwe], out.reshape(-1), M, Kin, mod_num, scaler)
    A = [[int(float(W[m, n]) * scaler) for n in range(Kin)] for m in range(M)]     # trunc toward zero
    qlast = qs[-1]
    for m in range(M):
        for c in range(C):
            last = sum(A[m][n] * int(mlwe[n][mod_num - 1, c]) for n in range(Kin)) % qlast
            assert int(out[m, mod_num - 1, c]) == last
            for im in range(mod_num - 1):
                q = qs[im]
                r = sum(A[m][n] * int(mlwe[n][im, c]) for n in range(Kin)) % q
                assert int(out[m, im, c]) == (r - last) * pow(qlast, -1, q) % q
    # column panel restriction computes the same numbers
    out2 = np.zeros_like(out)
    pc.PPMM(W, [m.reshape(-1) for m in mlwe], out2.reshape(-1), M, Kin, mod_num, scaler, 4, 8)
    assert np.array_equal(out2[:, :, 4:12], out[:, :, 4:12]) and not out2[:, :, :4].any() and not out2[:, :, 12:].any()


def test_ppmm_rescale_is_rounding_division():
    """Two primes (the reference's shape): the fused rescale returns the exact quotient (X - [X]_q1) / q1 of the
    integer X that both residues represent, so the output decodes to about X / q1."""
    N1, k, M, Kin = 4, 1, 2, 3
    qs = CFG2_Q[:2]
    ctx = make_small_ctx(qs, logN=5)
    pc = O.OraclePCMM(ctx, N1, k, [CFG2_Q[5]], qs)
    C = (k + 1) * N1
    rng = np.random.default_rng(0)
    W = rng.normal(0, 0.02, (M, Kin)).astype(np.float32)
    scaler = float(2 ** 20)
    small = [rng.integers(-1000, 1000, C) for _ in range(Kin)]
    mlwe = [np.array([[int(v) % q for v in small[n]] for q in qs], dtype=np.uint64) for n in range(Kin)]
    out = np.zeros((M, 2, C), dtype=np.uint64)
    pc.PPMM(W, [m.reshape(-1) for m in mlwe], out.reshape(-1), M, Kin, 2, scaler)
    A = [[int(float(W[m, n]) * scaler) for n in range(Kin)] for m in range(M)]
    for m in range(M):
        for c in range(C):
            X = sum(A[m][n] * int(small[n][c]) for n in range(Kin))
            want = (X - (X % qs[1])) // qs[1]
            assert int(out[m, 0, c]) == want % qs[0]


@pytest.mark.parametrize("mlwe_num", [16, 4])
def test_packing_decrypt_identity(mlwe_num):
    """mlweCipherPacking (PCMM_Scheme.cuh:361-425) pinned end to end on a small ring: decompose an RLWE ciphertext of mu into
    MLWE samples, build repacking keys the way addRepakcingKey does (key_i = (a_i, -a_i*s + p0*iota(s_i)), s_i[n] = s[i + n*k],
    PCMM_Scheme.cuh:128-224, ringSwitch.cuh:7-19; noise left out), pack, decrypt with s: the result is mu on the positions
    n*k + m*gap and 0 elsewhere, up to the rounding of the ModDown.  A wrong embedding position, lift, key slot or sign breaks it."""
    from tests.params import CFG3_P
    logN, N, N1, k = 8, 256, 16, 16
    P0, Q0, Q1 = CFG3_P[0], CFG2_Q[0], CFG2_Q[1]
    ctx = O.OracleContext(logN, [P0], [Q0, Q1])
    pc = O.OraclePCMM(ctx, N1, k, [P0], [Q0, Q1])
    rng = np.random.default_rng(100 + mlwe_num)
    s = [int(v) for v in rng.integers(-1, 2, N)]
    mu = [int(v) for v in rng.integers(-(1 << 20), 1 << 20, N)]
    a = [int(v) for v in rng.integers(0, Q0, N)]
    a_s = negacyclic_mul(a, [v % Q0 for v in s], Q0)
    b = [(m - x) % Q0 for m, x in zip(mu, a_s)]                       # decryption convention mu = a*s + b
    rlwe = np.zeros((2, 2, N), dtype=np.uint64)                         # [a | b], L + 1 = 2 limbs, level 0 in use
    rlwe[0, 0], rlwe[1, 0] = a, b
    mlwe = [np.zeros((1, k + 1, N1), dtype=np.uint64) for _ in range(mlwe_num)]
    pc.rlweCipherDecompose(rlwe.reshape(-1), [m.reshape(-1) for m in mlwe], 0)
    # repacking keys over [P0, Q0], coefficient domain first
    keys = np.zeros((k, 2, 2, N), dtype=np.uint64)
    for i in range(k):
        iota = [0] * N
        for n in range(N1):
            iota[n * k] = s[i + n * k]
        for j, q in enumerate((P0, Q0)):
            ai = [int(v) for v in rng.integers(0, q, N)]
            ais = negacyclic_mul(ai, [v % q for v in s], q)
            keys[i, 0, j] = ai
            keys[i, 1, j] = [(-x + P0 * t) % q for x, t in zip(ais, iota)]
        for y in range(2):
            ctx.ToNTTInplace(keys[i, y].reshape(-1), 0, 0, 1, 2, 2)      # primes [P0, Q0] = context primes 0, 1
    out = np.zeros((2, 2, N), dtype=np.uint64)
    pc.mlweCipherPacking(out.reshape(-1), [m.reshape(-1) for m in mlwe], keys.reshape(-1))
    ctx.FromNTTInplace(out.reshape(-1), 0, 1, 2, 1, 2)                   # limb 0 of both polynomials, prime Q0
    a2, b2 = [int(v) for v in out[0, 0]], [int(v) for v in out[1, 0]]
    dec = [(x + y) % Q0 for x, y in zip(negacyclic_mul(a2, [v % Q0 for v in s], Q0), b2)]
    gap = k // mlwe_num
    worst = 0
    for pos in range(N):
        want = mu[pos] if (pos % k) % gap == 0 else 0
        d = (dec[pos] - want) % Q0
        d = d - Q0 if d > Q0 // 2 else d
        worst = max(worst, abs(d))
    assert worst <= N, worst


def test_packing_rejects_what_the_reference_cannot_do():
    ctx = O.OracleContext(8, [CFG2_Q[5]], CFG2_Q[:3])
    pc = O.OraclePCMM(ctx, 16, 16, [CFG2_Q[5]], CFG2_Q[:3])               # two remaining moduli: the reference's embedding overlaps
    with pytest.raises(ValueError):
        pc.mlweCipherPacking(np.zeros(2 * 3 * 256, dtype=np.uint64), [np.zeros(2 * 17 * 16, dtype=np.uint64)], np.zeros(16 * 2 * 3 * 256, dtype=np.uint64))


def test_small_ring_ntt_is_the_negacyclic_transform():
    """PCMM_Context::ToNTTInplace / FromNTTInplace (size N1 over the ring-pack primes): round trip, the convolution theorem
    against the schoolbook negacyclic product, the closed form for a monomial, and the [batch][mod][poly][N1] layout."""
    N1, k = 256, 4
    qs = CFG2_Q[:3]
    ctx = O.OracleContext(10, [], qs)
    pc = O.OraclePCMM(ctx, N1, k, qs[:1], qs[1:])
    rng = np.random.default_rng(11)
    batch, mod_num, polys = 2, 2, 3
    data = np.empty((batch, mod_num, polys, N1), dtype=np.uint64)
    for j in range(mod_num):
        data[:, j] = rng.integers(0, qs[1 + j], (batch, polys, N1), dtype=np.uint64)
    work = data.copy()
    pc.ToNTTInplace(work.reshape(-1), polys, mod_num, 0, 1, batch)          # primes pq[1], pq[2]
    for j in range(mod_num):
        q = qs[1 + j]
        a, b = [int(v) for v in data[0, j, 0]], [int(v) for v in data[1, j, 2]]
        prod = [(int(x) * int(y)) % q for x, y in zip(work[0, j, 0], work[1, j, 2])]
        arr = np.array(prod, dtype=np.uint64).reshape(1, 1, 1, N1).copy()
        # inverse of the pointwise product = negacyclic product (one limb of prime j: start_mod_idx 1 + j)
        pc.FromNTTInplace(arr.reshape(-1), 1, 1, 0, 1 + j, 1)
        assert [int(v) for v in arr.reshape(-1)] == negacyclic_mul(a, b, q)
    back = work.copy()
    pc.FromNTTInplace(back.reshape(-1), polys, mod_num, 0, 1, batch)
    assert np.array_equal(back, data)
    # monomial X^5 modulo pq[0]: position bitrev(i) holds psi^(5 * (2 i + 1)), psi the 2*N1-th root the reference's search finds
    q = qs[0]
    mono = np.zeros(N1, dtype=np.uint64); mono[5] = 1
    pc.ToNTTInplace(mono, 1, 1, 0, 0, 1)
    psi = O.lib().orc_find_mth_root(2 * N1, q)
    assert pow(psi, N1, q) == q - 1
    from tests.helpers import bitrev
    for i in (0, 1, 7, 100, 255):
        assert int(mono[bitrev(i, 8)]) == pow(psi, 5 * (2 * i + 1), q)


def test_mlwe_secret_repacking_keys_and_mlwe_decryption_with_generated_keys():
    """convertMLWESKfromRLWESK, addRepakcingKey, mlweDecrypt and decodeCoeffs (PCMM_Scheme.cuh:23-48, 126-224, 531-576; PCMM_Context.cuh:149-178)
    with keys from the oracle's own generators: the small secrets are the strided coefficients of the big one; every repacking key satisfies
    a*s + b = p0*iota(s_i) + e with one small e for both primes; an MLWE sample of the gather decrypts to exactly the RLWE decryption at the
    gathered positions; and gather -> PPMM -> packing with these keys decrypts to W times the message."""
    from tests.params import CFG3_P
    logN, N, N1, k, h = 8, 256, 16, 16, 32
    P0, Q0, Q1 = CFG3_P[0], CFG2_Q[0], CFG2_Q[1]
    pq = [P0, Q0, Q1]
    ctx = O.OracleContext(logN, [P0], [Q0, Q1])
    pc = O.OraclePCMM(ctx, N1, k, [P0], [Q0, Q1])
    per_key = 4 * N + 8 * N * 2
    stream = O.salsa20_stream(5 * h + 64 + 8 * N * 2 + 4 * N + 9 * N + k * per_key, bytes(range(32)), 77)
    sx = np.zeros((3, N), dtype=np.uint64)
    ctx.keygen_secret(sx.reshape(-1), np.ascontiguousarray(stream[:5 * h]), h)
    sc = sx.copy()
    ctx.FromNTTInplace(sc.reshape(-1), 0, 0, 1, 3, 3)
    s = [int(v) if v <= 1 else -1 for v in sc[0]]
    # ---- MLWE secret ----
    msk = np.zeros((3, k, N1), dtype=np.uint64)
    pc.convertMLWESKfromRLWESK(msk.reshape(-1), sx.reshape(-1))
    small = msk.copy()
    pc.FromNTTInplace(small.reshape(-1), k, 3, 0, 0, 1)
    for j, q in enumerate(pq):
        for i in range(k):
            assert [int(v) for v in small[j, i]] == [s[i + n * k] % q for n in range(N1)]
    # ---- repacking keys ----
    o = 5 * h + 64
    pk = np.zeros((2, 2, N), dtype=np.uint64)
    ctx.keygen_public(pk.reshape(-1), sx.reshape(-1), np.ascontiguousarray(stream[o:o + 8 * N * 2]), np.ascontiguousarray(stream[o + 8 * N * 2:o + 8 * N * 2 + 4 * N]))
    o += 8 * N * 2 + 4 * N
    renc = np.ascontiguousarray(stream[o:o + 9 * N])
    o += 9 * N
    keys = np.zeros((k, 2, 2, N), dtype=np.uint64)
    msk_before = msk.copy()
    pc.addRepakcingKey(keys.reshape(-1), msk.reshape(-1), sx.reshape(-1), np.ascontiguousarray(stream[o:o + k * per_key]))
    assert np.array_equal(msk, msk_before)
    kc = keys.copy()
    for i in range(k):
        for y in range(2):
            ctx.FromNTTInplace(kc[i, y].reshape(-1), 0, 0, 1, 2, 2)
    seen = set()
    for i in (0, 5, k - 1):
        es = []
        for j, q in enumerate((P0, Q0)):
            a_s = negacyclic_mul([int(v) for v in kc[i, 0, j]], [v % q for v in s], q)
            iota = [0] * N
            for n in range(N1):
                iota[n * k] = s[i + n * k]
            e = [(x + int(b) - P0 * t) % q for x, b, t in zip(a_s, kc[i, 1, j], iota)]
            es.append([v - q if v > q // 2 else v for v in e])
        assert es[0] == es[1] and max(abs(v) for v in es[0]) <= 19 and any(es[0])
        seen.add(tuple(es[0]))
    assert len(seen) == 3                                                   # every key has its own noise
    # ---- encrypt, gather, MLWE decryption = RLWE decryption at the gathered positions ----
    rng = np.random.default_rng(3)
    mu = [int(v) for v in rng.integers(-(1 << 32), 1 << 32, N)]
    mx = np.zeros((2, N), dtype=np.uint64)
    for j, q in enumerate((Q0, Q1)):
        mx[j] = [v % q for v in mu]
    ctx.ToNTTInplace(mx.reshape(-1), 0, 1, 1, 2, 2)
    ct = np.zeros((2, 2, N), dtype=np.uint64)
    ctx.encrypt(ct.reshape(-1), mx.reshape(-1), pk.reshape(-1), renc, 1)
    dec = np.zeros((2, N), dtype=np.uint64)
    ctx.decrypt(dec.reshape(-1), ct.reshape(-1), sx.reshape(-1), 1)
    ctx.FromNTTInplace(dec.reshape(-1), 0, 1, 1, 2, 2)
    ctc = ct.copy()
    ctx.FromNTTInplace(ctc.reshape(-1), 0, 1, 2, 2, 2)
    mlwe_num = 4
    gap = k // mlwe_num
    mlwe = [np.zeros((2, k + 1, N1), dtype=np.uint64) for _ in range(mlwe_num)]
    pc.rlweCipherDecompose(ctc.reshape(-1), [m.reshape(-1) for m in mlwe], 1)
    for j in range(mlwe_num):
        before = mlwe[j].copy()
        plain = np.zeros((2, N1), dtype=np.uint64)
        pc.mlweDecrypt(plain.reshape(-1), mlwe[j].reshape(-1), msk.reshape(-1), 1)
        assert np.array_equal(mlwe[j], before)
        vals = pc.decodeCoeffs(plain.reshape(-1), 1 << 10, 1)
        pcoef = plain.copy()
        pc.FromNTTInplace(pcoef.reshape(-1), 1, 2, 0, 1, 1)
        for im in range(2):
            assert [int(v) for v in pcoef[im]] == [int(dec[im, j * gap + n * k]) for n in range(N1)]
        want = [(int(v) if v <= Q0 // 2 else int(v) - Q0) / 1024.0 for v in pcoef[0]]
        assert list(vals) == want
    # ---- gather -> PPMM -> packing with the generated keys decrypts to W * mu ----
    M = Kin = mlwe_num
    W = rng.normal(0, 0.02, (M, Kin)).astype(np.float32)
    scaler = float(1 << 26)
    C = (k + 1) * N1
    out = np.zeros((M, 2, C), dtype=np.uint64)
    pc.PPMM(W, [m.reshape(-1) for m in mlwe], out.reshape(-1), M, Kin, 2, scaler)
    rows = [np.ascontiguousarray(out[m, 0]) for m in range(M)]
    res = np.zeros((2, 2, N), dtype=np.uint64)
    pc.mlweCipherPacking(res.reshape(-1), rows, keys.reshape(-1))
    d2 = np.zeros((2, N), dtype=np.uint64)
    ctx.decrypt(d2.reshape(-1), res.reshape(-1), sx.reshape(-1), 0)
    ctx.FromNTTInplace(d2.reshape(-1), 0, 1, 1, 1, 2)
    got = [int(v) if v <= Q0 // 2 else int(v) - Q0 for v in d2[0]]
    A = [[int(np.float64(W[m, n]) * scaler) for n in range(Kin)] for m in range(M)]
    worst = biggest = 0
    for g in range(N1):
        for m in range(M):
            want = sum(A[m][n] * mu[n * gap + g * k] for n in range(Kin)) // Q1
            worst = max(worst, abs(got[g * k + m * gap] - want))
            biggest = max(biggest, abs(want))
    assert biggest > 1 << 16 and worst <= N, (worst, biggest)
