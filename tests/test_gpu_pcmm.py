"""GPU parity: RLWE -> MLWE gather and PPMM through the C ABI against the CPU oracle, bit-exact."""
import os

import numpy as np
import pytest

from ckks_llm_amd import DeviceBuffer, PCMM_Context, PCMM_Scheme
from oracle import oracle_py as O
from tests.gpu_common import Pair, to_dev, from_dev
from tests.helpers import limbs_uniform
from tests.params import CFG2_Q, CFG3_P, REF_PARAMS

pytestmark = pytest.mark.gpu


def make(logN, N1, q_ctx, p_ctx, p_rp, q_rp):
    pair = Pair(logN, p_ctx, q_ctx)
    rank = pair.N // N1
    dev = PCMM_Scheme(PCMM_Context(N1, rank, p_rp, q_rp, pair.dev))
    orc = O.OraclePCMM(pair.orc, N1, rank, p_rp, q_rp)
    return pair, dev, orc, rank


@pytest.mark.parametrize("plain", [False, True])
@pytest.mark.parametrize("logN,N1,mlwe_num", [(10, 128, 8), (10, 128, 2), (12, 256, 16), (10, 64, 1), (14, 32, 512), (14, 32, 64),
                                              (12, 8, 512), (10, 4, 256)])
def test_rlwe_decompose(logN, N1, mlwe_num, plain):
    """Both gather kernels (LDS-tiled with 16- or 8-word row segments, and one lane per word - forced through the launcher's
    test hook, and taken anyway when N1 is not a multiple of 8) against the oracle."""
    q = CFG2_Q[:3]
    pair, dev, orc, rank = make(logN, N1, q, CFG3_P[:1], [CFG3_P[0]], q[:2])
    if plain:
        dev.pcmm_context.set_option("gather_plain")
    N, L = pair.N, len(q) - 1
    for l in (L, 0):
        rlwe = limbs_uniform(l + 1, q, 2, N)                                  # [2][L+1][N], coefficient domain
        rlwe[:, :, 0] = 0                                                     # negate(0) = 0 corner
        per = (L + 1) * (rank + 1) * N1
        want = [np.zeros(per, dtype=np.uint64) for _ in range(mlwe_num)]
        orc.rlweCipherDecompose(rlwe.reshape(-1), want, l)
        bufs = [DeviceBuffer(8 * per) for _ in range(mlwe_num)]
        for b in bufs:
            b.zero()
        dev.rlweCipherDecompose(to_dev(rlwe), bufs, mlwe_num, 0, l, coeff_domain=True)
        for m in range(mlwe_num):
            assert np.array_equal(bufs[m].download(), want[m]), (l, m)
        # NTT-domain entry point (PCMM_Scheme.cuh:107-124): iNTT, gather, NTT back
        rl_ntt = rlwe.copy()
        pair.orc.ToNTTInplace(rl_ntt.reshape(-1), 0, 1, 2, l + 1, L + 1)
        d_rl = to_dev(rl_ntt)
        for b in bufs:
            b.zero()
        dev.rlweCipherDecompose(d_rl, bufs, mlwe_num, 0, l)
        for m in range(mlwe_num):
            assert np.array_equal(bufs[m].download(), want[m]), ("ntt", l, m)
        assert np.array_equal(from_dev(d_rl, rl_ntt.shape), rl_ntt)
    with pytest.raises(Exception):
        dev.rlweCipherDecompose(to_dev(rlwe), bufs * (rank + 1), rank + 1, 0, L, coeff_domain=True)


def run_ppmm(dev, orc, rank, N1, M, Kin, mod_num, qs, scaler, seed, strided=False, w_std=0.02):
    C = (rank + 1) * N1
    rng = np.random.default_rng(seed)
    W = rng.normal(0, w_std, (M, Kin)).astype(np.float32)
    W[0, 0] = 0.0
    mlwe = [limbs_uniform(seed * 1000 + n, qs[:mod_num], 1, C)[0] for n in range(Kin)]
    want = np.zeros((M, mod_num, C), dtype=np.uint64)
    orc.PPMM(W, [m.reshape(-1) for m in mlwe], want.reshape(-1), M, Kin, mod_num, scaler)
    dW = DeviceBuffer.from_numpy(W)
    dout = DeviceBuffer(want.nbytes)
    dout.zero()
    if strided:
        dall = to_dev(np.stack(mlwe))
        dev.PPMM_strided(dW, dall, dout, M, Kin, mod_num, scaler)
    else:
        bufs = [to_dev(m) for m in mlwe]
        dev.PPMM(dW, bufs, dout, M, Kin, N1, Kin, mod_num, scaler)
    got = from_dev(dout, want.shape)
    assert np.array_equal(got, want)
    return dev.pcmm_context.info("last_path")


@pytest.mark.parametrize("mod_num", [1, 2, 3])
def test_ppmm_small_36bit(mod_num):
    """C = 9*128 = 1152 columns (multiple of 64): the MFMA path when it is built, 36-bit primes."""
    q = CFG2_Q[:4]
    pair, dev, orc, rank = make(10, 128, q, CFG3_P[:1], [CFG3_P[0]], q[:3])
    assert run_ppmm(dev, orc, rank, 128, 48, 40, mod_num, q, float(2 ** 26), seed=mod_num) == 1          # MFMA kernel
    assert run_ppmm(dev, orc, rank, 128, 130, 64, mod_num, q, float(2 ** 26), seed=10 + mod_num, strided=True) == 1
    # 4 plaintext digits (|A| up to 2^30) and a K that is not a multiple of the MFMA depth
    assert run_ppmm(dev, orc, rank, 128, 16, 100, mod_num, q, float(2 ** 33), seed=20 + mod_num) == 1
    assert dev.pcmm_context.info("last_DW") == 4


@pytest.mark.parametrize("wide", [False, True])
def test_ppmm_plaintext_digit_edge(wide):
    """d balanced base-256 digits reach +-0x7f..7f, not 2^(8d-1) - 1: a plaintext entry of 0x7f7f7f stays on three digits, 0x7f7f80
    needs four (with 7-digit residues that means two slices of three digits); both must come out right, on whole rows of such entries."""
    q = REF_PARAMS[16]["q"][:2] if wide else CFG2_Q[:2]
    pair, dev, orc, rank = make(10, 128, list(q) + CFG2_Q[2:3], CFG3_P[:1], [CFG3_P[0]], list(q))
    C = (rank + 1) * 128
    M, Kin, scaler = 16, 64, float(2 ** 20)
    mlwe = [limbs_uniform(700 + n, q, 1, C)[0] for n in range(Kin)]
    for edge, want_dw in ((0x7F7F7F, 3), (0x7F7F80, 4)):
        W = np.zeros((M, Kin), dtype=np.float32)
        W[0, :] = edge / 2.0 ** 20
        W[1, :] = -edge / 2.0 ** 20
        W[2, ::2] = edge / 2.0 ** 20
        want = np.zeros((M, 2, C), dtype=np.uint64)
        orc.PPMM(W, [m.reshape(-1) for m in mlwe], want.reshape(-1), M, Kin, 2, scaler)
        dout = DeviceBuffer(want.nbytes)
        dev.PPMM(DeviceBuffer.from_numpy(W), [to_dev(m) for m in mlwe], dout, M, Kin, 128, Kin, 2, scaler)
        assert dev.pcmm_context.info("last_absmax") == edge and dev.pcmm_context.info("last_DW") == want_dw
        assert dev.pcmm_context.info("last_path") == 1
        assert dev.pcmm_context.info("last_slices") == (2 if wide and want_dw == 4 else 1)     # 7-digit residues: two slices of three digits
        assert np.array_equal(from_dev(dout, want.shape), want)


@pytest.mark.parametrize("wide", [False, True])
def test_ppmm_narrower_matrix_after_a_wider_one(wide):
    """The same context and shape called with plaintext matrices of 3, then 2, then 1, then 2 balanced digits: the kernel instance
    reads three digit planes whatever the matrix needs, so the planes above the measured width must be rewritten (to zero) on
    every call and not keep the digits of the call before."""
    q = REF_PARAMS[16]["q"][:2] if wide else CFG2_Q[:2]
    pair, dev, orc, rank = make(10, 128, list(q) + CFG2_Q[2:3], CFG3_P[:1], [CFG3_P[0]], list(q))
    for step, (scaler, want_dw) in enumerate(((float(2 ** 26), 3), (float(2 ** 17), 2), (float(2 ** 9), 1), (float(2 ** 18), 2))):
        assert run_ppmm(dev, orc, rank, 128, 40, 70, 2, q, scaler, seed=300 + step) == 1
        assert dev.pcmm_context.info("last_DW") == want_dw, (step, dev.pcmm_context.info("last_absmax"))


def test_ppmm_reference_form_on_mlwe_ciphertexts():
    """PCMM_Scheme::PPMM as the reference declares it: the scaler from the first operand's scale (PPMM_kernel.cuh:283-284), every
    ring-pack modulus, rows copied back into the MLWE ciphertexts and their scale updated (:345-348); fewer rows than operands and
    more rows than operands."""
    from ckks_llm_amd import MLWECiphertext
    q = CFG2_Q[:2]
    pair, dev, orc, rank = make(10, 128, list(q) + CFG2_Q[2:3], CFG3_P[:1], [CFG3_P[0]], list(q))
    dev.ppmm_target_scale = float(1 << 26)            # 36-bit moduli: rows must stay below q_ringpack[0] / 2
    C = (rank + 1) * 128
    rng = np.random.default_rng(5)
    for M, Kin in ((24, 40), (48, 16)):
        W = rng.normal(0, 0.02, (M, Kin)).astype(np.float32)
        scale = float(1 << 30)
        host = [limbs_uniform(50 + n, q, 1, C)[0] for n in range(Kin)]
        mlwe = []
        for n in range(Kin):
            m = MLWECiphertext(128, 1, 1, rank, scale)
            m.cipher_device.upload(host[n])
            mlwe.append(m)
        scaler = int(q[1] * float(1 << 26) / scale)
        want = np.zeros((M, 2, C), dtype=np.uint64)
        orc.PPMM(W, [h.reshape(-1) for h in host], want.reshape(-1), M, Kin, 2, float(scaler))
        dev.PPMM(DeviceBuffer.from_numpy(W), mlwe, M, Kin, 128, Kin)
        assert dev.last_scaler == scaler
        assert np.array_equal(dev.ppmm_output.download(np.uint64, want.size).reshape(want.shape), want)
        for i in range(Kin):
            got = mlwe[i].cipher_device.download(np.uint64).reshape(2, C)
            if i < min(M, Kin):
                assert np.array_equal(got[0], want[i, 0]) and np.array_equal(got[1], host[i][1])      # first modulus replaced, second untouched
                assert mlwe[i].scale == scale * scaler / q[1]
            else:
                assert np.array_equal(got, host[i]) and mlwe[i].scale == scale
    with pytest.raises(ValueError):
        dev.PPMM(DeviceBuffer.from_numpy(W), mlwe, M, Kin, 64, Kin)


def test_ppmm_reads_the_weights_in_every_call_unless_declared_static():
    """As the reference (PPMM_kernel.cuh:148 quantises W inside the call), a PPMM call multiplies by what the weight buffer holds
    when the call is made, also when a writer the library cannot see (a raw HIP copy here) has changed it.  A matrix declared
    static keeps its digit planes under (device address, shape, scaler): a second call reuses them; a matrix overwritten through
    the library's copy, a freed and reallocated buffer, an announced in-place change and a withdrawn declaration must all give
    the product of what the buffer holds now."""
    import ctypes
    q = CFG2_Q[:2]
    pair, dev, orc, rank = make(10, 128, list(q) + CFG2_Q[2:3], CFG3_P[:1], [CFG3_P[0]], list(q))
    C = (rank + 1) * 128
    M, Kin, scaler = 32, 64, float(2 ** 26)
    rng = np.random.default_rng(77)
    mlwe = [limbs_uniform(900 + n, q, 1, C)[0] for n in range(Kin)]
    bufs = [to_dev(m) for m in mlwe]
    hip = ctypes.CDLL("/opt/rocm/lib/libamdhip64.so")

    def raw_copy(dst, src, nbytes):                                   # device to device, not through the library
        assert hip.hipMemcpy(ctypes.c_void_p(dst.ptr), ctypes.c_void_p(src.ptr), ctypes.c_size_t(nbytes), 3) == 0

    def want_for(W):
        out = np.zeros((M, 2, C), dtype=np.uint64)
        orc.PPMM(W, [m.reshape(-1) for m in mlwe], out.reshape(-1), M, Kin, 2, scaler)
        return out

    def run(dW):
        dout = DeviceBuffer(8 * M * 2 * C)
        dout.zero()
        dev.PPMM(dW, bufs, dout, M, Kin, 128, Kin, 2, scaler)
        return from_dev(dout, (M, 2, C))

    W1 = rng.normal(0, 0.02, (M, Kin)).astype(np.float32)
    W2 = rng.normal(0, 0.02, (M, Kin)).astype(np.float32)
    W3 = rng.normal(0, 0.3, (M, Kin)).astype(np.float32)             # four plaintext digits: another kernel instance
    pc = dev.pcmm_context
    # default settings: nothing is kept
    dW = DeviceBuffer.from_numpy(W1)
    second, third = DeviceBuffer.from_numpy(W2), DeviceBuffer.from_numpy(W3)
    assert np.array_equal(run(dW), want_for(W1))
    raw_copy(dW, second, W2.nbytes)
    assert np.array_equal(run(dW), want_for(W2))                      # the new weights, unannounced
    raw_copy(dW, third, W3.nbytes)
    assert np.array_equal(run(dW), want_for(W3)) and pc.info("last_DW") == 4
    dW.upload(W1)
    assert np.array_equal(run(dW), want_for(W1)) and pc.info("last_DW") == 3
    # declared static: planes kept
    for declare in ("matrix", "handle"):
        if declare == "matrix":
            pc.weights_static(dW)
        else:
            pc.set_weight_cache(True)
        dW.upload(W1)
        assert np.array_equal(run(dW), want_for(W1))
        assert np.array_equal(run(dW), want_for(W1))                  # prepared planes
        raw_copy(dW, second, W2.nbytes)
        assert np.array_equal(run(dW), want_for(W1))                  # the promise was broken: the kept planes answer (documented)
        pc.weights_changed(dW)                                        # ... until the change is announced
        assert np.array_equal(run(dW), want_for(W2))
        dW.upload(W3)                                                 # overwritten in place through the library
        assert np.array_equal(run(dW), want_for(W3)) and pc.info("last_DW") == 4
        addr = dW.ptr
        dW.free()                                                     # ends the declaration of the matrix, drops its planes
        dW = DeviceBuffer.from_numpy(W1)                              # usually the same address again
        assert np.array_equal(run(dW), want_for(W1)), ("reallocated at the same address", dW.ptr == addr)
        if declare == "matrix":
            raw_copy(dW, second, W2.nbytes)
            assert np.array_equal(run(dW), want_for(W2))              # not static any more: read afresh
            pc.weights_static(dW)
            assert np.array_equal(run(dW), want_for(W2))
            pc.weights_static(dW, is_static=False)
        else:
            pc.set_weight_cache(False)
        raw_copy(dW, third, W3.nbytes)
        assert np.array_equal(run(dW), want_for(W3))                  # declaration withdrawn: every call reads the matrix


@pytest.mark.parametrize("wide", [False, True])
def test_ppmm_random_shapes_on_one_context(wide):
    """One context, a sequence of calls with random row counts, depths, modulus counts and plaintext magnitudes (1 to 4 digits),
    extreme plaintext rows and residues in every call: whatever the work space holds from the call before must not reach the next."""
    qs = REF_PARAMS[16]["q"][:3] if wide else CFG2_Q[:3]
    p_sp = REF_PARAMS[16]["p"][0] if wide else CFG3_P[0]
    pair, dev, orc, rank = make(10, 64, list(qs) + [REF_PARAMS[16]["q"][3] if wide else CFG2_Q[3]], [p_sp], [p_sp], list(qs))
    N1, scaler = 64, float(2 ** 20)
    C = (rank + 1) * N1
    rng = np.random.default_rng(777 + wide)
    widths = set()
    # up to 34 bits against the 36-bit primes (two slices of three digits), up to 48 against the 49-bit ones (three slices)
    for it, bits in enumerate((22, 12, 47, 7, 30, 15, 23, 9, 40, 13) if wide else (22, 12, 34, 7, 15, 29, 9, 33, 18, 13)):
        mod_num, M, Kin = int(rng.integers(1, 4)), int(rng.integers(4, 200)), int(rng.integers(1, 260))
        amax = (1 << bits) - 1
        W = (rng.integers(-amax, amax + 1, (M, Kin)) / scaler).astype(np.float32)
        W[0, :], W[1, :], W[2, :] = np.float32(amax / scaler), np.float32(-amax / scaler), 0
        q = qs[:mod_num]
        mlwe = [limbs_uniform(5000 + 300 * it + n, q, 1, C)[0] for n in range(Kin)]
        for j in range(mod_num):
            edge = [0, 1, q[j] - 1, (q[j] - 1) // 2, (q[j] + 1) // 2]
            for n in range(Kin):
                for t, v in enumerate(edge):
                    mlwe[n][j][(7 * t + 3) % C] = v
                    mlwe[n][j][C - 1 - t] = edge[(t + n) % 5]
        want = np.zeros((M, mod_num, C), dtype=np.uint64)
        orc.PPMM(W, [m.reshape(-1) for m in mlwe], want.reshape(-1), M, Kin, mod_num, scaler)
        dout = DeviceBuffer(want.nbytes)
        bufs = [to_dev(m) for m in mlwe]
        dev.PPMM(DeviceBuffer.from_numpy(W), bufs, dout, M, Kin, N1, Kin, mod_num, scaler)
        widths.add(dev.pcmm_context.info("last_DW"))
        assert np.array_equal(from_dev(dout, want.shape), want), (it, bits, M, Kin, mod_num, dev.pcmm_context.info("last_path"))
        for b in bufs + [dout]:
            b.free()
    assert widths >= ({1, 2, 3, 4, 6, 7} if wide else {1, 2, 3, 4, 5})


def test_ppmm_reference_shape_50bit_primes():
    """The reference's own shape: two 50-bit ring-pack primes {q0, q1}, p_ringpack = {p_last}
    (test_rlwe_decomp.cu:36-49), scaler = q1 * 2^49 / scale (PPMM_kernel.cuh:283-284).  Residues of up to 50 bits take the MFMA
    kernel with 7 digits, in one launch as long as the plaintext matrix fits 3 digits and in slices of three digits beyond."""
    P = REF_PARAMS[15]
    q = P["q"][:2]
    pair, dev, orc, rank = make(10, 128, q, P["p"][:1], [P["p"][0]], q)
    scaler = float(int(q[1] * float(2 ** 49) / float(2 ** 49)))
    assert run_ppmm(dev, orc, rank, 128, 16, 24, 2, q, float(2 ** 20), seed=5, w_std=0.1) == 1          # MFMA kernel, 7 residue digits
    assert dev.pcmm_context.info("last_DC") == 7 and dev.pcmm_context.info("last_DW") <= 3
    assert run_ppmm(dev, orc, rank, 128, 8, 8, 2, q, scaler / 2 ** 30, seed=6, w_std=0.1) == 1
    assert run_ppmm(dev, orc, rank, 128, 8, 8, 2, q, float(2 ** 33), seed=7, w_std=0.1) == 1            # |A| needs 4 digits: two slices
    assert dev.pcmm_context.info("last_slices") == 2
    # the reference's own scale: scaler = q1 * 2^49 / 2^49 (PPMM_kernel.cuh:283-284), plaintext entries of 46 bits, two slices
    assert run_ppmm(dev, orc, rank, 128, 40, 70, 2, q, scaler, seed=8, w_std=0.05) == 1
    assert dev.pcmm_context.info("last_slices") == 2 and dev.pcmm_context.info("last_DW") == 6
    assert run_ppmm(dev, orc, rank, 128, 40, 70, 2, q, scaler, seed=9, w_std=0.12) == 1                 # 48-bit entries: seven digits
    assert dev.pcmm_context.info("last_slices") == 3 and dev.pcmm_context.info("last_DW") == 7


@pytest.mark.parametrize("mod_num", [1, 2, 3])
def test_ppmm_wide_primes_with_extreme_operands(mod_num):
    """49- to 50-bit primes (the reference's logN = 16 set, some just above 2^49) through the 7-digit MFMA kernel: row and K padding,
    plaintext entries at the edge of 3 digits, residues 0, 1, q - 1, (q - 1) / 2 and (q + 1) / 2 in whole columns and whole samples."""
    q = REF_PARAMS[16]["q"][:3]
    assert max(q) > 1 << 49 and max(q) < 1 << 50
    N1, M, Kin = 128, 130, 200
    pair, dev, orc, rank = make(10, N1, q + REF_PARAMS[16]["q"][3:4], REF_PARAMS[16]["p"][:1], [REF_PARAMS[16]["p"][0]], q)
    C = (rank + 1) * N1
    rng = np.random.default_rng(40 + mod_num)
    scaler = float(2 ** 20)
    W = rng.uniform(-7.9, 7.9, (M, Kin)).astype(np.float32)
    W[3, :] = 0x7F7F7F / 2.0 ** 20                                        # the largest |A| that three balanced digits hold
    W[4, :] = -0x7F7F7F / 2.0 ** 20
    W[5, :] = 0.0
    mlwe = [limbs_uniform(900 + n, q[:mod_num], 1, C)[0] for n in range(Kin)]
    for j in range(mod_num):
        edge = [0, 1, q[j] - 1, (q[j] - 1) // 2, (q[j] + 1) // 2]
        for n in range(Kin):
            for t, v in enumerate(edge):
                mlwe[n][j][64 * t + 3] = v                                # whole columns of one edge value
                mlwe[n][j][C - 1 - t] = edge[(t + n) % 5]                 # mixed along K
        for t, v in enumerate(edge):
            mlwe[7 + t][j][:] = v                                         # whole samples
    want = np.zeros((M, mod_num, C), dtype=np.uint64)
    orc.PPMM(W, [m.reshape(-1) for m in mlwe], want.reshape(-1), M, Kin, mod_num, scaler)
    dout = DeviceBuffer(want.nbytes)
    dev.PPMM(DeviceBuffer.from_numpy(W), [to_dev(m) for m in mlwe], dout, M, Kin, N1, Kin, mod_num, scaler)
    assert dev.pcmm_context.info("last_path") == 1 and dev.pcmm_context.info("last_DC") == 7 and dev.pcmm_context.info("last_DW") == 3
    assert np.array_equal(from_dev(dout, want.shape), want)


def test_ppmm_shape_errors():
    q = CFG2_Q[:2]
    pair, dev, orc, rank = make(10, 128, q, [], [], q)
    with pytest.raises(ValueError):
        dev.PPMM(0, [], 0, 4, 4, 64, 4, 2, 1.0)            # mat_K != N1  (PPMM_kernel.cuh:256-259)
    with pytest.raises(ValueError):
        dev.PPMM(0, [], 0, 4, 4, 128, 5, 2, 1.0)           # mat_N != mlwe_num (:260-263)


@pytest.mark.parametrize("logN,N1,mlwe_num,primes", [(12, 128, 32, "36"), (12, 128, 8, "36"), (10, 64, 16, "36"), (16, 128, 512, "36"),
                                                     (16, 128, 64, "36"), (16, 256, 256, "36"), (16, 64, 1024, "36"), (16, 4096, 16, "36"),
                                                     (16, 128, 512, "49"), (16, 128, 128, "49"), (16, 256, 256, "36/49"), (16, 64, 1024, "49"),
                                                     (12, 128, 32, "49")])
def test_mlwe_packing(logN, N1, mlwe_num, primes):
    """mlweCipherPacking through the C ABI against the oracle: embedding, lift to the special prime, NTT, inner product with the
    repacking keys, iNTT, division by the special prime, + (0, b), NTT - bit-exact on random samples and random keys (the
    oracle itself is pinned by a decrypt identity with real keys).  On 36-bit primes, on the reference's own 49-bit special prime
    and moduli (at N = 2^16 the stage-fused launches then hand whole limbs over instead of the 5-byte form and balance their sums
    every few terms), and on a 36-bit special prime under 49-bit moduli."""
    p0 = REF_PARAMS[16]["p"][0] if primes == "49" else CFG3_P[0]
    q = CFG2_Q[:2] if primes == "36" else REF_PARAMS[16]["q"][:2]
    pair, dev, orc, rank = make(logN, N1, q, [p0], [p0], q)
    N = pair.N
    assert rank % mlwe_num == 0
    rng = np.random.default_rng(logN * 1000 + mlwe_num)
    mlwe = [rng.integers(0, q[0], size=(1, rank + 1, N1), dtype=np.uint64) for _ in range(mlwe_num)]
    for m in mlwe[:2]:
        m[0, :, 0] = q[0] - 1                              # largest residues: the lift's upper branch
        m[0, :, 1] = q[0] // 2 + 1
        m[0, :, 2] = q[0] // 2
    keys = np.empty((rank, 4, N), dtype=np.uint64)
    for j, pr in enumerate((p0, q[0], p0, q[0])):
        keys[:, j, :] = rng.integers(0, pr, size=(rank, N), dtype=np.uint64)
    want = np.zeros((2, 2, N), dtype=np.uint64)
    orc.mlweCipherPacking(want.reshape(-1), [m.reshape(-1) for m in mlwe], keys.reshape(-1))
    bufs = [DeviceBuffer.from_numpy(m) for m in mlwe]
    dkeys = DeviceBuffer.from_numpy(keys)
    dout = DeviceBuffer(want.nbytes); dout.zero()
    embed, mult = DeviceBuffer(8 * (rank + 1) * 2 * N), DeviceBuffer(8 * 4 * N)
    dev.mlweCipherPacking(dout, bufs, mlwe_num, 0, dkeys, embed, mult)
    got = dout.download(np.uint64).reshape(want.shape)
    assert np.array_equal(got[:, 0], want[:, 0])
    assert not got[:, 1].any()                             # limbs above the level are not touched


def test_mlwe_packing_errors():
    from ckks_llm_amd import CkksError
    q = CFG2_Q[:3]
    pair, dev, orc, rank = make(10, 64, q, CFG3_P[:1], [CFG3_P[0]], q)          # three ring-pack moduli: not supported
    b = DeviceBuffer(8 * 17 * 64)
    big = DeviceBuffer(8 * 17 * 2 * 1024)
    with pytest.raises(CkksError):
        dev.mlweCipherPacking(big, [b], 1, 0, big, big, big)
    pair, dev, orc, rank = make(10, 64, q[:2], CFG3_P[:1], [CFG3_P[0]], q[:2])
    with pytest.raises(CkksError):
        dev.mlweCipherPacking(big, [b] * 3, 3, 0, big, big, big)                  # 3 does not divide the rank


@pytest.mark.parametrize("N1", [16, 64, 128, 256, 1024])
def test_small_ring_ntt(N1):
    """PCMM_Context::ToNTTInplace / FromNTTInplace: size-N1 transforms over the ring-pack primes in the reference's
    [batch][mod][poly][N1] layout against the oracle (N1 < 256, the BERT layer's token-count ring among them, runs a kernel of its
    own), and the error for a modulus range outside the ring-pack primes."""
    from ckks_llm_amd import CkksError
    q = CFG2_Q[:3]
    pair, dev, orc, rank = make(12, N1, q, CFG3_P[:1], [CFG3_P[0]], q[:2])
    pq = [CFG3_P[0]] + q[:2]
    rng = np.random.default_rng(N1)
    batch, mod_num, polys = 2, 2, 5
    data = np.empty((batch, mod_num, polys, N1), dtype=np.uint64)
    for j in range(mod_num):
        data[:, j] = rng.integers(0, pq[1 + j], (batch, polys, N1), dtype=np.uint64)
    want = data.copy()
    orc.ToNTTInplace(want.reshape(-1), polys, mod_num, 0, 1, batch)
    d = to_dev(data)
    dev.pcmm_context.ToNTTInplace(d, polys, mod_num, 0, 1, batch)
    assert np.array_equal(from_dev(d, data.shape), want)
    dev.pcmm_context.FromNTTInplace(d, polys, mod_num, 0, 1, batch)
    assert np.array_equal(from_dev(d, data.shape), data)
    with pytest.raises(CkksError):
        dev.pcmm_context.ToNTTInplace(d, polys, 3, 0, 1, batch)              # moduli 1..3 of three


@pytest.mark.parametrize("M,Kin,wide", [(768, 768, False), (4096, 4096, False), (768, 768, True)])
def test_ppmm_full_size_sampled_against_oracle(M, Kin, wide):
    """BASELINE configs 4 and 5 at their real shape (N = 2^16, N1 = 128, rank 512, C = 65,664 columns, 12 primes below 2^36, W ~ N(0, 0.02)
    at scale 2^26): the whole product runs on the device; 24 rows of W over four column panels (the first columns, a panel inside the a
    part that straddles a 64-column tile edge, a panel in the first and the last columns of the b part) are recomputed by the oracle with the full contraction length
    and compared on every modulus.  Operands: 16 distinct seeded samples, repeated."""
    L, N1 = (2, 128) if wide else (12, 128)
    primes = REF_PARAMS[16]["q"][:2] if wide else CFG2_Q[:L]          # wide: the reference's own two 49-bit ring-pack moduli
    pair = Pair(16, [], primes)
    rank = pair.N // N1
    C = (rank + 1) * N1
    dev = PCMM_Scheme(PCMM_Context(N1, rank, [], primes, pair.dev))
    orc = O.OraclePCMM(pair.orc, N1, rank, [], primes)
    rng = np.random.default_rng(M)
    W = rng.normal(0, 0.02, (M, Kin)).astype(np.float32)
    seeds, dseeds = [], []
    for s in range(16):
        a = np.empty((L, C), dtype=np.uint64)
        for j, q in enumerate(primes):
            a[j] = rng.integers(0, q, C, dtype=np.uint64)
        seeds.append(a)
        dseeds.append(to_dev(a))
    per = 8 * L * C
    bufs = []
    for n in range(Kin):
        b = DeviceBuffer(per)
        b.L_.ckks_memcpy_d2d(b.ptr, dseeds[n % 16].ptr, per)
        bufs.append(b)
    dout = DeviceBuffer(8 * M * L * C)
    scaler = float(2 ** 26)
    dev.PPMM(DeviceBuffer.from_numpy(W), bufs, dout, M, Kin, N1, Kin, L, scaler)
    assert dev.pcmm_context.info("last_path") == 1 and dev.pcmm_context.info("last_DW") == 3
    assert dev.pcmm_context.info("last_DC") == (7 if wide else 5)
    rows = sorted(set([0, M - 1, 127, 128] + [int(v) for v in rng.integers(0, M, 20)]))
    Wsub = np.ascontiguousarray(W[rows])
    mlwe = [seeds[n % 16].reshape(-1) for n in range(Kin)]
    want = np.zeros((len(rows), L, C), dtype=np.uint64)             # only the panel columns get touched
    panels = [(0, 8), (60, 8), (1024 * 64 + 30, 8), (C - 8, 8)]     # the last two lie in the column panels whose tiles are cut into jobs by prime
    for c0, cnt in panels:
        orc.PPMM(Wsub, mlwe, want.reshape(-1), len(rows), Kin, L, scaler, c0, cnt)
    for r, m in enumerate(rows):
        for j in range(L):
            for c0, cnt in panels:
                got = dout.download(np.uint64, cnt, 8 * ((m * L + j) * C + c0))
                assert np.array_equal(got, want[r, j, c0:c0 + cnt]), (m, j, c0)
    for b in bufs + dseeds + [dout]:
        b.free()


@pytest.mark.parametrize("logN,N1,L,parts", [(13, 128, 2, [(64, 0, 64)]), (14, 64, 3, [(256, 0, 256), (128, 256, 128), (256, 384, 64)]),
                                             (16, 128, 12, [(512, 0, 512), (256, 512, 256)]), (16, 128, 2, [(512, 0, 512), (512, 512, 256)])])
def test_gather_to_digit_planes_equals_decompose_then_ppmm(logN, N1, L, parts):
    """pcmm_packed_begin / pcmm_rlwe_decompose_packed / pcmm_ppmm_packed against the two-step path on the same ciphertexts (and through it against
    the oracle, which pins that path): bit-identical outputs.  parts = (samples extracted from a ciphertext, offset, how many of them are used);
    the third shape is BASELINE config 4 (768 samples from two ciphertexts, the second with every other sample), the fourth the reference layer's
    choice (Bert.cuh:411-412, 420: 512 + 512 extracted, the first 768 multiplied)."""
    from ckks_llm_amd import CkksError
    primes = CFG2_Q[:L]
    pair = Pair(logN, [], primes)
    N = pair.N
    rank = N // N1
    C = (rank + 1) * N1
    dev = PCMM_Scheme(PCMM_Context(N1, rank, [], primes, pair.dev))
    Kin = sum(t for _, _, t in parts)
    M = 96 if logN < 16 else 768
    rng = np.random.default_rng(logN)
    W = rng.normal(0, 0.02, (M, Kin)).astype(np.float32)
    dW = DeviceBuffer.from_numpy(W)
    cts = [to_dev(limbs_uniform(100 + i, primes, 2, N)) for i in range(len(parts))]
    before = [from_dev(c, (2, L, N)) for c in cts]
    scaler = float(2 ** 26)
    # two-step path
    bufs = []
    for (n, off, take), ct in zip(parts, cts):
        part = [DeviceBuffer(8 * L * C) for _ in range(n)]
        dev.rlweCipherDecompose(ct, part, n, 0, L - 1)
        bufs += part[:take]
    want = DeviceBuffer(8 * M * L * C)
    dev.PPMM(dW, bufs, want, M, Kin, N1, Kin, L, scaler)
    assert dev.pcmm_context.info("last_path") == 1
    with pytest.raises(ValueError):
        dev.PPMM_packed(dW, want, M, scaler)                               # the planes are not open
    want_host = want.download()
    # fused path
    got = DeviceBuffer(8 * M * L * C)
    got.zero()
    dev.packed_begin(Kin, L)
    for (n, off, take), ct in zip(parts, cts):
        dev.rlweCipherDecompose_packed(ct, n, off, L - 1, take)
    dev.PPMM_packed(dW, got, M, scaler)
    assert np.array_equal(got.download(), want_host)
    for c, b in zip(cts, before):
        assert np.array_equal(from_dev(c, b.shape), b)                     # the ciphertexts are back in the NTT domain, unchanged
    with pytest.raises(CkksError):
        dev.rlweCipherDecompose_packed(cts[0], 48, 0, L - 1)               # not a multiple of 64
    with pytest.raises(CkksError):
        dev.rlweCipherDecompose_packed(cts[0], parts[0][0], Kin, L - 1, 64)  # beyond the opened shape
    for b in bufs + cts + [want, got, dW]:
        b.free()
