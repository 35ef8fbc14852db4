"""GPU parity of the key side of the ring-packed PCMM (MLWE secret, repacking keys, MLWE decryption and decoding) through the C ABI
against the CPU oracle, bit-exact; and the reference's own test program for this path (test_rlwe_decomp.cu) replayed through the
mirror classes with its precision check."""
import numpy as np
import pytest

from ckks_llm_amd import (CkksError, Ciphertext, Context_23, DeviceBuffer, MLWEPlaintext, MLWESecretKey, PCMM_Context, PCMM_Scheme,
                          Plaintext, Scheme_23, SecretKey)
from oracle import oracle_py as O
from tests.gpu_common import Pair, to_dev, from_dev
from tests.params import CFG2_Q, CFG3_P

pytestmark = pytest.mark.gpu

KEY = bytes(range(3, 35))


@pytest.mark.parametrize("logN,N1", [(12, 256), (13, 512), (12, 128), (11, 64)])
def test_mlwe_keys_and_decryption_match_oracle(logN, N1):
    P0, Q0, Q1 = CFG3_P[0], CFG2_Q[0], CFG2_Q[1]
    pair = Pair(logN, [P0], [Q0, Q1])
    N = pair.N
    k = N // N1
    dev_pc = PCMM_Context(N1, k, [P0], [Q0, Q1], pair.dev)
    orc_pc = O.OraclePCMM(pair.orc, N1, k, [P0], [Q0, Q1])
    L_ = pair.dev.L_
    h = 64
    sx = np.zeros((3, N), dtype=np.uint64)
    pair.orc.keygen_secret(sx.reshape(-1), O.salsa20_stream(5 * h, KEY, 1), h)
    d_sx = to_dev(sx)
    # MLWE secret
    want = np.zeros((3, k, N1), dtype=np.uint64)
    orc_pc.convertMLWESKfromRLWESK(want.reshape(-1), sx.reshape(-1))
    d_msk = to_dev(np.zeros(want.shape, dtype=np.uint64))
    assert L_.pcmm_convert_mlwe_sk(dev_pc.h, d_msk.ptr, d_sx.ptr) == 0
    assert np.array_equal(from_dev(d_msk, want.shape), want)
    assert np.array_equal(from_dev(d_sx, sx.shape), sx)                    # the RLWE secret comes back as it was
    msk = want
    # repacking keys: key i draws from the stream under nonce 100 + i
    per_key = 4 * N + 8 * N * 2
    rnd = np.concatenate([O.salsa20_stream(per_key, KEY, 100 + i) for i in range(k)])
    want = np.zeros((k, 2, 2, N), dtype=np.uint64)
    orc_pc.addRepakcingKey(want.reshape(-1), msk.reshape(-1), sx.reshape(-1), rnd)
    d_keys = to_dev(np.full(want.shape, 3, dtype=np.uint64))
    scratch = DeviceBuffer(8 * N * 3)
    assert L_.pcmm_add_repacking_key(dev_pc.h, d_keys.ptr, d_msk.ptr, d_sx.ptr, KEY, 100, scratch.ptr) == 0
    assert np.array_equal(from_dev(d_keys, want.shape), want)
    assert np.array_equal(from_dev(d_msk, msk.shape), msk)                 # every modulus of the MLWE secret is back in the NTT domain
    # MLWE decryption and decoding of random samples at both levels
    rng = np.random.default_rng(logN)
    for l in (1, 0):
        sample = np.zeros((2, k + 1, N1), dtype=np.uint64)
        for j, q in enumerate((Q0, Q1)[: l + 1]):
            sample[j] = rng.integers(0, q, (k + 1, N1), dtype=np.uint64)
        plain = np.zeros((2, N1), dtype=np.uint64)
        orc_pc.mlweDecrypt(plain.reshape(-1), sample.reshape(-1), msk.reshape(-1), l)
        d_sample, d_plain = to_dev(sample), to_dev(np.zeros((2, N1), dtype=np.uint64))
        assert L_.pcmm_mlwe_decrypt(dev_pc.h, d_plain.ptr, d_sample.ptr, d_msk.ptr, l) == 0
        assert np.array_equal(from_dev(d_plain, plain.shape)[: l + 1], plain[: l + 1])
        assert np.array_equal(from_dev(d_sample, sample.shape), sample)
        vals = orc_pc.decodeCoeffs(plain.reshape(-1), 1 << 20, l)
        d_vals = DeviceBuffer(8 * N1)
        assert L_.pcmm_decode_coeffs(dev_pc.h, d_vals.ptr, d_plain.ptr, scratch.ptr, 1 << 20, l) == 0
        assert np.array_equal(d_vals.download(np.float64), vals)
    assert L_.pcmm_mlwe_decrypt(dev_pc.h, d_plain.ptr, d_sample.ptr, d_msk.ptr, 2) != 0
    odd = PCMM_Context(32, N // 32, [P0], [Q0, Q1], pair.dev)
    assert L_.pcmm_convert_mlwe_sk(odd.h, d_msk.ptr, d_sx.ptr) != 0        # N1 = 32: the key side needs a multiple of 64


def test_reference_test_program_flow():
    """test_rlwe_decomp.cu:23-198 with the reference's object names: keys, encode_coeffs, encryptMsg, rlweCipherDecompose, mlweDecrypt of a
    sample, PPMM, mlweCipherPacking, decryptMsg, decode_coeffs; the result is compared with the plain product the program computes
    (:86-92), as its GetPrecisionStats call does (:195)."""
    logN, PCMM_N1 = 12, 256
    P0, Q0, Q1 = CFG3_P[0], CFG2_Q[0], CFG2_Q[1]
    context = Context_23(logN, [P0], [Q0, Q1])
    scheme = Scheme_23(context, key=KEY)
    N, L, slots = context.N, context.L, context.N // 2
    mlwe_rank = N // PCMM_N1
    p_ringpack, q_ringpack = [context.pVec[context.p_num - 1]], [context.qVec[0], context.qVec[1]]
    sk = SecretKey(context, h=192, key=KEY, nonce=9)
    pcmm_context = PCMM_Context(PCMM_N1, mlwe_rank, p_ringpack, q_ringpack, context)
    pcmm_scheme = PCMM_Scheme(pcmm_context, key=KEY)
    mlwe_sk = MLWESecretKey(PCMM_N1, pcmm_context.ringpack_pq_count - 1, mlwe_rank)
    pcmm_scheme.convertMLWESKfromRLWESK(mlwe_sk, sk)
    scheme.addEncKey(sk)
    pcmm_scheme.addRepakcingKey(mlwe_sk, sk)
    rng = np.random.default_rng(0)
    real_mes_host = rng.uniform(-0.1, 0.1, N)
    mat_M = mat_N = mlwe_rank
    plain_mat_host = rng.uniform(-0.1, 0.1, (mat_M, mat_N)).astype(np.float32)
    plain_gemm_host = np.zeros(N)
    msg_mat = real_mes_host.reshape(PCMM_N1, mat_N)                         # [idx_K][idx_N]
    plain_gemm_host.reshape(PCMM_N1, mat_M)[:] = msg_mat @ plain_mat_host.astype(np.float64).T
    precision = 1 << 28
    target_level = 1
    decomp_num = N // PCMM_N1
    C = (mlwe_rank + 1) * PCMM_N1
    mlwe_cipher_decomposed = [DeviceBuffer(8 * 2 * C) for _ in range(decomp_num)]
    plain_m1 = Plaintext(N, L, target_level, slots, precision)
    m2_dec = Plaintext(N, L, target_level, slots, precision)
    c1, c2 = Ciphertext(N, L, L, slots, precision), Ciphertext(N, L, L, slots, precision)
    context.encode_coeffs(DeviceBuffer.from_numpy(real_mes_host), plain_m1)
    scheme.encryptMsg(c1, plain_m1)
    pcmm_scheme.rlweCipherDecompose(c1.cipher_device, mlwe_cipher_decomposed, decomp_num, 0, c1.l)
    # a sample decrypts to the strided coefficients of the message (the commented-out check of the program, :143-151)
    mlwe_dec = MLWEPlaintext(PCMM_N1, 1, 1, precision)
    d_small = DeviceBuffer(8 * PCMM_N1)
    for j in (0, 5):
        pcmm_scheme.mlweDecrypt(mlwe_cipher_decomposed[j], mlwe_sk, mlwe_dec, 1)
        pcmm_context.decodeCoeffs(mlwe_dec, d_small)
        got = d_small.download(np.float64)
        assert np.abs(got - real_mes_host[j::mlwe_rank]).max() < 1e-4
    # PPMM with the reference's scale rule (PPMM_kernel.cuh:283-284, 345-348): the product lands on the scale target_scale
    target_scale = 1 << 26
    scaler = float(int(q_ringpack[1] * float(target_scale) / float(precision)))
    d_out = DeviceBuffer(8 * mat_M * 2 * C)
    pcmm_scheme.PPMM(DeviceBuffer.from_numpy(plain_mat_host), mlwe_cipher_decomposed, d_out, mat_M, mat_N, PCMM_N1, decomp_num, 2, scaler)
    assert pcmm_context.info("last_path") == 1
    rows = [DeviceBuffer(8 * C) for _ in range(mat_M)]
    for m in range(mat_M):
        rows[m].L_.ckks_memcpy_d2d(rows[m].ptr, d_out.ptr + 8 * m * 2 * C, 8 * C)
    new_scale = precision * scaler / q_ringpack[1]
    embed, mult = DeviceBuffer(8 * (mlwe_rank + 1) * 2 * N), DeviceBuffer(8 * 4 * N)
    c2.cipher_device.zero()
    pcmm_scheme.mlweCipherPacking(c2.cipher_device, rows, decomp_num, 0, pcmm_scheme.repackingKeys, embed, mult)
    c2.l, c2.scale = 0, new_scale
    scheme.decryptMsg(m2_dec, sk, c2)
    d_vals = DeviceBuffer(8 * N)
    context.decode_coeffs(m2_dec, d_vals)
    real_values_computed = d_vals.download(np.float64)
    err = np.abs(real_values_computed - plain_gemm_host)
    # GetPrecisionStats (precision.cuh:104): log2 of the inverse of the error
    assert np.abs(plain_gemm_host).max() > 0.02
    assert err.max() < 2.0 ** -12, err.max()
    assert np.median(err) < 2.0 ** -15
