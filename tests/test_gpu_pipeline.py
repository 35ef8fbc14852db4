"""GPU end-to-end check of the ring-packed PCMM pipeline through the C ABI, the way the reference's test_rlwe_decomp.cu runs it
(encrypt, rlweCipherDecompose, PPMM, mlweCipherPacking, decrypt, compare with the plaintext product, :92-98,195): the decrypted
coefficients must be the matrix product of W with the coefficient-packed message, up to the scheme's rounding and noise.
Key generation, encryption and decryption are plain host arithmetic here (they are not on the GPU path)."""
import os

import numpy as np
import pytest

from ckks_llm_amd import Context_23, DeviceBuffer, PCMM_Context, PCMM_Scheme
from tests.helpers import negacyclic_mul, precision_table
from tests.params import CFG2_Q, CFG3_P

pytestmark = pytest.mark.gpu


def centred(v, q):
    v %= q
    return v - q if v > q // 2 else v


@pytest.mark.parametrize("mlwe_num", [16, 4])
def test_encrypt_decompose_ppmm_pack_decrypt(mlwe_num):
    logN, N, N1, k = 10, 1024, 64, 16
    P0, Q0, Q1 = CFG3_P[0], CFG2_Q[0], CFG2_Q[1]
    gap = k // mlwe_num
    ctx = Context_23(logN, [P0], [Q0, Q1])
    sch = PCMM_Scheme(PCMM_Context(N1, k, [P0], [Q0, Q1], ctx))
    rng = np.random.default_rng(7 + mlwe_num)
    s = [int(v) for v in rng.integers(-1, 2, N)]
    mu = [int(v) for v in rng.integers(-(1 << 30), 1 << 30, N)]
    # ---- encrypt at level 1 (primes Q0, Q1), decryption convention mu = a*s + b (Scheme_23.cuh:125-126) ----
    ct = np.zeros((2, 2, N), dtype=np.uint64)
    e = [int(v) for v in rng.integers(-3, 4, N)]                            # one noise polynomial, reduced modulo every prime
    for j, q in enumerate((Q0, Q1)):
        a = [int(v) for v in rng.integers(0, q, N)]
        a_s = negacyclic_mul(a, [v % q for v in s], q)
        ct[0, j] = a
        ct[1, j] = [(m + ee - x) % q for m, ee, x in zip(mu, e, a_s)]
    d_ct = DeviceBuffer.from_numpy(ct)
    ctx.ToNTTInplace(d_ct, 0, 1, 2, 2, 2)                                   # primes 1, 2 of [P0 | Q0 Q1]
    # ---- repacking keys over [P0 | Q0]: key_i = (a_i, -a_i*s + P0*iota(s_i) + e_i), s_i[n] = s[i + n*k] (PCMM_Scheme.cuh:128-224) ----
    keys = np.zeros((k, 2, 2, N), dtype=np.uint64)
    for i in range(k):
        iota = [0] * N
        for n in range(N1):
            iota[n * k] = s[i + n * k]
        ek = [int(v) for v in rng.integers(-3, 4, N)]
        for j, q in enumerate((P0, Q0)):
            ai = [int(v) for v in rng.integers(0, q, N)]
            ais = negacyclic_mul(ai, [v % q for v in s], q)
            keys[i, 0, j] = ai
            keys[i, 1, j] = [(-x + P0 * t + ee) % q for x, t, ee in zip(ais, iota, ek)]
    d_keys = DeviceBuffer.from_numpy(keys)
    ctx.ToNTTInplace(d_keys, 0, 0, 2 * k, 2, 2)                             # primes 0, 1
    # ---- GPU pipeline ----
    C = (k + 1) * N1
    samples = [DeviceBuffer(8 * 2 * C) for _ in range(mlwe_num)]
    sch.rlweCipherDecompose(d_ct, samples, mlwe_num, 0, 1)
    M = Kin = mlwe_num
    W = rng.normal(0, 0.02, (M, Kin)).astype(np.float32)
    scaler = float(1 << 26)
    d_out = DeviceBuffer(8 * M * 2 * C)
    sch.PPMM(DeviceBuffer.from_numpy(W), samples, d_out, M, Kin, N1, Kin, 2, scaler)
    assert sch.pcmm_context.info("last_path") == 1                           # the MFMA kernel ran
    rows = [DeviceBuffer(8 * C) for _ in range(M)]                           # row m, first modulus (PPMM_kernel.cuh:345-348)
    for m in range(M):
        rows[m].L_.ckks_memcpy_d2d(rows[m].ptr, d_out.ptr + 8 * m * 2 * C, 8 * C)
    d_res = DeviceBuffer(8 * 2 * 2 * N)
    d_res.zero()
    embed, mult = DeviceBuffer(8 * (k + 1) * 2 * N), DeviceBuffer(8 * 4 * N)
    sch.mlweCipherPacking(d_res, rows, M, 0, d_keys, embed, mult)
    ctx.FromNTTInplace(d_res, 0, 1, 2, 1, 2)                                 # limb 0 (prime Q0) of both polynomials
    res = d_res.download(np.uint64).reshape(2, 2, N)
    # ---- decrypt and compare with the plaintext product ----
    a2, b2 = [int(v) for v in res[0, 0]], [int(v) for v in res[1, 0]]
    dec = [centred(x + y, Q0) for x, y in zip(negacyclic_mul(a2, [v % Q0 for v in s], Q0), b2)]
    A = [[int(np.float64(W[m, n]) * scaler) for n in range(Kin)] for m in range(M)]     # the reference's quantisation (:148)
    worst, biggest = 0, 0
    for g in range(N1):
        for m in range(M):
            exact = sum(A[m][n] * mu[n * gap + g * k] for n in range(Kin))             # sample n holds mu[n*gap + g*k]
            want = exact // Q1                                                            # fused rescale by the last prime
            pos = g * k + m * gap
            worst = max(worst, abs(dec[pos] - want))
            biggest = max(biggest, abs(want))
    # positions that no packed sample covers decrypt to rounding noise only
    if gap > 1:
        assert max(abs(dec[p]) for p in range(N) if (p % k) % gap) <= 16 * N
    assert biggest > 1 << 15                                                  # the check is not vacuous
    # rescale and ModDown rounding are O(N); the key noise contributes sum_i a_i * e_i / P0, about sqrt(k * N) * Q0 / P0 * 3
    assert worst <= 16 * N, (worst, biggest)


@pytest.mark.parametrize("activations", ["normal", "reference_file"])
def test_bert_base_layer_on_encrypted_activations(activations):
    """BASELINE config 4 end to end at its real ring: 128 tokens x 768 activations ~ N(0, 1), coefficient-packed into two RLWE ciphertexts at
    N = 2^16 (ternary secret of weight 192, Gaussian error 3.2, public-key encryption), times W 768 x 768 ~ N(0, 0.02), out as three ring-packed
    ciphertexts of 256 features each - the sequence of Bert::PCMM_Boot_768_768 between its slot/coefficient conversions (Bert.cuh:411-424, 473,
    482, 491) - with every key generated on the device, the gather writing PPMM's operand planes directly, and the decrypted result compared with
    the plaintext product as the reference's test program does (GetPrecisionStats, precision.cuh:104).  "reference_file" takes the activations
    from tests/golden/hidden_states.bin, the 128 x 768 fp32 BERT hidden states the reference holds for its own layer test
    (test_bert_infer.cu:117; values in [-11.1, 4.25], unlike the unit normal ones)."""
    from ckks_llm_amd import Ciphertext, MLWESecretKey, Plaintext, Scheme_23, SecretKey
    logN, N1 = 16, 128
    P0, Q0, Q1 = CFG3_P[0], CFG2_Q[0], CFG2_Q[1]
    ctx = Context_23(logN, [P0], [Q0, Q1])
    N, L = ctx.N, ctx.L
    k = N // N1
    key = bytes(range(32))
    scheme = Scheme_23(ctx, key=key)
    sk = SecretKey(ctx, h=192, key=key, nonce=1)
    pc = PCMM_Context(N1, k, [P0], [Q0, Q1], ctx)
    ps = PCMM_Scheme(pc, key=key)
    mlwe_sk = MLWESecretKey(N1, pc.ringpack_pq_count - 1, k)
    ps.convertMLWESKfromRLWESK(mlwe_sk, sk)
    scheme.addEncKey(sk)
    ps.addRepakcingKey(mlwe_sk, sk)
    rng = np.random.default_rng(4)
    tokens, feat = N1, 768
    if activations == "reference_file":
        X = np.fromfile(os.path.join(os.path.dirname(__file__), "golden", "hidden_states.bin"), dtype="<f4").astype(np.float64)
        assert X.size == tokens * feat and 11.0 < np.abs(X).max() < 11.2
        X = X.reshape(tokens, feat)
    else:
        X = rng.normal(0, 1, (tokens, feat))
    W = rng.normal(0, 0.02, (feat, feat)).astype(np.float32)
    want = X @ W.astype(np.float64).T                                      # [token][output feature]
    x_scale = 1 << 33
    cts = []
    for lo, hi in ((0, 512), (512, 768)):
        coeffs = np.zeros((tokens, k))
        coeffs[:, : hi - lo] = X[:, lo:hi]                                  # coefficient n * k + m = X[n][lo + m]
        msg = Plaintext(N, L, L, N // 2, x_scale)
        ctx.encode_coeffs(DeviceBuffer.from_numpy(coeffs.reshape(-1)), msg)
        ct = Ciphertext(N, L, L, N // 2, x_scale)
        scheme.encryptMsg(ct, msg)
        cts.append(ct)
    C = (k + 1) * N1
    scaler = float(1 << 29)
    out = DeviceBuffer(8 * feat * 2 * C)
    ps.packed_begin(feat, 2)
    ps.rlweCipherDecompose_packed(cts[0].cipher_device, 512, 0, 1)
    ps.rlweCipherDecompose_packed(cts[1].cipher_device, 512, 512, 1, take=256)
    ps.PPMM_packed(DeviceBuffer.from_numpy(W), out, feat, scaler)
    assert pc.info("last_path") == 1 and pc.info("last_DW") == 4
    rows = [DeviceBuffer(8 * C) for _ in range(feat)]
    for m in range(feat):
        rows[m].L_.ckks_memcpy_d2d(rows[m].ptr, out.ptr + 8 * m * 2 * C, 8 * C)
    out_scale = x_scale * scaler / Q1
    embed, mult = DeviceBuffer(8 * (k + 1) * 2 * N), DeviceBuffer(8 * 4 * N)
    dec, d_vals = Plaintext(N, L, 0, N // 2, 1), DeviceBuffer(8 * N)
    decrypted = np.zeros_like(want)
    for j in range(3):
        res = Ciphertext(N, L, 0, N // 2, out_scale)
        res.cipher_device.zero()
        ps.mlweCipherPacking(res.cipher_device, rows[256 * j: 256 * (j + 1)], 256, 0, ps.repackingKeys, embed, mult)
        res.l, res.scale = 0, out_scale
        scheme.decryptMsg(dec, sk, res)
        ctx.decode_coeffs(dec, d_vals)
        got = d_vals.download(np.float64).reshape(tokens, k)                # coefficient n * k + 2 m = Y[n][256 j + m]
        decrypted[:, 256 * j: 256 * (j + 1)] = got[:, 0:512:2]
        assert np.abs(got[:, 1:512:2]).max() < 2.0 ** -9                    # the positions between the packed samples hold noise only
    assert np.abs(want).max() > 1.0
    # output scale 2^26: the floor is the repacking noise over that scale
    precision_table(decrypted, want, "BERT-base 768 x 768 layer, %s activations" % activations, min_bits=12, median_bits=15)


def test_layer_on_the_references_own_parameter_set():
    """The same layer on the reference's own configuration: Context_23(16, 15, 192) (its compiled-in logN = 16 set: 28 Q and 4 P primes
    of 49 - 50 bits, 8 T primes), ring-pack primes {p_last} and {q0, q1} as its test program picks them (test_rlwe_decomp.cu:36-49),
    messages at its precision 2^49 and its scaler q1 * 2^49 / scale (PPMM_kernel.cuh:283-284), which makes the plaintext entries 45
    bits wide.  768 activations x 768 outputs, decrypted and compared with the plain product."""
    from ckks_llm_amd import Ciphertext, MLWESecretKey, Plaintext, Scheme_23, SecretKey
    ctx = Context_23(16, 15, 192)
    N, L, N1 = ctx.N, ctx.L, 128
    k = N // N1
    key = bytes(range(32))
    scheme = Scheme_23(ctx, key=key)
    sk = SecretKey(ctx, key=key, nonce=1)
    p_rp, q_rp = [ctx.pVec[-1]], [ctx.qVec[0], ctx.qVec[1]]
    pc = PCMM_Context(N1, k, p_rp, q_rp, ctx)
    ps = PCMM_Scheme(pc, key=key)
    mlwe_sk = MLWESecretKey(N1, pc.ringpack_pq_count - 1, k)
    ps.convertMLWESKfromRLWESK(mlwe_sk, sk)
    scheme.addEncKey(sk)
    ps.addRepakcingKey(mlwe_sk, sk)
    rng = np.random.default_rng(16)
    tokens, feat = N1, 768
    X = rng.normal(0, 0.05, (tokens, feat))
    W = rng.normal(0, 0.02, (feat, feat)).astype(np.float32)
    want = X @ W.astype(np.float64).T
    x_scale = ctx.precision                                                  # 2^49
    C = (k + 1) * N1
    samples = []
    for lo, hi in ((0, 512), (512, 768)):
        coeffs = np.zeros((tokens, k))
        coeffs[:, : hi - lo] = X[:, lo:hi]
        msg = Plaintext(N, L, 1, N // 2, x_scale)
        ctx.encode_coeffs(DeviceBuffer.from_numpy(coeffs.reshape(-1)), msg)
        ct = Ciphertext(N, L, 1, N // 2, x_scale)
        scheme.encryptMsg(ct, msg)
        part = [DeviceBuffer(8 * 2 * C) for _ in range(512)]
        ps.rlweCipherDecompose(ct.cipher_device, part, 512, 0, 1)
        samples += part[: hi - lo]
    scaler = float(int(q_rp[1] * float(1 << 49) / float(x_scale)))
    out = DeviceBuffer(8 * feat * 2 * C)
    ps.PPMM(DeviceBuffer.from_numpy(W), samples, out, feat, feat, N1, feat, 2, scaler)
    assert pc.info("last_path") == 1 and pc.info("last_DC") == 7 and pc.info("last_DW") == 6 and pc.info("last_slices") == 2
    rows = [DeviceBuffer(8 * C) for _ in range(feat)]
    for m in range(feat):
        rows[m].L_.ckks_memcpy_d2d(rows[m].ptr, out.ptr + 8 * m * 2 * C, 8 * C)
    out_scale = x_scale * scaler / q_rp[1]
    embed, mult = DeviceBuffer(8 * (k + 1) * 2 * N), DeviceBuffer(8 * 4 * N)
    dec, d_vals = Plaintext(N, L, 0, N // 2, 1), DeviceBuffer(8 * N)
    decrypted = np.zeros_like(want)
    for j in range(3):
        res = Ciphertext(N, L, 0, N // 2, out_scale)
        res.cipher_device.zero()
        ps.mlweCipherPacking(res.cipher_device, rows[256 * j: 256 * (j + 1)], 256, 0, ps.repackingKeys, embed, mult)
        res.l, res.scale = 0, out_scale
        scheme.decryptMsg(dec, sk, res)
        ctx.decode_coeffs(dec, d_vals)
        got = d_vals.download(np.float64).reshape(tokens, k)
        decrypted[:, 256 * j: 256 * (j + 1)] = got[:, 0:512:2]
    assert np.abs(want).max() > 0.05 and np.abs(want).max() < 0.4
    precision_table(decrypted, want, "768 x 768 layer on the reference's logN = 16 set, precision 2^49", min_bits=33, median_bits=36)


def test_bert_mirror_layers_with_loaded_weights(tmp_path):
    """The Python mirrors of Bert_model_weights and Bert: weights from a `model.safetensors` written with the safetensors package,
    PCMM_768_768 (two inputs of 512 samples) and layer_output (768 x 3072, six inputs) on encrypted activations at N = 2^16,
    decrypted and compared with the plain products."""
    from safetensors.numpy import save_file
    from ckks_llm_amd import Bert, Ciphertext, MLWESecretKey, Plaintext, Scheme_23, SecretKey
    rng = np.random.default_rng(9)
    pre = "bert.encoder.layer.0."
    tensors = {pre + "attention.self.query.weight": rng.normal(0, 0.02, (768, 768)).astype(np.float32),
               pre + "output.dense.weight": rng.normal(0, 0.02, (768, 3072)).astype(np.float32),
               pre + "output.dense.bias": rng.normal(0, 0.02, 768).astype(np.float32),
               "cls.seq_relationship.bias": np.zeros(2, np.float16)}
    save_file(tensors, str(tmp_path / "model.safetensors"))
    logN, N1 = 16, 128
    P0, Q0, Q1 = CFG3_P[0], CFG2_Q[0], CFG2_Q[1]
    ctx = Context_23(logN, [P0], [Q0, Q1])
    N, L, k = ctx.N, ctx.L, ctx.N // N1
    key = bytes(range(1, 33))
    scheme = Scheme_23(ctx, key=key)
    sk = SecretKey(ctx, h=192, key=key, nonce=1)
    pc = PCMM_Context(N1, k, [P0], [Q0, Q1], ctx)
    ps = PCMM_Scheme(pc, key=key)
    mlwe_sk = MLWESecretKey(N1, pc.ringpack_pq_count - 1, k)
    ps.convertMLWESKfromRLWESK(mlwe_sk, sk)
    scheme.addEncKey(sk)
    ps.addRepakcingKey(mlwe_sk, sk)
    bert = Bert(str(tmp_path) + "/", ctx, scheme, ps, sk, target_scale=float(1 << 26))
    w = bert.model_weights
    assert w.opened and len(w.loaded) == 3 and len(w.missing) == 14 + 16 * 12 - 3 and "cls.seq_relationship.bias" in w.missing
    assert np.array_equal(w.output_dense_bias[0].download(np.float32), tensors[pre + "output.dense.bias"])
    assert w.output_dense_bias[1] is None and w.pooler_dense_weight is None
    x_scale = 1 << 33
    d_vals = DeviceBuffer(8 * N)

    def encrypt_part(X, first, count, extract):
        coeffs = np.zeros((N1, k))
        coeffs[:, 0:count * (k // extract):k // extract] = X[:, first:first + count]
        msg = Plaintext(N, L, L, N // 2, x_scale)
        ctx.encode_coeffs(DeviceBuffer.from_numpy(coeffs.reshape(-1)), msg)
        ct = Ciphertext(N, L, L, N // 2, x_scale)
        scheme.encryptMsg(ct, msg)
        return ct

    def worst_error(ct, Y, first, count):
        dec = Plaintext(N, L, 0, N // 2, 1)
        scheme.decryptMsg(dec, sk, ct)
        ctx.decode_coeffs(dec, d_vals)
        got = d_vals.download(np.float64).reshape(N1, k)
        return np.abs(got[:, 0:count * (k // count):k // count] - Y[:, first:first + count]).max()

    X = rng.normal(0, 1, (N1, 768))
    Y = X @ tensors[pre + "attention.self.query.weight"].astype(np.float64).T
    ins = [encrypt_part(X, 0, 512, 512), encrypt_part(X, 512, 256, 512)]
    outs = [Ciphertext(N, L, 0, N // 2, 1) for _ in range(3)]
    bert.PCMM_Boot_768_768(w.attention_self_query_weight[0], ins, outs, L, 0)          # the reference's signature (Bert.h:62)
    assert max(worst_error(outs[j], Y, 256 * j, 256) for j in range(3)) < 2.0 ** -10
    X = rng.normal(0, 0.6, (N1, 3072))
    Y = X @ tensors[pre + "output.dense.weight"].astype(np.float64).T
    O = [None] * 12
    for i in range(6):
        O[2 * i] = encrypt_part(X, 512 * i, 512, 512)
    bert.layer_output(O, 0, [])                                                         # Bert.h:61; layer_res is not touched
    assert O[0].l == 0 and max(worst_error(O[0], Y, 0, 512), worst_error(O[2], Y, 512, 256)) < 2.0 ** -10


def test_llm_projection_4096_on_encrypted_activations():
    """BASELINE config 5 from encryption to decryption: 128 tokens x 4096 activations ~ N(0, 1) in eight RLWE ciphertexts of 512 samples
    at N = 2^16 (ternary secret of weight 192, Gaussian error 3.2, public-key encryption), times W 4096 x 4096 ~ N(0, 0.02) quantised at
    2^26 (three balanced int8 digits against five residue digits on the matrix cores), the 4096 product rows ring-packed into sixteen
    ciphertexts of 256 features, decrypted, decoded and compared with the plain fp64 product in the reference's unit.  Ring-pack moduli
    [p0 | q0, q1], the shape the reference's packing supports."""
    from ckks_llm_amd import Ciphertext, MLWESecretKey, Plaintext, Scheme_23, SecretKey
    logN, N1 = 16, 128
    P0, Q0, Q1 = CFG3_P[0], CFG2_Q[0], CFG2_Q[1]
    ctx = Context_23(logN, [P0], [Q0, Q1])
    N, L = ctx.N, ctx.L
    k = N // N1
    key = bytes(range(5, 37))
    scheme = Scheme_23(ctx, key=key)
    sk = SecretKey(ctx, h=192, key=key, nonce=1)
    pc = PCMM_Context(N1, k, [P0], [Q0, Q1], ctx)
    ps = PCMM_Scheme(pc, key=key)
    mlwe_sk = MLWESecretKey(N1, pc.ringpack_pq_count - 1, k)
    ps.convertMLWESKfromRLWESK(mlwe_sk, sk)
    scheme.addEncKey(sk)
    ps.addRepakcingKey(mlwe_sk, sk)
    rng = np.random.default_rng(4096)
    tokens, feat = N1, 4096
    X = rng.normal(0, 1, (tokens, feat))
    W = rng.normal(0, 0.02, (feat, feat)).astype(np.float32)
    want = X @ W.astype(np.float64).T                                      # [token][output feature]
    x_scale = 1 << 36
    C = (k + 1) * N1
    scaler = float(1 << 26)
    ps.packed_begin(feat, 2)
    for i in range(feat // 512):
        msg = Plaintext(N, L, L, N // 2, x_scale)
        ctx.encode_coeffs(DeviceBuffer.from_numpy(np.ascontiguousarray(X[:, 512 * i: 512 * (i + 1)]).reshape(-1)), msg)   # coefficient n * k + m = X[n][512 i + m]
        ct = Ciphertext(N, L, L, N // 2, x_scale)
        scheme.encryptMsg(ct, msg)
        ps.rlweCipherDecompose_packed(ct.cipher_device, 512, 512 * i, 1)
    out = DeviceBuffer(8 * feat * 2 * C)
    ps.PPMM_packed(DeviceBuffer.from_numpy(W), out, feat, scaler)
    assert pc.info("last_path") == 1 and pc.info("last_DW") == 3 and pc.info("last_DC") == 5
    rows = [out.ptr + 8 * m * 2 * C for m in range(feat)]                   # row m, first modulus (PPMM_kernel.cuh:345-348)
    out_scale = x_scale * scaler / Q1
    embed, mult = DeviceBuffer(8 * (k + 1) * 2 * N), DeviceBuffer(8 * 4 * N)
    dec, d_vals = Plaintext(N, L, 0, N // 2, 1), DeviceBuffer(8 * N)
    decrypted = np.zeros_like(want)
    res = Ciphertext(N, L, 0, N // 2, out_scale)
    for j in range(feat // 256):
        res.cipher_device.zero()
        ps.mlweCipherPacking(res.cipher_device, rows[256 * j: 256 * (j + 1)], 256, 0, ps.repackingKeys, embed, mult)
        res.l, res.scale = 0, out_scale
        scheme.decryptMsg(dec, sk, res)
        ctx.decode_coeffs(dec, d_vals)
        got = d_vals.download(np.float64).reshape(tokens, k)                # coefficient n * k + 2 m = Y[n][256 j + m]
        decrypted[:, 256 * j: 256 * (j + 1)] = got[:, 0:512:2]
    assert np.abs(want).max() > 4.0
    precision_table(decrypted, want, "Llama-7B-shaped projection 4096 x 4096", min_bits=12, median_bits=15)
