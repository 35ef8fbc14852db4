"""Side measurements printed in bench.py's JSON line: PPMM at the BERT-base shape (BASELINE configs[3]) against the
int8 MFMA roofline and one textbook hybrid key switch (configs[2]) against the HBM roofline."""
import numpy as np

MFMA_I8_PEAK_MACS = 2.5166e15      # 5.033 POP/s dense int8
HBM_PEAK = 8.0e12


def bench_ppmm(P, M=768, Kin=768, N1=128, L=12, reps=3, primes=None, label=None, scaler=None):
    from ckks_llm_amd import Context_23, DeviceBuffer, PCMM_Context, PCMM_Scheme
    primes = list(primes[:L]) if primes is not None else P.CFG2_Q[:L]
    ctx = Context_23(16, [], primes)
    rank = (1 << 16) // N1
    C = (rank + 1) * N1
    sch = PCMM_Scheme(PCMM_Context(N1, rank, [], primes, ctx))
    rng = np.random.default_rng(4)
    W = rng.normal(0, 0.02, (M, Kin)).astype(np.float32)
    dW = DeviceBuffer.from_numpy(W)
    # synthetic MLWE operands: 16 distinct seeded ciphertexts of uniform residues, copied into Kin separate buffers
    seeds = []
    rng5 = np.random.default_rng(5)
    for s in range(16):
        a = np.empty((L, C), dtype=np.uint64)
        for j, q in enumerate(primes):
            a[j] = rng5.integers(0, q, C, dtype=np.uint64)
        seeds.append(DeviceBuffer.from_numpy(a))
    per = 8 * L * C
    bufs = []
    for n in range(Kin):
        b = DeviceBuffer(per)
        b.L_.ckks_memcpy_d2d(b.ptr, seeds[n % 16].ptr, per)
        bufs.append(b)
    out = DeviceBuffer(8 * M * L * C)
    scaler = float(2 ** 26) if scaler is None else float(scaler)
    sch.PPMM(dW, bufs, out, M, Kin, N1, Kin, L, scaler)      # warm-up (also allocates the workspace)
    ctx.sync()
    best = 1e30
    for _ in range(reps):
        ctx.timer_start()
        sch.PPMM(dW, bufs, out, M, Kin, N1, Kin, L, scaler)
        best = min(best, ctx.timer_stop())
    # the same with the weight matrix declared static: its digit planes are kept, the call neither reads W nor waits for the stream
    sch.pcmm_context.weights_static(dW)
    sch.PPMM(dW, bufs, out, M, Kin, N1, Kin, L, scaler)
    ctx.sync()
    best_static = 1e30
    for _ in range(reps):
        ctx.timer_start()
        sch.PPMM(dW, bufs, out, M, Kin, N1, Kin, L, scaler)
        best_static = min(best_static, ctx.timer_stop())
    DW, DC, path = sch.pcmm_context.info("last_DW"), sch.pcmm_context.info("last_DC"), sch.pcmm_context.info("last_path")
    word_macs = float(M) * Kin * C * L
    macs = word_macs * DW * DC
    res = {"workload": label or ("configs[%d]: PPMM %dx%d, %d tokens (N1), N=2^16, %d primes <2^36, C=%d columns; the product alone - the ring packing behind it exists "
                                "for two ring-pack moduli only (the reference's shape), so no packing stage follows this %d-prime product") % (3 if M == 768 else 4, M, Kin, N1, L, C, L),
           "ms": round(best, 3), "ms_is": "PCMM_Scheme::PPMM as the reference runs it: the weight matrix is quantised and split inside every call (the library's default)",
           "ms_weights_static": round(best_static, 3), "frac_weights_static": round(macs / (best_static * 1e-3) / MFMA_I8_PEAK_MACS, 4),
           "word_MAC_per_s": round(word_macs / (best * 1e-3), 1), "int8_MAC_per_s": round(macs / (best * 1e-3), 1),
           "D_w": DW, "D_c": DC, "plaintext_slices": sch.pcmm_context.info("last_slices"), "kernel": "int8 MFMA" if path == 1 else "generic u128",
           "roofline": {"bound": "mfma", "achieved": round(macs / (best * 1e-3) / 1e12, 2), "peak": round(MFMA_I8_PEAK_MACS / 1e12, 1),
                        "unit": "TMAC/s (int8)", "frac": round(macs / (best * 1e-3) / MFMA_I8_PEAK_MACS, 4)}}
    for b in bufs + seeds + [out, dW]:
        b.free()
    return res


def bench_keyswitch(P, reps=10):
    from ckks_llm_amd import Context_23, DeviceBuffer
    q, p = P.CFG2_Q, P.CFG3_P
    ctx = Context_23(16, p, q)
    N, W, nq, l, dn = 1 << 16, 30, 24, 23, 4
    rng = np.random.default_rng(3)
    evk = np.empty((2 * dn, W, N), dtype=np.uint64)
    for j, m in enumerate(p + q):
        evk[:, j, :] = rng.integers(0, m, size=(2 * dn, N), dtype=np.uint64)
    inp = np.empty((nq, N), dtype=np.uint64)
    for j, m in enumerate(q):
        inp[j] = rng.integers(0, m, N, dtype=np.uint64)
    devk, dinp, dout = DeviceBuffer.from_numpy(evk), DeviceBuffer.from_numpy(inp), DeviceBuffer(8 * 2 * nq * N)
    scratch = DeviceBuffer(8 * (dn + 2) * W * N)
    for _ in range(3):
        ctx.hybrid_keyswitch(dout, dinp, devk, l, scratch)
    ctx.timer_start()
    for _ in range(reps):
        ctx.hybrid_keyswitch(dout, dinp, devk, l, scratch)
    ms = ctx.timer_stop() / reps
    stage_bytes = 1008 * 8 * N           # stage-sum of minimal limb moves: ModUp 24+96, NTT 2*120, IP 360+60, iNTT 2*60, ModDown 60+48
    return {"workload": "configs[2]: hybrid key switch N=2^16, 24 Q + 6 P primes, dnum=4", "us": round(ms * 1e3, 1),
            "keyswitch_per_s": round(1e3 / ms, 1),
            "roofline": {"bound": "hbm", "achieved": round(stage_bytes / (ms * 1e-3) / 1e9, 1), "peak": 8000.0, "unit": "GB/s",
                         "frac": round(stage_bytes / (ms * 1e-3) / HBM_PEAK, 4), "algorithmic_bytes": stage_bytes}}


def bench_rescale(P, reps=20):
    """rescaleAndEqual (Scheme_23.cuh:321-385) of one ciphertext at N = 2^16, 24 primes, from the top level."""
    from ckks_llm_amd import Context_23, DeviceBuffer
    q = P.CFG2_Q
    ctx = Context_23(16, [], q)
    N, l = 1 << 16, len(q) - 1
    rng = np.random.default_rng(6)
    c = np.stack([rng.integers(0, m, (2, N), dtype=np.uint64) for m in q], axis=1)
    d, scratch = DeviceBuffer.from_numpy(c), DeviceBuffer(8 * 2 * len(q) * N)
    for _ in range(3):
        ctx.rescaleAndEqual(d, scratch, l)
    ctx.timer_start()
    for _ in range(reps):
        ctx.rescaleAndEqual(d, scratch, l)
    ms = ctx.timer_stop() / reps
    alg = (2 * (l + 1) + 2 * l) * 8 * N        # every limb of the ciphertext read once, every remaining limb written once
    return {"workload": "rescaleAndEqual: 1 ciphertext, N=2^16, level 23 -> 22 (24 primes <2^36)", "us": round(ms * 1e3, 1),
            "roofline": {"bound": "hbm", "achieved": round(alg / (ms * 1e-3) / 1e9, 1), "peak": 8000.0, "unit": "GB/s",
                         "frac": round(alg / (ms * 1e-3) / HBM_PEAK, 4), "algorithmic_bytes": alg}}


def bench_ntt_ref_primes(P, cts=27, reps=10):
    """The headline transform on the reference's own logN = 16 moduli: its 28 Q primes of 49 bits (Params.cuh:88-171), a batch of 27
    ciphertexts (1512 limbs, 756 MiB).  These primes take the FP64 back end that balances after every register round, with the data
    in place between the two launches (8-byte words; the 5-byte form is for primes below 2^39); the integer back end is timed beside it."""
    from ckks_llm_amd import Context_23, DeviceBuffer
    primes = list(P.REF_PARAMS[16]["q"])
    N, L1, polys = 1 << 16, len(primes), 2 * cts
    limbs = polys * L1
    ctx = Context_23(16, [], primes)
    rng = np.random.default_rng(12)
    one = np.empty((2, L1, N), dtype=np.uint64)
    for j, q in enumerate(primes):
        one[:, j] = rng.integers(0, q, (2, N), dtype=np.uint64)
    buf = DeviceBuffer(8 * limbs * N)
    for c in range(cts):
        buf.L_.ckks_memcpy_h2d(buf.ptr + c * one.nbytes, one.ctypes.data, one.nbytes)
    res = {"workload": "RNS NTT+iNTT, N=2^16, the reference's 28 Q primes of 49 bits, batch of %d ciphertexts (%d limbs, %d MiB) per step" % (cts, limbs, limbs * 8 * N >> 20)}
    for name, mode in (("fp64_balanced", 0), ("integer", 1)):
        ctx.set_arith_mode(mode)
        for _ in range(3):
            ctx.FromNTTInplace(buf, 0, 0, polys, L1, L1)
            ctx.ToNTTInplace(buf, 0, 0, polys, L1, L1)
        ctx.timer_start()
        for _ in range(reps):
            ctx.FromNTTInplace(buf, 0, 0, polys, L1, L1)
            ctx.ToNTTInplace(buf, 0, 0, polys, L1, L1)
        ms = ctx.timer_stop() / reps
        rate = 2 * limbs / (ms * 1e-3)
        res[name] = {"ms_per_step": round(ms, 4), "limb_transforms_per_s": round(rate, 1),
                     "frac_of_hbm_roofline_whole_transform": round(rate * 16 * N / HBM_PEAK, 4)}
    back = buf.download(np.uint64, one.size).reshape(one.shape)
    assert np.array_equal(back, one), "NTT round trip changed the data"
    ctx.set_arith_mode(0)
    buf.free()
    return res


def bench_small_batches(P, reps=100):
    """Forward transform of small batches at N = 2^16 (24 primes below 2^36): the automatic launch form (the paired one-launch
    kernel up to 128 limbs), the paired kernel with a limb's tiles on one XCD and spread over the XCDs, and two launches.
    Times are per call from HIP events around `reps` calls in a row; the 8-limb line is bound by the host's launch rate."""
    from ckks_llm_amd import Context_23, DeviceBuffer
    q = list(P.CFG2_Q[:8])
    N, L1 = 1 << 16, len(q)
    ctx = Context_23(16, [], q)
    rng = np.random.default_rng(7)
    one = np.stack([rng.integers(0, m, N, dtype=np.uint64) for m in q])
    rows = []
    for polys in (1, 2, 3, 4, 5, 6, 8, 12, 18):
        buf = DeviceBuffer.from_numpy(np.tile(one, (polys, 1)))
        row = {"limbs": polys * L1}
        for name, mode in (("automatic_us", 0), ("paired_one_xcd_us", 4), ("paired_spread_us", 5), ("two_launches_us", 1)):
            ctx.set_ntt_mode(mode)
            for _ in range(5):
                ctx.ToNTTInplace(buf, 0, 0, polys, L1, L1)
            ctx.timer_start()
            for _ in range(reps):
                ctx.ToNTTInplace(buf, 0, 0, polys, L1, L1)
            row[name] = round(ctx.timer_stop() / reps * 1e3, 1)
        ctx.check()
        rows.append(row)
        buf.free()
    ctx.set_ntt_mode(0)
    return {"workload": "forward NTT of small batches, N=2^16, 8 primes <2^36 x 1..18 polynomials", "rows": rows}


def bench_mult_23(P, reps=10):
    """Scheme_23::mult_23 (KeySwitch_23.cuh:192-236) on the reference's own logN = 16 parameter set at the top level: tensor product,
    key switch through the T basis with a relinearisation key generated on the device, the two additions."""
    from ckks_llm_amd import Ciphertext, Context_23, DeviceBuffer, Plaintext, Scheme_23, SecretKey
    ctx = Context_23(16, 15, 192)
    N, L, K, T, RB = ctx.N, ctx.L, ctx.K, ctx.t_num, ctx.Ri_blockNum
    key = bytes(range(32))
    scheme = Scheme_23(ctx, key=key)
    sk = SecretKey(ctx, key=key, nonce=1)
    scheme.addEncKey(sk)
    scheme.addMultKey_23(sk)
    msg = Plaintext(N, L, L, N // 2, 1 << 40)
    ctx.encode_coeffs(DeviceBuffer.from_numpy(np.random.default_rng(0).uniform(-1, 1, N)), msg)
    a, b = Ciphertext(N, L, L, N // 2, 1 << 40), Ciphertext(N, L, L, N // 2, 1 << 40)
    scheme.encryptMsg(a, msg)
    scheme.encryptMsg(b, msg)
    res = Ciphertext(N, L, L, N // 2, 1)
    for _ in range(3):
        scheme.mult_23(res, a, b)
    ctx.sync()
    ctx.timer_start()
    for _ in range(reps):
        scheme.mult_23(res, a, b)
    ms = ctx.timer_stop() / reps
    Q, digits, blocks = L + 1, -(-(L + 1) // K), -(-(K + L + 1) // ctx.gamma)
    # stage sum of minimal limb moves: tensor product r4Q w3Q, iNTT 2Q, Qj -> T rQ w(digits T), NTT 2 digits T, inner product
    # r(digits T + 2 digits blocks T) w(2 blocks T), iNTT 4 blocks T, T -> PQ r(2 blocks T) w2(K+Q), ModDown r2(K+Q) w2Q, NTT 4Q, additions r4Q w2Q
    limbs = 7 * Q + 2 * Q + Q + digits * T + 2 * digits * T + digits * T + 2 * digits * blocks * T + 2 * blocks * T + 4 * blocks * T \
        + 2 * blocks * T + 2 * (K + Q) + 2 * (K + Q) + 2 * Q + 4 * Q + 6 * Q
    alg = limbs * 8 * N
    return {"workload": "mult_23 on the reference's logN=16 parameter set (28 Q + 4 P primes of 49-50 bits, 8 T primes of 60 bits), level 27",
            "ms": round(ms, 4), "mult_per_s": round(1e3 / ms, 1),
            "roofline": {"bound": "hbm", "achieved": round(alg / (ms * 1e-3) / 1e9, 1), "peak": 8000.0, "unit": "GB/s",
                         "frac": round(alg / (ms * 1e-3) / HBM_PEAK, 4), "algorithmic_bytes": alg}}


def bench_packing(P, N1=128, reps=5):
    """MLWE -> RLWE packing after PPMM (PCMM_Scheme::mlweCipherPacking): rank = 512 samples of N1 = 128 into one ciphertext at
    N = 2^16, one special prime and q0.  Algorithmic bytes: samples in, the embedded polynomials out and through one NTT,
    embedded 'a' polynomials and keys into the inner product, and the small tail (4 limbs through iNTT, ModDown, NTT)."""
    from ckks_llm_amd import Context_23, DeviceBuffer, PCMM_Context, PCMM_Scheme
    p0, q = P.CFG3_P[0], P.CFG2_Q[:2]
    ctx = Context_23(16, [p0], q)
    N = 1 << 16
    rank = N // N1
    sch = PCMM_Scheme(PCMM_Context(N1, rank, [p0], q, ctx))
    rng = np.random.default_rng(6)
    sample = DeviceBuffer.from_numpy(rng.integers(0, q[0], size=(rank + 1) * N1, dtype=np.uint64))
    bufs = []
    for _ in range(rank):
        b = DeviceBuffer(8 * (rank + 1) * N1)
        b.L_.ckks_memcpy_d2d(b.ptr, sample.ptr, b.nbytes)
        bufs.append(b)
    keys = DeviceBuffer(8 * rank * 4 * N)
    one_key = np.empty((4, N), dtype=np.uint64)
    for j, pr in enumerate((p0, q[0], p0, q[0])):
        one_key[j] = rng.integers(0, pr, N, dtype=np.uint64)
    k0 = DeviceBuffer.from_numpy(one_key)
    for i in range(rank):
        keys.L_.ckks_memcpy_d2d(keys.ptr + i * one_key.nbytes, k0.ptr, one_key.nbytes)
    out, embed, mult = DeviceBuffer(8 * 2 * 2 * N), DeviceBuffer(8 * (rank + 1) * 2 * N), DeviceBuffer(8 * 4 * N)
    sch.mlweCipherPacking(out, bufs, rank, 0, keys, embed, mult)
    ctx.timer_start()
    for _ in range(reps):
        sch.mlweCipherPacking(out, bufs, rank, 0, keys, embed, mult)
    ms = ctx.timer_stop() / reps
    limb = 8.0 * N
    alg = 8.0 * rank * (rank + 1) * N1 + (rank + 1) * 2 * limb + 2 * (rank * 2) * limb + rank * 6 * limb + 4 * limb * 6
    return {"workload": "mlweCipherPacking: 512 MLWE samples (N1=128) -> 1 RLWE ciphertext, N=2^16, primes [p0|q0]", "ms": round(ms, 3),
            "packings_per_s": round(1e3 / ms, 1),
            "roofline": {"bound": "hbm", "achieved": round(alg / (ms * 1e-3) / 1e9, 1), "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                         "frac": round(alg / (ms * 1e-3) / HBM_PEAK, 4), "algorithmic_bytes": alg}}


def bench_decompose(P, N1=128, L1=12, reps=5):
    """RLWE -> MLWE decomposition in front of PPMM (PCMM_Scheme::rlweCipherDecompose): one ciphertext at N = 2^16 with 12 primes
    into rank = 512 samples.  The output is rank times the input; algorithmic bytes = input read once + output written once."""
    from ckks_llm_amd import Context_23, DeviceBuffer, PCMM_Context, PCMM_Scheme
    primes = P.CFG2_Q[:L1]
    ctx = Context_23(16, [], primes)
    N = 1 << 16
    rank = N // N1
    sch = PCMM_Scheme(PCMM_Context(N1, rank, [], primes, ctx))
    rng = np.random.default_rng(7)
    rl = np.empty((2, L1, N), dtype=np.uint64)
    for j, q in enumerate(primes):
        rl[:, j] = rng.integers(0, q, (2, N), dtype=np.uint64)
    d = DeviceBuffer.from_numpy(rl)
    bufs = [DeviceBuffer(8 * L1 * (rank + 1) * N1) for _ in range(rank)]
    sch.rlweCipherDecompose(d, bufs, rank, 0, L1 - 1)
    ctx.timer_start()
    for _ in range(reps):
        sch.rlweCipherDecompose(d, bufs, rank, 0, L1 - 1)
    ms = ctx.timer_stop() / reps
    alg = 8.0 * rank * L1 * (rank + 1) * N1 + 2 * L1 * 8.0 * N * 3        # samples out; ciphertext through iNTT, gather, NTT
    return {"workload": "rlweCipherDecompose: 1 RLWE ciphertext (N=2^16, 12 primes) -> 512 MLWE samples (N1=128)", "ms": round(ms, 3),
            "roofline": {"bound": "hbm", "achieved": round(alg / (ms * 1e-3) / 1e9, 1), "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                         "frac": round(alg / (ms * 1e-3) / HBM_PEAK, 4), "algorithmic_bytes": alg}}


def bench_pcmm_fused(P, M=768, N1=128, L=12, reps=5):
    """configs[3] as a layer runs it: two RLWE ciphertexts -> 512 + 256 samples -> PPMM 768 x 768, with the gather writing the int8 digit
    planes of the MFMA kernel directly (no 8-byte MLWE samples in between), next to the two-step path on the same ciphertexts."""
    from ckks_llm_amd import Context_23, DeviceBuffer, PCMM_Context, PCMM_Scheme
    primes = P.CFG2_Q[:L]
    ctx = Context_23(16, [], primes)
    N = 1 << 16
    rank = N // N1
    C = (rank + 1) * N1
    sch = PCMM_Scheme(PCMM_Context(N1, rank, [], primes, ctx))
    rng = np.random.default_rng(6)
    parts = [(512, 0), (256, 512)]
    Kin = 768
    W = rng.normal(0, 0.02, (M, Kin)).astype(np.float32)
    dW = DeviceBuffer.from_numpy(W)
    sch.pcmm_context.weights_static(dW)                  # a layer's own weights, as the Bert mirrors declare theirs
    cts = []
    for _ in parts:
        a = np.empty((2, L, N), dtype=np.uint64)
        for j, q in enumerate(primes):
            a[:, j] = rng.integers(0, q, (2, N), dtype=np.uint64)
        cts.append(DeviceBuffer.from_numpy(a))
    out = DeviceBuffer(8 * M * L * C)
    scaler = float(2 ** 26)

    def fused():
        sch.packed_begin(Kin, L)
        for (n, off), ct in zip(parts, cts):
            sch.rlweCipherDecompose_packed(ct, n, off, L - 1)
        sch.PPMM_packed(dW, out, M, scaler)

    bufs = [DeviceBuffer(8 * L * C) for _ in range(Kin)]

    def two_step():
        for (n, off), ct in zip(parts, cts):
            sch.rlweCipherDecompose(ct, bufs[off:off + n], n, 0, L - 1)
        sch.PPMM(dW, bufs, out, M, Kin, N1, Kin, L, scaler)

    res = {}
    for name, f in (("two_step", two_step), ("fused", fused)):
        f()
        ctx.sync()
        best = 1e30
        for _ in range(reps):
            ctx.timer_start()
            f()
            best = min(best, ctx.timer_stop())
        res[name + "_ms"] = round(best, 3)
    sch.packed_begin(Kin, L)
    for (n, off), ct in zip(parts, cts):
        sch.rlweCipherDecompose_packed(ct, n, off, L - 1)
    best = 1e30
    for _ in range(reps):
        ctx.timer_start()
        sch.PPMM_packed(dW, out, M, scaler)
        best = min(best, ctx.timer_stop())
    DW = sch.pcmm_context.info("last_DW")
    macs = float(M) * Kin * C * L * DW * 5
    res.update({"workload": "configs[3] as a layer: 2 RLWE ciphertexts (N=2^16, 12 primes) -> 512 + 256 samples -> PPMM 768x768, "
                            "weight matrix declared static (digit planes kept between calls)",
                "ppmm_on_digit_planes_ms": round(best, 3),
                "roofline": {"bound": "mfma", "achieved": round(macs / (best * 1e-3) / 1e12, 2), "peak": round(MFMA_I8_PEAK_MACS / 1e12, 1),
                             "unit": "TMAC/s (int8)", "frac": round(macs / (best * 1e-3) / MFMA_I8_PEAK_MACS, 4)},
                "layer_frac_of_mfma_peak": {"two_step": round(macs / (res["two_step_ms"] * 1e-3) / MFMA_I8_PEAK_MACS, 4),
                                            "fused": round(macs / (res["fused_ms"] * 1e-3) / MFMA_I8_PEAK_MACS, 4)}})
    for b in bufs + cts + [out, dW]:
        b.free()
    return res


def bench_hoisted_level(P, gs=16, bs=4, reps=3):
    """The giant step of one level of the slot <-> coefficient transforms (EncodingMatrix::Giant_Rotate_And_Mult_PlaintT) on the
    reference's logN = 16 parameter set at the top level: gs - 1 keyed rotations and the unrotated pair, each multiplied into bs
    baby steps.  Algorithmic bytes: every key once, the digits, P * (a, b), every plaintext and the bs output pairs once."""
    import ctypes as C
    from ckks_llm_amd import Context_23, DeviceBuffer
    R = P.REF_PARAMS[16]
    ctx = Context_23(16, R["p"], R["q"], R["t"], R["gamma"])
    N, T, RB, dnum, l = ctx.N, ctx.t_num, ctx.Ri_blockNum, ctx.dnum, ctx.L
    digits, blockNum = -(-(l + 1) // ctx.K), -(-(ctx.K + l + 1) // ctx.gamma)
    rng = np.random.default_rng(8)
    chunk = DeviceBuffer.from_numpy(rng.integers(0, min(R["t"]), size=8 * N, dtype=np.uint64))

    def filled(limbs):
        buf = DeviceBuffer(8 * N * limbs)
        for i in range(0, limbs, 8):
            n = min(8, limbs - i)
            buf.L_.ckks_memcpy_d2d(buf.ptr + 8 * N * i, chunk.ptr, 8 * N * n)
        return buf

    keys = [None] + [filled(2 * dnum * RB * T) for _ in range(gs - 1)]
    plains = [filled(T) for _ in range(bs * gs)]
    up, pqT, out = filled(ctx.Qj_blockNum * T), filled(2 * RB * T), DeviceBuffer(8 * N * bs * 2 * RB * T)
    tab = lambda bufs: (C.c_void_p * len(bufs))(*[(b.ptr if b is not None else None) for b in bufs])
    ints = lambda v: (C.c_int * len(v))(*v)
    args = (ctx.h, out.ptr, pqT.ptr, up.ptr, tab(keys), ints([-1] + list(range(1, gs))), tab(plains), ints([gs] * bs), bs, gs, l)
    assert ctx.L_.ckks_giant_rotate_mult_plain_t(*args) == 0
    ctx.timer_start()
    for _ in range(reps):
        ctx.L_.ckks_giant_rotate_mult_plain_t(*args)
    ms = ctx.timer_stop() / reps
    limbs = (gs - 1) * 2 * digits * blockNum * T + digits * T + 2 * blockNum * T + bs * gs * T + bs * 2 * blockNum * T
    nbytes = limbs * 8 * N
    return {"workload": "Giant_Rotate_And_Mult_PlaintT N=2^16, reference logN=16 primes (28 Q, 4 P, 8 T of 60 bits), level 27, gs=%d bs=%d" % (gs, bs),
            "ms": round(ms, 3),
            "roofline": {"bound": "hbm", "achieved": round(nbytes / (ms * 1e-3) / 1e9, 1), "peak": 8000.0, "unit": "GB/s",
                         "frac": round(nbytes / (ms * 1e-3) / HBM_PEAK, 4), "algorithmic_bytes": nbytes}}


def cpu_ppmm(P, M=768, Kin=768, N1=128, L=12, seconds_target=8.0):
    """The CPU oracle's PPMM (the reference's 128-bit accumulation, OpenMP over rows) at the configs[3] shape on a panel of the
    C = 65,664 columns, sized to a few seconds and scaled to the whole product (every column costs the same)."""
    import time
    from oracle import oracle_py as O
    primes = P.CFG2_Q[:L]
    rank = (1 << 16) // N1
    C = (rank + 1) * N1
    octx = O.OracleContext(16, [], primes)
    orc = O.OraclePCMM(octx, N1, rank, [], primes)
    rng = np.random.default_rng(4)
    W = rng.normal(0, 0.02, (M, Kin)).astype(np.float32)
    rng5 = np.random.default_rng(5)
    seeds = []
    for s in range(16):
        a = np.empty((L, C), dtype=np.uint64)
        for j, q in enumerate(primes):
            a[j] = rng5.integers(0, q, C, dtype=np.uint64)
        seeds.append(a.reshape(-1))
    mlwe = [seeds[n % 16] for n in range(Kin)]
    out = np.zeros(M * L * C, dtype=np.uint64)
    cols = 64
    orc.PPMM(W, mlwe, out, M, Kin, L, float(2 ** 26), 0, cols)          # untimed: first touch of the output pages, thread start
    t0 = time.perf_counter()
    orc.PPMM(W, mlwe, out, M, Kin, L, float(2 ** 26), 0, cols)
    once = time.perf_counter() - t0
    cols = int(min(C, max(64, cols * seconds_target / max(once, 1e-3)))) // 64 * 64
    t0 = time.perf_counter()
    orc.PPMM(W, mlwe, out, M, Kin, L, float(2 ** 26), 0, cols)
    dt = time.perf_counter() - t0
    word_macs = float(M) * Kin * cols * L
    return {"value": round(word_macs / dt, 1), "unit": "word_MAC_per_s", "cores": O.lib().orc_max_threads(), "kind": "port",
            "ms_whole_product_extrapolated": round(dt * C / cols * 1e3, 1),
            "sample": "oracle PPMM %dx%d, %d primes, columns 0..%d of %d (%.1f s), scaled by %d / %d to the whole product" % (M, Kin, L, cols - 1, C, dt, C, cols)}


def cpu_keyswitch(P, seconds_target=8.0):
    """The CPU oracle's hybrid key switch at the configs[2] shape (whole size), repeated for a few seconds."""
    import time
    from oracle import oracle_py as O
    q, p = P.CFG2_Q, P.CFG3_P
    octx = O.OracleContext(16, p, q)
    N, Wd, nq, l, dn = 1 << 16, 30, 24, 23, 4
    rng = np.random.default_rng(3)
    evk = np.empty((2 * dn, Wd, N), dtype=np.uint64)
    for j, m in enumerate(p + q):
        evk[:, j, :] = rng.integers(0, m, size=(2 * dn, N), dtype=np.uint64)
    inp = np.empty((nq, N), dtype=np.uint64)
    for j, m in enumerate(q):
        inp[j] = rng.integers(0, m, N, dtype=np.uint64)
    out = np.zeros(2 * nq * N, dtype=np.uint64)
    t0 = time.perf_counter()
    octx.hybrid_keyswitch(out, inp.reshape(-1), evk.reshape(-1), l)
    once = time.perf_counter() - t0
    reps = max(1, min(50, int(seconds_target / max(once, 1e-3))))
    t0 = time.perf_counter()
    for _ in range(reps):
        octx.hybrid_keyswitch(out, inp.reshape(-1), evk.reshape(-1), l)
    dt = (time.perf_counter() - t0) / reps
    return {"value": round(1.0 / dt, 2), "unit": "keyswitch_per_s", "ms": round(dt * 1e3, 1), "cores": O.lib().orc_max_threads(), "kind": "port",
            "sample": "%d x oracle hybrid key switch, N=2^16, 24 Q + 6 P primes, dnum=4 (whole size)" % reps}


def with_traffic(entry, key, traffic, seconds):
    """Beside the fraction on the stage sum (what the reference's unfused stages would move), the fraction on the bytes the
    fused launches really move (rocprofv3 counters, summed over the call's launches)."""
    moved = traffic.get(key)
    r = entry["roofline"]
    r["achieved_is"] = "stage-sum bytes of the reference's unfused stages / time"
    r["traffic"] = moved
    if moved:
        r["traffic_GBps"] = round(moved / seconds / 1e9, 1)
        r["traffic_frac"] = round(moved / seconds / HBM_PEAK, 4)
    return entry


def measured_peaks(copy_gbs=None):
    """Ceilings measured in this run: a register-only loop of the int8 matrix instruction (MAC/s), and the device-to-device copy
    (bytes read + written per second) that the caller measured on the transform's own batch, or one measured here."""
    import ctypes as C
    from ckks_llm_amd import DeviceBuffer
    from ckks_llm_amd._lib import load_library
    L = load_library()
    macs = C.c_double()
    if L.ckks_measure_mfma_i8_peak(None, C.byref(macs)) != 0:
        raise RuntimeError("ckks_measure_mfma_i8_peak failed")
    if copy_gbs is None:
        half = 384 << 20
        buf = DeviceBuffer(2 * half)
        import time
        for _ in range(2):
            L.ckks_memcpy_d2d(buf.ptr + half, buf.ptr, half)
        L.ckks_sync()
        t0 = time.perf_counter()
        for _ in range(5):
            L.ckks_memcpy_d2d(buf.ptr + half, buf.ptr, half)
        L.ckks_sync()
        copy_gbs = 2.0 * half * 5 / (time.perf_counter() - t0) / 1e9
        buf.free()
    return {"mfma_i8_TMACs": round(macs.value / 1e12, 1), "hbm_copy_GBps": round(copy_gbs, 1),
            "how": "int8 MFMA: loop of v_mfma_i32_16x16x64_i8 on registers alone, two workgroups of 512 lanes per compute unit; HBM: "
                   "device-to-device copy of 384 MiB, bytes read + bytes written per second; both in this run"}


def add_measured(entry, peaks):
    """peak_measured / frac_of_measured beside the published peak in an entry's roofline."""
    r = entry.get("roofline")
    if not r:
        return
    if r.get("bound") == "mfma":
        r["peak_measured"] = peaks["mfma_i8_TMACs"]
        r["frac_of_measured"] = round(r["achieved"] / peaks["mfma_i8_TMACs"], 4)
    else:
        r["peak_measured"] = peaks["hbm_copy_GBps"]
        r["frac_of_measured"] = round(r["achieved"] / peaks["hbm_copy_GBps"], 4)


def run(P, traffic_info=({}, ""), copy_gbs=None):
    traffic, note = traffic_info
    ref_label = "PPMM 768x768 on the reference's own two 49-bit ring-pack moduli (Params.cuh, logN = 16), N=2^16, 128 tokens, plaintext scaled by 2^26"
    ref_scale_label = ("PPMM 768x768 as the reference's BERT layer calls it: its two 49-bit ring-pack moduli and its scaler q1 * 2^49 / scale "
                       "with scale = 2^49 (PPMM_kernel.cuh:283-284), i.e. 46-bit plaintext entries, N=2^16, 128 tokens")
    res = {"ppmm": bench_ppmm(P), "ppmm_ref_primes": bench_ppmm(P, L=2, primes=P.REF_PARAMS[16]["q"], label=ref_label),
            "ppmm_ref_primes_ref_scaler": bench_ppmm(P, L=2, primes=P.REF_PARAMS[16]["q"], label=ref_scale_label, scaler=float(P.REF_PARAMS[16]["q"][1])), "ppmm_4096": bench_ppmm(P, M=4096, Kin=4096, reps=2), "pcmm_layer": bench_pcmm_fused(P), "keyswitch": bench_keyswitch(P), "rescale": bench_rescale(P), "ntt_ref_primes": bench_ntt_ref_primes(P), "small_batches": bench_small_batches(P), "mult_23_ref_params": bench_mult_23(P),
            "decompose": bench_decompose(P), "packing": bench_packing(P), "hoisted_level": bench_hoisted_level(P)}
    with_traffic(res["keyswitch"], "hybrid_keyswitch_config3", traffic, res["keyswitch"]["us"] * 1e-6)
    with_traffic(res["rescale"], "rescale_one_ciphertext_level23", traffic, res["rescale"]["us"] * 1e-6)
    with_traffic(res["mult_23_ref_params"], "mult_23_ref_params_level27", traffic, res["mult_23_ref_params"]["ms"] * 1e-3)
    with_traffic(res["decompose"], "rlwe_decompose_512_samples", traffic, res["decompose"]["ms"] * 1e-3)
    with_traffic(res["packing"], "mlwe_packing_512_samples", traffic, res["packing"]["ms"] * 1e-3)
    with_traffic(res["hoisted_level"], "giant_rotate_gs16_bs4", traffic, res["hoisted_level"]["ms"] * 1e-3)
    res["traffic_source"] = note
    peaks = measured_peaks(copy_gbs)
    for key in ("ppmm", "ppmm_ref_primes", "ppmm_ref_primes_ref_scaler", "ppmm_4096", "pcmm_layer", "keyswitch", "rescale", "mult_23_ref_params",
                "decompose", "packing", "hoisted_level"):
        add_measured(res[key], peaks)
    res["measured_peaks"] = peaks
    return res


LEGS = {"ppmm": lambda P: bench_ppmm(P), "ppmm_4096": lambda P: bench_ppmm(P, M=4096, Kin=4096, reps=2), "pcmm_layer": bench_pcmm_fused,
        "keyswitch": bench_keyswitch, "rescale": bench_rescale, "ntt_ref_primes": bench_ntt_ref_primes, "mult_23_ref_params": bench_mult_23, "decompose": bench_decompose,
        "packing": bench_packing, "hoisted_level": bench_hoisted_level, "cpu_ppmm": cpu_ppmm, "cpu_keyswitch": cpu_keyswitch,
        "small_batches": bench_small_batches}

if __name__ == "__main__":
    # one leg on its own, for profiling:  python3 bench_extra.py keyswitch
    import json
    import os
    import sys
    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    import ckks_llm_amd.params as params
    if len(sys.argv) != 2 or sys.argv[1] not in LEGS:
        sys.exit("usage: bench_extra.py <%s>" % " | ".join(LEGS))
    print(json.dumps(LEGS[sys.argv[1]](params)))
