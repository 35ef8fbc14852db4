"""Range check of the library's exact-integer FP64 arithmetic, on the CPU.

tests/cpp/f64_ranges.cpp compiles the FP64 transform back ends, the conversion sums and the PPMM recombination of
ckks_llm_amd/csrc (the functions the kernels are built from) for the host with their range hooks on: every multiplication,
balance, sum and bit-pattern conversion reports to a checker that redoes the step in 128-bit integers and records a violation if
an operand is no integer below 2^53, a product is not h + l, h - c q is not exact, or a result is not the residue it should be.
Here whole transforms, conversions, ModDown sums and PPMM epilogues run through it on worst-case and random inputs at the range
ends of each back end, and the results are compared with the oracle or with Python integers.  The counterpart of the
reference's `check_mod_operation` assertions (src/ckks/include/uint128.cuh:19, 175-177, 209-211, 222-224).
"""
import ctypes as C
import os
import subprocess

import numpy as np
import pytest
import sympy

from oracle import oracle_py as O
from tests.params import CFG2_Q, CFG3_P, REF_PARAMS

HERE = os.path.dirname(os.path.abspath(__file__))
CPP = os.path.join(HERE, "cpp")
u64p = C.POINTER(C.c_uint64)


def _lib():
    path = os.path.join(CPP, "libf64_ranges.so")
    if not os.path.exists(path):
        subprocess.check_call(["make", "-C", CPP, "libf64_ranges.so"], stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)
    L = C.CDLL(path)
    L.f64r_stats.argtypes = [C.POINTER(C.c_long), C.POINTER(C.c_double), C.c_char_p, C.c_int]
    L.f64r_ntt.argtypes = [C.c_int, C.c_int, C.c_uint64, u64p, C.c_uint64, u64p, C.c_int, C.c_int]
    L.f64r_conv.argtypes = [C.c_int, C.c_int, u64p, u64p, u64p, u64p, u64p, u64p, u64p, C.c_long]
    L.f64r_conv_split.argtypes = [C.c_int, C.c_int, u64p, u64p, u64p, u64p, u64p, u64p, u64p, C.c_long]
    L.f64r_moddown.argtypes = [C.c_int, C.c_uint64, C.c_int, u64p, u64p, C.c_uint64, u64p, u64p, C.c_long]
    L.f64r_ppmm.argtypes = [C.c_int, C.c_int, C.c_uint64, C.c_uint64, C.c_uint64, C.c_uint64, C.c_int, C.POINTER(C.c_int), u64p, u64p, C.c_long]
    return L


@pytest.fixture(scope="module")
def lib():
    return _lib()


def _p(a):
    return a.ctypes.data_as(u64p)


def _u64(v):
    return np.ascontiguousarray(np.array(v, dtype=object).astype(np.uint64))


def stats(L):
    out, dout, first = (C.c_long * 2)(), (C.c_double * 3)(), C.create_string_buffer(256)
    L.f64r_stats(out, dout, first, 256)
    return {"checks": out[0], "violations": out[1], "max_abs": dout[0], "max_mulmod": dout[1], "max_balance": dout[2], "first": first.value.decode()}


def clean(L, what):
    s = stats(L)
    assert s["checks"] > 0, what
    assert s["violations"] == 0, (what, s["first"])
    assert s["max_abs"] < 2.0 ** 53, what
    return s


def largest_ntt_prime(below, logN):
    """Largest prime under `below` that has a 2N-th root of unity."""
    step = 2 << logN
    q = (below - 1) // step * step + 1
    while not sympy.isprime(q):
        q -= step
    return q


def patterns(q, N, seed):
    rng = np.random.default_rng(seed)
    i = np.arange(N, dtype=np.uint64)
    yield "all q - 1", np.full(N, q - 1, dtype=np.uint64)
    yield "alternating 0, q - 1", np.where(i & 1 == 1, np.uint64(q - 1), np.uint64(0))
    yield "around q / 2", np.uint64(q // 2) + (i & np.uint64(1))
    yield "blocks of q - 1 and 1", np.where((i >> np.uint64(4)) & np.uint64(1) == 1, np.uint64(q - 1), np.uint64(1))
    yield "random", rng.integers(0, q, N, dtype=np.uint64)


# (prime, logN, wide back end, forms of the data between the passes: 0 in place, 1 the 40-bit form, 2 the 36-bit form)
def ntt_cases():
    top36 = max(CFG2_Q)
    top39 = max(CFG3_P)
    return [
        ("largest 36-bit prime of the headline set", top36, 16, 0, (2,)),
        ("largest 36-bit prime of the headline set", top36, 12, 0, (0, 1, 2)),
        ("largest special prime (38 bits)", top39, 12, 0, (0, 1)),
        ("largest prime below 2^39", largest_ntt_prime(1 << 39, 13), 13, 0, (0, 1)),
        ("largest prime below 2^41", largest_ntt_prime(1 << 41, 13), 13, 0, (0,)),
        ("the reference's first 49-bit prime", REF_PARAMS[16]["q"][0], 12, 1, (0,)),
        ("largest prime below 2^50", largest_ntt_prime(1 << 50, 13), 13, 1, (0,)),
        ("largest prime below 2^50", largest_ntt_prime(1 << 50, 16), 16, 1, (0,)),
        ("a small prime on the wide back end", largest_ntt_prime(1 << 30, 10), 10, 1, (0,)),
    ]


@pytest.mark.parametrize("case", ntt_cases(), ids=lambda c: "%s logN=%d" % (c[0], c[2]))
def test_whole_transforms_stay_exact(lib, case):
    """Forward and inverse transforms of one limb, pass by pass as the kernels run them, on extreme and random words: no range
    violation, and the words are the oracle's."""
    name, q, logN, wide, forms = case
    N = 1 << logN
    orc = O.OracleContext(logN, [], [q])
    psi, psiinv, n_inv = orc.table("psi_table"), orc.table("psiinv_table"), int(orc.table("n_inv")[0])
    assert len(psi) == N and len(psiinv) == N
    for form in forms:
        for label, data in patterns(q, N, seed=logN + form):
            want = data.copy()
            orc.ToNTTInplace(want, 0, 0, 1, 1, 1)
            got = data.copy()
            lib.f64r_reset()
            assert lib.f64r_ntt(wide, form, q, _p(psi), n_inv, _p(got), logN, 0) == 0
            s = clean(lib, (name, "forward", form, label))
            assert np.array_equal(got, want), (name, "forward", form, label)
            want_inv = data.copy()
            orc.FromNTTInplace(want_inv, 0, 0, 1, 1, 1)
            got = data.copy()
            lib.f64r_reset()
            assert lib.f64r_ntt(wide, form, q, _p(psiinv), n_inv, _p(got), logN, 1) == 0
            s2 = clean(lib, (name, "inverse", form, label))
            assert np.array_equal(got, want_inv), (name, "inverse", form, label)
            # the header comments of the back ends promise these: products within 0.51 q (narrow) resp. within 2 q (wide, the last
            # inverse stage multiplies sums of up to 8 q) of zero
            assert max(s["max_mulmod"], s2["max_mulmod"]) < (2.0 if wide else 0.52), (name, form, label, s["max_mulmod"], s2["max_mulmod"])


def test_the_checker_sees_a_violation(lib):
    """The wide back end's ranges are needed: a 49-bit prime on the back end for primes below 2^41 (no balance between the
    register rounds) must trip the checker - a checker that cannot fail proves nothing."""
    q, logN = REF_PARAMS[16]["q"][0], 12
    orc = O.OracleContext(logN, [], [q])
    data = np.full(1 << logN, q - 1, dtype=np.uint64)
    lib.f64r_reset()
    assert lib.f64r_ntt(0, 0, q, _p(orc.table("psiinv_table")), int(orc.table("n_inv")[0]), _p(data), logN, 1) == 0
    s = stats(lib)
    assert s["violations"] > 0 and s["first"]


def _crt_consts(src, tgt):
    D = 1
    for d in src:
        D *= d
    hatinv = [pow(D // d % d, -1, d) for d in src]
    hat = [[D // d % r for d in src] for r in tgt]
    dmod = [D % r for r in tgt]
    return D, hatinv, hat, dmod


def test_conversion_sums_below_2_41(lib):
    """conv_kernel_f64's sums for the largest bases it takes (16 sources, primes up to 2^41): extreme and random residues against
    Python integers, with the reference's v = (int) sum y_j / d_j (BasisConv.cuh:84-159)."""
    step = 1 << 14
    pool, q = [], (1 << 41) + 1
    while len(pool) < 24:
        q = largest_ntt_prime(q - 1, 13)
        pool.append(q)
    src, tgt = pool[:16], pool[16:]
    D, hatinv, hat, dmod = _crt_consts(src, tgt)
    count = 4096
    rng = np.random.default_rng(5)
    x = np.stack([rng.integers(0, d, count, dtype=np.uint64) for d in src])
    x[:, 0] = [d - 1 for d in src]
    x[:, 1] = 0
    x[:, 2] = [d // 2 for d in src]
    x[:, 3] = [(d - 1) * pow(D // d % d, 1, d) % d for d in src]          # y_j = d_j - 1 for every source: the largest sums
    out = np.zeros((len(tgt), count), dtype=np.uint64)
    lib.f64r_reset()
    assert lib.f64r_conv(len(src), len(tgt), _p(_u64(src)), _p(_u64(tgt)), _p(_u64(hatinv)), _p(_u64([h for row in hat for h in row])), _p(_u64(dmod)),
                         _p(x), _p(out), count) == 0
    clean(lib, "conv_f64")
    for n in range(count):
        y = [int(x[j, n]) * hatinv[j] % src[j] for j in range(len(src))]
        vv = 0.0
        for j in range(len(src)):
            vv += float(y[j]) / float(src[j])
        v = int(vv)
        for k, r in enumerate(tgt):
            assert int(out[k, n]) == (sum(y[j] * hat[k][j] for j in range(len(src))) - v * D) % r, (n, k)
        if n >= 64 and n % 64:
            continue


def test_conversion_sums_wide_targets(lib):
    """conv_kernel_split's sums: 60-bit sources (the reference's T basis), targets just below 2^50."""
    src = list(REF_PARAMS[16]["t"])[:8]
    tgt = [largest_ntt_prime(1 << 50, 16)] + list(REF_PARAMS[16]["q"][:3]) + list(REF_PARAMS[16]["p"][:1])
    D, hatinv, hat, dmod = _crt_consts(src, tgt)
    hat31 = [[h * (1 << 31) % r for h in row] for row, r in zip(hat, tgt)]
    count = 2048
    rng = np.random.default_rng(6)
    y = np.stack([rng.integers(0, d, count, dtype=np.uint64) for d in src])
    y[:, 0] = [d - 1 for d in src]
    y[:, 1] = 0
    y[:, 2] = [(1 << 31) - 1 for _ in src]
    y[:, 3] = [d - (d % (1 << 31)) - 1 if d % (1 << 31) else d - 1 for d in src]
    out = np.zeros((len(tgt), count), dtype=np.uint64)
    lib.f64r_reset()
    flat = lambda m: _u64([h for row in m for h in row])
    assert lib.f64r_conv_split(len(src), len(tgt), _p(_u64(src)), _p(_u64(tgt)), _p(flat(hat)), _p(flat(hat31)), _p(_u64(dmod)), _p(y), _p(out), count) == 0
    clean(lib, "conv_split")
    for n in range(0, count, 1 if count <= 4096 else 7):
        vv = 0.0
        for j in range(len(src)):
            vv += float(int(y[j, n])) / float(src[j])
        v = int(vv)
        for k, r in enumerate(tgt):
            assert int(out[k, n]) == (sum(int(y[j, n]) * hat[k][j] for j in range(len(src))) - v * D) % r, (n, k)


@pytest.mark.parametrize("wide", [0, 1])
def test_moddown_sum(lib, wide):
    """The ModDown of the fused key switch with the most special primes it admits (8), each larger than q, on extreme residues."""
    K = 8
    if wide:
        q = REF_PARAMS[16]["q"][0]
        ps, nxt = [], 1 << 50
        while len(ps) < K:
            nxt = largest_ntt_prime(nxt - 1, 16)
            ps.append(nxt)
    else:
        q = min(CFG2_Q)
        ps, nxt = [], 1 << 39
        while len(ps) < K:
            nxt = largest_ntt_prime(nxt - 1, 16)
            ps.append(nxt)
    P = 1
    for p in ps:
        P *= p
    phat = [P // p % q for p in ps]
    pinv = pow(P % q, -1, q)
    count = 4096
    rng = np.random.default_rng(7 + wide)
    x = np.stack([rng.integers(0, p, count, dtype=np.uint64) for p in ps])
    own = rng.integers(0, q, count, dtype=np.uint64)
    x[:, 0] = [p - 1 for p in ps]
    own[0] = 0
    x[:, 1] = 0
    own[1] = q - 1
    out = np.zeros(count, dtype=np.uint64)
    lib.f64r_reset()
    assert lib.f64r_moddown(wide, q, K, _p(x), _p(_u64(phat)), pinv, _p(own), _p(out), count) == 0
    clean(lib, "moddown")
    for n in range(count):
        s = sum(int(x[i, n]) * phat[i] for i in range(K))
        assert int(out[n]) == (int(own[n]) - s) * pinv % q, n


@pytest.mark.parametrize("shape", [(0, 7), (0, 8), (1, 9)], ids=["3x5 digits", "4x5 digits", "3x7 digits (wide)"])
def test_ppmm_recombination(lib, shape):
    """The epilogue of the digit-plane PPMM on the largest anti-diagonal sums the launcher admits (a diagonal holds at most DW digit
    pairs per k, a product of two balanced digits is at most 2^14, and the launcher takes DW * Kpad <= 2^14: |S_e| <= 2^28), both
    signs, for the largest prime of each form; also the fused rescale."""
    wide, ND = shape
    q = largest_ntt_prime(1 << 50, 16) if wide else largest_ntt_prime((0x7f7f7f7f7f + 1), 16)
    q_last = REF_PARAMS[16]["q"][1] if wide else max(CFG2_Q)
    count = 8192
    rng = np.random.default_rng(9 + ND)
    bound = 1 << 28
    S = rng.integers(-bound, bound + 1, (count, ND), dtype=np.int64)
    S[0] = bound
    S[1] = -bound
    S[2] = [bound if e % 2 else -bound for e in range(ND)]
    S[3] = 0
    S = np.ascontiguousarray(S.astype(np.int32))
    r_last = rng.integers(0, q_last, count, dtype=np.uint64)
    r_last[0], r_last[1] = q_last - 1, 0
    c32, c64, qli = (1 << 32) % q, (1 << 64) % q, pow(q_last % q, -1, q)
    for last in (1, 0):
        out = np.zeros(count, dtype=np.uint64)
        lib.f64r_reset()
        assert lib.f64r_ppmm(wide, ND, q, c32, c64, qli, last, S.ctypes.data_as(C.POINTER(C.c_int)), _p(r_last), _p(out), count) == 0
        clean(lib, ("ppmm", shape, last))
        for n in range(count):
            val = sum(int(S[n, e]) << (8 * e) for e in range(ND))
            want = val % q if last else (val - int(r_last[n])) * qli % q
            assert int(out[n]) == want, (n, last)


def test_sanitizer_build_of_the_range_check():
    """The same program as a stand-alone binary under AddressSanitizer and UBSan: transforms at three sizes and every form, round
    trip and zero violations."""
    exe = os.path.join(CPP, "f64_ranges_san.bin")
    if not os.path.exists(exe):
        subprocess.check_call(["make", "-C", CPP, "f64_ranges_san.bin"], stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)
    q36, q49 = max(CFG2_Q), REF_PARAMS[16]["q"][0]
    args = ["%d:8:0:0" % q36, "%d:10:0:1" % q36, "%d:12:0:2" % q36, "%d:13:0:0" % q36, "%d:12:1:0" % q49, "%d:16:1:0" % q49]
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", UBSAN_OPTIONS="halt_on_error=1:print_stacktrace=1")
    # when this suite itself runs under the host compiler's sanitizer runtimes (the oracle's SAN=1 build), those must not be
    # preloaded into this binary, which brings its own; anything else in the variable stays
    if env.get("LD_PRELOAD"):
        env["LD_PRELOAD"] = " ".join(x for x in env["LD_PRELOAD"].replace(":", " ").split() if "libasan" not in x and "libubsan" not in x)
    r = subprocess.run([exe] + args, capture_output=True, text=True, env=env, timeout=300)
    assert r.returncode == 0, (r.stdout[-2000:], r.stderr[-2000:])
    assert "runtime error" not in r.stderr and "AddressSanitizer" not in r.stderr, r.stderr[-2000:]
