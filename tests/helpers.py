"""Shared test helpers: seeded inputs and small exact (Python big-int) algebra used to pin the oracle."""
import numpy as np


def uniform_residues(rng, q, shape):
    """Uniform u64 residues in [0, q)."""
    return rng.integers(0, q, size=shape, dtype=np.uint64)


def limbs_uniform(seed, primes, n_polys, N):
    """[n_polys][len(primes)][N] uniform residues, limb (y, j) modulo primes[j]."""
    rng = np.random.default_rng(seed)
    out = np.empty((n_polys, len(primes), N), dtype=np.uint64)
    for j, q in enumerate(primes):
        out[:, j, :] = uniform_residues(rng, q, (n_polys, N))
    return out


def bitrev(x, bits):
    r = 0
    for _ in range(bits):
        r = (r << 1) | (x & 1)
        x >>= 1
    return r


def negacyclic_mul(a, b, q):
    """Schoolbook product in Z_q[x]/(x^n+1) with Python ints."""
    n = len(a)
    c = [0] * n
    for i in range(n):
        if a[i] == 0:
            continue
        for j in range(n):
            k = i + j
            if k < n:
                c[k] = (c[k] + a[i] * b[j]) % q
            else:
                c[k - n] = (c[k - n] - a[i] * b[j]) % q
    return c


def crt(residues, primes):
    """Exact CRT reconstruction into [0, prod primes)."""
    M = 1
    for p in primes:
        M *= p
    x = 0
    for r, p in zip(residues, primes):
        Mi = M // p
        x += int(r) * Mi * pow(Mi, -1, p)
    return x % M, M


def precision_table(got, want, label, min_bits, median_bits):
    """The reference states the agreement of a decrypted result with its plaintext model as GetPrecisionStats' table of
    log2(1 / |difference|) (precision.cuh:104-249; test programs print it).  Prints that table and asserts on its worst and median row."""
    from ckks_llm_amd.precision import GetPrecisionStats
    stats = GetPrecisionStats(np.asarray(got, dtype=np.float64).reshape(-1), np.asarray(want, dtype=np.float64).reshape(-1))
    print("%s: precision in bits (log2 of 1 / |decrypted - plain product|)%s" % (label, stats.String()))
    assert stats.MinPrecision.Real >= min_bits, (label, "worst coefficient", stats.MinPrecision.Real, "bits, wanted", min_bits)
    assert stats.MedianPrecision.Real >= median_bits, (label, "median", stats.MedianPrecision.Real, "bits, wanted", median_bits)
    return stats
