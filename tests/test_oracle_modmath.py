"""Pins the oracle's scalar modmath against Python big-int arithmetic (brute force, edge operands)."""
import random

import pytest

from oracle import oracle_py as O
from tests.params import CFG2_Q, CFG3_P, REF_PARAMS

PRIMES = CFG2_Q[:3] + CFG3_P[:2] + REF_PARAMS[16]["q"][:2] + REF_PARAMS[16]["t"][:3] + [65537, 998244353]


@pytest.mark.parametrize("q", PRIMES)
def test_mulmod_pow_inv_shoup(q):
    L = O.lib()
    rnd = random.Random(q)
    xs = [0, 1, 2, q - 1, q - 2, q // 2] + [rnd.randrange(q) for _ in range(200)]
    for a in xs:
        b = rnd.randrange(q)
        assert L.orc_mulmod(a, b, q) == a * b % q
        assert L.orc_xshoup(b, q) == (b << 64) // q
        if a:
            assert L.orc_invmod(a, q) * a % q == 1
        e = rnd.randrange(1 << 40)
        assert L.orc_powmod(a, e, q) == pow(a, e, q)
    # Shoup product: exact for any a < 2^64 (lazy inputs 2q-1, 4q-1, 2^64-1) and b < q
    for a in [0, q - 1, 2 * q - 1, 4 * q - 1, (1 << 64) - 1] + [rnd.randrange(1 << 64) for _ in range(300)]:
        b = rnd.randrange(q)
        assert L.orc_mulmod_shoup(a, b, (b << 64) // q, q) == a * b % q


@pytest.mark.parametrize("q", PRIMES)
def test_barrett(q):
    import ctypes as C
    L = O.lib()
    hi, lo = C.c_uint64(), C.c_uint64()
    L.orc_barrett_mu(q, C.byref(hi), C.byref(lo))
    assert (hi.value << 64) | lo.value == (1 << 128) // q
    rnd = random.Random(q + 1)
    # 128-bit Barrett: accumulators as large as 64 products of two residues, plus wrapped (negative) values that
    # the base-conversion correction can produce stay outside its domain and are not asserted here
    bound = min(64 * q * q, (1 << 128) - 1)
    for a in [0, q - 1, q, q * q - 1, bound - 1] + [rnd.randrange(bound) for _ in range(500)]:
        assert L.orc_barrett128(a >> 64, a & ((1 << 64) - 1), q, hi.value, lo.value) == a % q
    for a in [0, q - 1, q, 2 * q, (1 << 62)] + [rnd.randrange(1 << 62) for _ in range(300)]:
        assert L.orc_barrett64(a, q, hi.value) == a % q
