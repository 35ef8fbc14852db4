"""GPU parity of the transform that allocates nothing (ckks_ntt_noalloc) against the ordinary entry points, through the C ABI.

Two calls in a row on one context, the second on a smaller batch: the fixed inter-pass area keeps the first call's contents,
and the second call must not see them.  Bit-exact, forward and inverse, plus the size limit and a ring without the 5-byte form.
"""
import numpy as np
import pytest

from ckks_llm_amd import CkksError
from tests.gpu_common import Pair, to_dev, from_dev
from tests.helpers import limbs_uniform
from tests.params import CFG2_Q

pytestmark = pytest.mark.gpu


def _both_ways(pair, primes, poly_num, seed):
    N, mod_num = pair.N, len(primes)
    data = limbs_uniform(seed, primes, poly_num, N)
    ref, got = to_dev(data), to_dev(data)
    pair.dev.ToNTTInplace(ref, 0, 0, poly_num, mod_num, mod_num)
    pair.dev.ntt_noalloc(got, 0, 0, poly_num, mod_num, mod_num, False)
    fwd = from_dev(ref, data.shape)
    assert np.array_equal(from_dev(got, data.shape), fwd)
    want = data.copy()
    pair.orc.ToNTTInplace(want.reshape(-1), 0, 0, poly_num, mod_num, mod_num)
    assert np.array_equal(fwd, want)
    pair.dev.ntt_noalloc(got, 0, 0, poly_num, mod_num, mod_num, True)
    assert np.array_equal(from_dev(got, data.shape), data)
    # inverse of arbitrary words against the ordinary inverse
    ref.upload(data)
    got.upload(data)
    pair.dev.FromNTTInplace(ref, 0, 0, poly_num, mod_num, mod_num)
    pair.dev.ntt_noalloc(got, 0, 0, poly_num, mod_num, mod_num, True)
    assert np.array_equal(from_dev(got, data.shape), from_dev(ref, data.shape))
    ref.free()
    got.free()


def test_two_calls_in_a_row_second_smaller():
    pair = Pair(16, [], CFG2_Q)
    assert pair.dev.ntt_noalloc_max_limbs() >= 48
    _both_ways(pair, CFG2_Q, 2, seed=71)            # one ciphertext: 48 limbs
    _both_ways(pair, CFG2_Q[:5], 1, seed=72)        # 5 limbs, the area still holds the first call's data
    _both_ways(pair, CFG2_Q, 2, seed=73)


def test_limit_is_reported():
    pair = Pair(16, [], CFG2_Q)
    cap = pair.dev.ntt_noalloc_max_limbs()
    polys = cap // len(CFG2_Q) + 1
    buf = to_dev(np.zeros((polys, len(CFG2_Q), pair.N), dtype=np.uint64))
    with pytest.raises(CkksError, match="limit"):
        pair.dev.ntt_noalloc(buf, 0, 0, polys, len(CFG2_Q), len(CFG2_Q), False)
    buf.free()


def test_ring_without_inter_pass_buffer():
    q = CFG2_Q[:3]
    pair = Pair(12, [], q)
    _both_ways(pair, q, 4, seed=74)
    _both_ways(pair, q, 2, seed=75)
