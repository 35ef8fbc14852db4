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


def _free_device_bytes(hip):
    import ctypes
    free, total = ctypes.c_size_t(), ctypes.c_size_t()
    assert hip.hipMemGetInfo(ctypes.byref(free), ctypes.byref(total)) == 0
    return free.value


def test_the_entry_allocates_nothing_and_leaves_the_context_alone():
    """On a fresh context (whose inter-pass buffer does not exist yet) the first call, at the largest batch the entry takes, leaves
    the device's free memory and the context's own buffer as they were, and does not touch the context's launch mode.  The same
    call recorded into a HIP graph (a capture refuses every allocation) replays with the ordinary entry point's result."""
    import ctypes
    hip = ctypes.CDLL("libamdhip64.so")
    # another context first: the runtime loads the kernels' code on the first launch of a process, which is not this entry's doing
    warm = Pair(16, [], CFG2_Q[:2])
    tiny = to_dev(limbs_uniform(80, CFG2_Q[:2], 1, warm.N))
    warm.dev.ntt_noalloc(tiny, 0, 0, 1, 2, 2, False)
    warm.dev.sync()
    pair = Pair(16, [], CFG2_Q)
    d, N = pair.dev, pair.N
    cap = d.ntt_noalloc_max_limbs()
    polys, mods = 2, min(len(CFG2_Q), cap // 2)
    data = limbs_uniform(81, CFG2_Q[:mods], polys, N)
    got, ref = to_dev(data), to_dev(data)
    d.sync()
    assert d.info("ntt_mid_bytes") == 0
    d.set_ntt_mode(1)
    before = _free_device_bytes(hip)
    d.ntt_noalloc(got, 0, 0, polys, mods, mods, False)
    d.sync()
    assert _free_device_bytes(hip) == before
    assert d.info("ntt_mid_bytes") == 0 and d.info("ntt_mode") == 1
    d.set_ntt_mode(0)
    d.ToNTTInplace(ref, 0, 0, polys, mods, mods)
    want = from_dev(ref, data.shape)
    assert np.array_equal(from_dev(got, data.shape), want)
    # under capture
    stream = ctypes.c_void_p()
    assert hip.hipStreamCreate(ctypes.byref(stream)) == 0
    d.set_stream(stream)
    graph, gexec = ctypes.c_void_p(), ctypes.c_void_p()
    assert hip.hipStreamBeginCapture(stream, 0) == 0
    d.ntt_noalloc(got, 0, 0, polys, mods, mods, False)
    assert hip.hipStreamEndCapture(stream, ctypes.byref(graph)) == 0
    assert hip.hipGraphInstantiate(ctypes.byref(gexec), graph, None, None, ctypes.c_size_t(0)) == 0
    for rep in range(3):
        fresh = limbs_uniform(90 + rep, CFG2_Q[:mods], polys, N)
        got.upload(fresh)
        ref.upload(fresh)
        assert hip.hipGraphLaunch(gexec, stream) == 0
        assert hip.hipStreamSynchronize(stream) == 0
        d.set_stream(None)
        d.ToNTTInplace(ref, 0, 0, polys, mods, mods)          # eager work between the replays
        d.sync()
        d.set_stream(stream)
        assert np.array_equal(from_dev(got, data.shape), from_dev(ref, data.shape)), rep
    assert hip.hipGraphExecDestroy(gexec) == 0 and hip.hipGraphDestroy(graph) == 0
    d.set_stream(None)
    assert hip.hipStreamDestroy(stream) == 0
    got.free()
    ref.free()


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
