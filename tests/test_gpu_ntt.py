"""GPU parity: batched NTT / iNTT through the C ABI against the CPU oracle, bit-exact."""
import numpy as np
import pytest

from tests.gpu_common import Pair, to_dev, from_dev
from tests.helpers import limbs_uniform
from tests.params import CFG1_Q, CFG2_Q, CFG3_P, REF_PARAMS

pytestmark = pytest.mark.gpu


def check_fwd_inv(pair, primes_idx0, primes, poly_num, seed, mode=None):
    """Forward vs oracle, inverse vs oracle, round trip; limbs (y, j) at (y*len + j)."""
    if mode is not None:
        pair.dev.set_arith_mode(mode)
    N, mod_num = pair.N, len(primes)
    data = limbs_uniform(seed, primes, poly_num, N)
    want = data.copy()
    pair.orc.ToNTTInplace(want.reshape(-1), 0, primes_idx0, poly_num, mod_num, mod_num)
    buf = to_dev(data)
    pair.dev.ToNTTInplace(buf, 0, primes_idx0, poly_num, mod_num, mod_num)
    got = from_dev(buf, data.shape)
    assert np.array_equal(got, want)
    pair.dev.FromNTTInplace(buf, 0, primes_idx0, poly_num, mod_num, mod_num)
    assert np.array_equal(from_dev(buf, data.shape), data)
    # inverse of arbitrary (non-transform) data against the oracle
    want_inv = data.copy()
    pair.orc.FromNTTInplace(want_inv.reshape(-1), 0, primes_idx0, poly_num, mod_num, mod_num)
    buf.upload(data)
    pair.dev.FromNTTInplace(buf, 0, primes_idx0, poly_num, mod_num, mod_num)
    assert np.array_equal(from_dev(buf, data.shape), want_inv)
    buf.free()



def needs_extra_forms(dev):
    """Launch forms 2 (chained) and 3 (one workgroup per limb) exist only in a library built with EXTRA_FORMS=1."""
    if not dev.info("ntt_extra_forms"):
        pytest.skip("library built without the extra launch forms (make EXTRA_FORMS=1)")


def test_config1_n4096_4primes_batch16():
    """BASELINE config 1: N = 2^12, 4 primes < 2^36, batch of 16 polynomials, seed 1."""
    pair = Pair(12, [], CFG1_Q)
    for mode in (0, 1):       # FP64 back end, integer back end
        check_fwd_inv(pair, 0, CFG1_Q, 16, seed=1, mode=mode)


@pytest.mark.parametrize("logN", [8, 9, 10, 11, 13, 14, 15])
def test_all_ring_sizes(logN):
    q = CFG2_Q[:3]
    pair = Pair(logN, [], q)
    for mode in (0, 1):
        check_fwd_inv(pair, 0, q, 3, seed=logN, mode=mode)


def test_config2_one_ciphertext_n65536_24primes():
    """BASELINE config 2: N = 2^16, 24 primes, one ciphertext = 2 polys x 24 limbs, seed 2."""
    pair = Pair(16, [], CFG2_Q)
    check_fwd_inv(pair, 0, CFG2_Q, 2, seed=2, mode=0)


def test_n65536_integer_backend_and_large_primes():
    """The reference's logN = 16 set (Params.cuh:88-171): its 49-bit q and p primes take the FP64 back end that balances after every
    register round, its 60-bit t primes the integer back end; a call over [p | q | t] goes out as one launch sequence per run of
    primes of one back end.  Both arithmetic modes against the oracle."""
    P = REF_PARAMS[16]
    p, q, t = P["p"][:1], P["q"][:2], P["t"][:2]
    pair = Pair(16, p, q, t, gamma=2)
    for mode in (0, 1):
        check_fwd_inv(pair, 0, p + q + t, 1, seed=3, mode=mode)
        check_fwd_inv(pair, 0, p + q, 2, seed=5, mode=mode)
    # 36-bit primes through the integer back end as well
    pair2 = Pair(16, [], CFG2_Q[:2])
    check_fwd_inv(pair2, 0, CFG2_Q[:2], 2, seed=4, mode=1)


@pytest.mark.parametrize("logN", [8, 11, 12, 14, 15, 16])
def test_wide_fp64_backend_at_its_range_ends(logN):
    """FP64 butterflies for primes of 41 to 50 bits: the two largest NTT-friendly primes below 2^50 (every bound of the range analysis
    is tightest there), a 49-bit prime of the reference and the smallest prime the back end takes (just above 2^41), on uniform residues
    and on the inputs that drive every butterfly to the ends of its range: all q - 1, alternating 0 / q - 1, alternating 1 / q - 1 in
    blocks, all against the oracle in both directions."""
    from ckks_llm_amd.params import small_primes
    top = small_primes(50, 1 << 17, 2)
    low = small_primes(42, 1 << 17, 1)
    assert all((1 << 49) < m < (1 << 50) for m in top) and (1 << 41) <= low[0] < (1 << 42)
    primes = top + [REF_PARAMS[16]["q"][0]] + low
    pair = Pair(logN, [], primes)
    pair.dev.set_arith_mode(0)
    N = pair.N
    check_fwd_inv(pair, 0, primes, 2, seed=40 + logN, mode=0)
    pats = []
    for kind in range(4):
        d = np.empty((1, len(primes), N), dtype=np.uint64)
        for j, m in enumerate(primes):
            if kind == 0:
                d[0, j] = m - 1
            elif kind == 1:
                d[0, j] = np.where(np.arange(N) % 2 == 0, 0, m - 1)
            elif kind == 2:
                d[0, j] = np.where((np.arange(N) // 16) % 2 == 0, 1, m - 1)
            else:
                d[0, j] = np.where(np.arange(N) % 3 == 0, m // 2, m // 2 + 1)
        pats.append(d)
    for d in pats:
        for inverse in (False, True):
            want = d.copy()
            (pair.orc.FromNTTInplace if inverse else pair.orc.ToNTTInplace)(want.reshape(-1), 0, 0, 1, len(primes), len(primes))
            buf = to_dev(d)
            (pair.dev.FromNTTInplace if inverse else pair.dev.ToNTTInplace)(buf, 0, 0, 1, len(primes), len(primes))
            assert np.array_equal(from_dev(buf, d.shape), want), (logN, inverse)
            buf.free()


def test_n65536_inter_pass_formats():
    """N = 2^16, FP64 back end: primes below 2^39 take the 5-byte inter-pass buffer, 40-bit primes the in-place 8-byte form, and
    ntt_mode 1 forces the in-place form; all against the oracle.  A batch wider than one launch chunk is not needed: chunks
    only re-use the buffer in stream order."""
    from ckks_llm_amd.params import small_primes
    q40 = small_primes(40, 1 << 17, 2)
    assert all((1 << 39) <= p < (1 << 41) for p in q40)
    pair = Pair(16, [], CFG2_Q[:3] + q40)
    check_fwd_inv(pair, 0, CFG2_Q[:3], 3, seed=21, mode=0)            # compact
    check_fwd_inv(pair, 3, q40, 2, seed=22, mode=0)                   # FP64, in place
    check_fwd_inv(pair, 0, CFG2_Q[:3] + q40, 1, seed=23, mode=0)      # mixed call: in place
    pair.dev.set_ntt_mode(1)
    check_fwd_inv(pair, 0, CFG2_Q[:3], 3, seed=24, mode=0)            # forced in place
    # maximal and minimal residues through the 40-bit codec
    N = pair.N
    pair.dev.set_ntt_mode(0)
    data = np.stack([np.full(N, p - 1, dtype=np.uint64) for p in CFG2_Q[:3]])[None].copy()
    data[0, :, ::2] = 0
    want = data.copy()
    pair.orc.ToNTTInplace(want.reshape(-1), 0, 0, 1, 3, 5)
    d = to_dev(data)
    pair.dev.ToNTTInplace(d, 0, 0, 1, 3, 5)
    assert np.array_equal(from_dev(d, data.shape), want)


def test_reference_addressing_and_ext_variant():
    """start_poly_idx / start_mod_idx / poly_mod_len addressing (ntt_60bit.cuh:446-455) and the batch stride of the
    _for_externalProduct variants (ntt_60bit.cuh:913-934)."""
    P = REF_PARAMS[14]
    p, q, t = P["p"], P["q"][:4], P["t"][:3]
    pair = Pair(12, p, q, t, gamma=3)
    N, K = pair.N, len(p)
    rng = np.random.default_rng(5)
    buf_h = rng.integers(0, 1 << 35, size=(3, 7, N), dtype=np.uint64)          # 3 polys, poly_mod_len 7
    want = buf_h.copy()
    pair.orc.ToNTTInplace(want.reshape(-1), 2, K + 1, 3, 3, 7)                  # limbs 2..4 of each poly, primes q1..q3
    d = to_dev(buf_h)
    pair.dev.ToNTTInplace(d, 2, K + 1, 3, 3, 7)
    got = from_dev(d, buf_h.shape)
    assert np.array_equal(got, want)
    assert np.array_equal(got[:, :2], buf_h[:, :2]) and np.array_equal(got[:, 5:], buf_h[:, 5:])
    pair.dev.FromNTTInplace(d, 2, K + 1, 3, 3, 7)
    assert np.array_equal(from_dev(d, buf_h.shape), buf_h)
    # ext: batch 2, stride 9 limbs, 2 polys x 3 T-limbs
    T0 = K + len(q)
    e_h = rng.integers(0, 1 << 59, size=(2, 9, N), dtype=np.uint64)
    for j in range(9):
        e_h[:, j] %= np.uint64(t[j % 3])
    want = e_h.copy()
    pair.orc.ToNTTInplace_for_externalProduct(want.reshape(-1), 0, T0, 2, 3, 3, 9, 2)
    d2 = to_dev(e_h)
    pair.dev.ToNTTInplace_for_externalProduct(d2, 0, T0, 2, 3, 3, 9, 2)
    assert np.array_equal(from_dev(d2, e_h.shape), want)
    pair.orc.FromNTTInplace_for_externalProduct(want.reshape(-1), 0, T0, 2, 3, 3, 9, 2)
    pair.dev.FromNTTInplace_for_externalProduct(d2, 0, T0, 2, 3, 3, 9, 2)
    assert np.array_equal(from_dev(d2, e_h.shape), want) and np.array_equal(want, e_h)


@pytest.mark.parametrize("logN,polys,mode", [(16, 9, 0), (16, 5, 1), (15, 7, 0), (15, 3, 1)])
def test_one_launch_transform_matches_two_launch_and_oracle(logN, polys, mode):
    """The chained transform (ntt_mode 2: both passes in one launch, the second pass of a limb behind its first pass on the
    same XCD) against the oracle, both directions, both arithmetic back ends; launches in a row reuse the completion
    words that the finishing launch returns to zero."""
    q = CFG2_Q[:5]
    pair = Pair(logN, [], q)
    N, L1 = pair.N, len(q)
    needs_extra_forms(pair.dev)
    pair.dev.set_arith_mode(mode)
    data = limbs_uniform(40 + logN, q, polys, N)
    want = data.copy()
    pair.orc.ToNTTInplace(want.reshape(-1), 0, 0, polys, L1, L1)
    want_inv = data.copy()
    pair.orc.FromNTTInplace(want_inv.reshape(-1), 0, 0, polys, L1, L1)
    pair.dev.set_ntt_mode(2)
    buf = to_dev(data)
    pair.dev.ToNTTInplace(buf, 0, 0, polys, L1, L1)
    pair.dev.check()
    assert np.array_equal(from_dev(buf, data.shape), want)
    pair.dev.FromNTTInplace(buf, 0, 0, polys, L1, L1)
    pair.dev.check()
    assert np.array_equal(from_dev(buf, data.shape), data)
    pair.dev.FromNTTInplace(buf, 0, 0, polys, L1, L1)
    pair.dev.check()
    assert np.array_equal(from_dev(buf, data.shape), want_inv)
    # a sub-range of limbs with the reference addressing: primes 1..3 of polys 0..polys-1
    buf.upload(data)
    pair.dev.ToNTTInplace(buf, 1, 1, polys, 3, L1)
    pair.dev.check()
    got = from_dev(buf, data.shape)
    assert np.array_equal(got[:, 1:4], want[:, 1:4]) and np.array_equal(got[:, 0], data[:, 0]) and np.array_equal(got[:, 4], data[:, 4])
    buf.free()


@pytest.mark.parametrize("logN,polys,mode", [(16, 9, 0), (16, 5, 1), (15, 7, 0), (15, 3, 1)])
def test_whole_limb_transform_matches_oracle(logN, polys, mode):
    """One workgroup per limb, both passes in one launch (ntt_mode 3): against the oracle, both directions, both arithmetic
    back ends, and with the reference's sub-range addressing."""
    q = CFG2_Q[:5]
    pair = Pair(logN, [], q)
    N, L1 = pair.N, len(q)
    needs_extra_forms(pair.dev)
    pair.dev.set_arith_mode(mode)
    data = limbs_uniform(40 + logN, q, polys, N)
    want = data.copy()
    pair.orc.ToNTTInplace(want.reshape(-1), 0, 0, polys, L1, L1)
    want_inv = data.copy()
    pair.orc.FromNTTInplace(want_inv.reshape(-1), 0, 0, polys, L1, L1)
    pair.dev.set_ntt_mode(3)
    buf = to_dev(data)
    pair.dev.ToNTTInplace(buf, 0, 0, polys, L1, L1)
    assert np.array_equal(from_dev(buf, data.shape), want)
    pair.dev.FromNTTInplace(buf, 0, 0, polys, L1, L1)
    assert np.array_equal(from_dev(buf, data.shape), data)
    pair.dev.FromNTTInplace(buf, 0, 0, polys, L1, L1)
    assert np.array_equal(from_dev(buf, data.shape), want_inv)
    buf.upload(data)
    pair.dev.ToNTTInplace(buf, 1, 1, polys, 3, L1)
    got = from_dev(buf, data.shape)
    assert np.array_equal(got[:, 1:4], want[:, 1:4]) and np.array_equal(got[:, 0], data[:, 0]) and np.array_equal(got[:, 4], data[:, 4])
    buf.free()


@pytest.mark.parametrize("polys,mode", [(11, 6), (19, 0), (12, 0), (53, 0)])
def test_resident_transform_matches_oracle(polys, mode):
    """The resident transform (one persistent workgroup per compute unit carries whole limbs through both passes in its registers;
    N = 2^16, primes below 2^36, at least 256 limbs) against the oracle, both directions and the reference's sub-range addressing:
    264 limbs (a full round and a few), 456 (a second round three quarters full: all resident), 288 (the 32 limbs beyond the first
    round go out as two launches), 1272 (five rounds less eight limbs)."""
    q = CFG2_Q
    pair = Pair(16, [], q)
    N, L1 = pair.N, len(q)
    data = limbs_uniform(600 + polys, q, polys, N)
    want = data.copy()
    pair.orc.ToNTTInplace(want.reshape(-1), 0, 0, polys, L1, L1)
    want_inv = data.copy()
    pair.orc.FromNTTInplace(want_inv.reshape(-1), 0, 0, polys, L1, L1)
    pair.dev.set_ntt_mode(mode)
    buf = to_dev(data)
    for _ in range(2):
        pair.dev.ToNTTInplace(buf, 0, 0, polys, L1, L1)
        assert np.array_equal(from_dev(buf, data.shape), want)
        pair.dev.FromNTTInplace(buf, 0, 0, polys, L1, L1)
        assert np.array_equal(from_dev(buf, data.shape), data)
    pair.dev.FromNTTInplace(buf, 0, 0, polys, L1, L1)
    assert np.array_equal(from_dev(buf, data.shape), want_inv)
    # limbs 1 .. 22 of every polynomial (the first and the last stay as they are)
    buf.upload(data)
    pair.dev.ToNTTInplace(buf, 1, 1, polys, L1 - 2, L1)
    got = from_dev(buf, data.shape)
    assert np.array_equal(got[:, 1:L1 - 1], want[:, 1:L1 - 1]) and np.array_equal(got[:, 0], data[:, 0]) and np.array_equal(got[:, L1 - 1], data[:, L1 - 1])
    buf.free()


@pytest.mark.parametrize("primes,polys,arith,mode", [("36", 9, 0, 4), ("36", 5, 1, 4), ("49", 3, 0, 4), ("mixed", 2, 0, 4), ("36", 1, 0, 4),
                                                    ("36", 7, 0, 5), ("49", 2, 0, 5), ("36", 3, 1, 5), ("36", 8, 0, 0), ("36", 11, 0, 0)])
def test_paired_transform_matches_oracle(primes, polys, arith, mode):
    """The paired transform (both passes in one launch, a workgroup per (limb, tile) that waits between its two tiles for the
    limb's first pass) against the oracle: 5-byte and in-place inter-pass forms, all three arithmetic back ends, limb counts
    that are no multiple of eight, several launches in a row on the same completion words, the reference's sub-range
    addressing.  Mode 5 spreads the tiles of a limb over all XCDs, so that what one pass hands to the other really crosses
    from one L2 to another; mode 0 with 40 and with 55 limbs is the automatic choice of the two numberings."""
    q = {"36": CFG2_Q[:5], "49": REF_PARAMS[16]["q"][:5], "mixed": CFG2_Q[:2] + REF_PARAMS[16]["q"][:2] + REF_PARAMS[16]["t"][:1]}[primes]
    pair = Pair(16, [], q)
    N, L1 = pair.N, len(q)
    pair.dev.set_arith_mode(arith)
    data = limbs_uniform(140 + polys, q, polys, N)
    want = data.copy()
    pair.orc.ToNTTInplace(want.reshape(-1), 0, 0, polys, L1, L1)
    want_inv = data.copy()
    pair.orc.FromNTTInplace(want_inv.reshape(-1), 0, 0, polys, L1, L1)
    pair.dev.set_ntt_mode(mode)
    buf = to_dev(data)
    for _ in range(3):
        pair.dev.ToNTTInplace(buf, 0, 0, polys, L1, L1)
        pair.dev.check()
        assert np.array_equal(from_dev(buf, data.shape), want)
        pair.dev.FromNTTInplace(buf, 0, 0, polys, L1, L1)
        pair.dev.check()
        assert np.array_equal(from_dev(buf, data.shape), data)
    pair.dev.FromNTTInplace(buf, 0, 0, polys, L1, L1)
    pair.dev.check()
    assert np.array_equal(from_dev(buf, data.shape), want_inv)
    buf.upload(data)
    pair.dev.ToNTTInplace(buf, 1, 1, polys, 3, L1)
    pair.dev.check()
    got = from_dev(buf, data.shape)
    assert np.array_equal(got[:, 1:4], want[:, 1:4]) and np.array_equal(got[:, 0], data[:, 0]) and np.array_equal(got[:, 4], data[:, 4])
    buf.free()


@pytest.mark.parametrize("mode,arith,polys", [(4, 0, 2), (5, 0, 3), (4, 1, 2), (0, 0, 6)])
def test_paired_transform_completes_when_every_wait_runs_out(mode, arith, polys):
    """With a poll limit of zero a workgroup of the paired transform never waits: it takes over whatever first-pass tiles nobody
    has claimed and, unless its limb is complete at the first look, leaves its second-pass tiles to the last workgroup of the limb
    to leave.  The transform must still come out right, in place and through the 5-byte form, on both back ends, again and again
    on the same protocol words, and the context stays usable; the counter of left-over tiles says that the path was taken."""
    q = CFG2_Q[:3]
    pair = Pair(16, [], q)
    pair.dev.set_arith_mode(arith)
    data = limbs_uniform(5, q, polys, pair.N)
    want = data.copy()
    pair.orc.ToNTTInplace(want.reshape(-1), 0, 0, polys, 3, 3)
    buf = to_dev(data)
    pair.dev.set_ntt_mode(mode)
    pair.dev.set_ntt_chain(0, 0)
    before = pair.dev.info("ntt_pair_deferred_tiles")
    for rep in range(3):
        pair.dev.ToNTTInplace(buf, 0, 0, polys, 3, 3)
        pair.dev.check()
        assert np.array_equal(from_dev(buf, data.shape), want), rep
        pair.dev.FromNTTInplace(buf, 0, 0, polys, 3, 3)
        pair.dev.check()
        assert np.array_equal(from_dev(buf, data.shape), data), rep
    assert pair.dev.info("ntt_pair_deferred_tiles") > before
    # back to the default limits: same words, nothing left over from the forced runs
    pair.dev.set_ntt_chain(0, -1)
    pair.dev.ToNTTInplace(buf, 0, 0, polys, 3, 3)
    pair.dev.check()
    assert np.array_equal(from_dev(buf, data.shape), want)
    buf.free()


def test_paired_transform_larger_than_the_chip_holds():
    """A paired launch with several times more workgroups than fit the chip at once (mode 4 forces the form at any size): the
    protocol does not need the workgroups of a limb to be resident together."""
    q = CFG2_Q[:6]
    pair = Pair(16, [], q)
    polys = 2 * (pair.dev.info("ntt_pair_resident_blocks") // 16) // len(q) + 3
    assert 16 * polys * len(q) > pair.dev.info("ntt_pair_resident_blocks")
    data = limbs_uniform(17, q, polys, pair.N)
    want = data.copy()
    pair.orc.ToNTTInplace(want.reshape(-1), 0, 0, polys, len(q), len(q))
    buf = to_dev(data)
    for mode in (4, 5):
        pair.dev.set_ntt_mode(mode)
        buf.upload(data)
        pair.dev.ToNTTInplace(buf, 0, 0, polys, len(q), len(q))
        pair.dev.check()
        assert np.array_equal(from_dev(buf, data.shape), want), mode
        pair.dev.FromNTTInplace(buf, 0, 0, polys, len(q), len(q))
        pair.dev.check()
        assert np.array_equal(from_dev(buf, data.shape), data), mode
    buf.free()


def test_paired_transforms_of_two_contexts_on_two_streams():
    """Two contexts, each on a stream of its own, run paired transforms at the same time (each context has its own completion
    words); twenty rounds in flight without a synchronisation, then both results against the oracle."""
    import ctypes
    hip = ctypes.CDLL("libamdhip64.so")
    q = CFG2_Q[:4]
    pairs = [Pair(16, [], q), Pair(16, [], q)]
    streams = []
    for p_ in pairs:
        s = ctypes.c_void_p()
        assert hip.hipStreamCreate(ctypes.byref(s)) == 0
        p_.dev.set_stream(s)
        streams.append(s)
    N, L1 = pairs[0].N, len(q)
    datas = [limbs_uniform(300 + i, q, 2 + i, N) for i in range(2)]
    wants = []
    for p_, d in zip(pairs, datas):
        w = d.copy()
        p_.orc.ToNTTInplace(w.reshape(-1), 0, 0, d.shape[0], L1, L1)
        wants.append(w)
    bufs = [to_dev(d) for d in datas]
    for p_ in pairs:
        p_.dev.check()                       # uploads done before the streams start
    for _ in range(10):
        for p_, b, d in zip(pairs, bufs, datas):
            p_.dev.ToNTTInplace(b, 0, 0, d.shape[0], L1, L1)
        for p_, b, d in zip(pairs, bufs, datas):
            p_.dev.FromNTTInplace(b, 0, 0, d.shape[0], L1, L1)
    for p_, b, d in zip(pairs, bufs, datas):
        p_.dev.ToNTTInplace(b, 0, 0, d.shape[0], L1, L1)
    for p_ in pairs:
        p_.dev.check()
    for b, d, w in zip(bufs, datas, wants):
        assert np.array_equal(from_dev(b, d.shape), w)
        b.free()
    for p_, s in zip(pairs, streams):
        p_.dev.set_stream(None)
        assert hip.hipStreamDestroy(s) == 0


@pytest.mark.parametrize("skew,spin", [(1, 0), (3, 0), (2, -1), (64, -1)])
def test_chained_transform_finishing_launch_and_skews(skew, spin):
    """With a poll limit of zero every second-pass workgroup of the chained transform leaves its tile to the finishing launch,
    which must then produce the whole second pass; any skew gives the same residues.  13 limbs: chains of unequal length."""
    q = CFG2_Q[:13]
    pair = Pair(16, [], q)
    N, L1 = pair.N, len(q)
    data = limbs_uniform(77, q, 1, N)
    want = data.copy()
    pair.orc.ToNTTInplace(want.reshape(-1), 0, 0, 1, L1, L1)
    needs_extra_forms(pair.dev)
    pair.dev.set_ntt_mode(2)
    pair.dev.set_ntt_chain(skew, spin)
    buf = to_dev(data)
    before = pair.dev.info("ntt_chain_deferred_tiles")
    pair.dev.ToNTTInplace(buf, 0, 0, 1, L1, L1)
    pair.dev.check()
    assert np.array_equal(from_dev(buf, data.shape), want)
    pair.dev.FromNTTInplace(buf, 0, 0, 1, L1, L1)
    pair.dev.check()
    assert np.array_equal(from_dev(buf, data.shape), data)
    left = pair.dev.info("ntt_chain_deferred_tiles") - before
    if spin == 0:
        assert left == 2 * 13 * 16          # every second-pass tile of both transforms
    buf.free()


def test_tables_match_oracle():
    P = REF_PARAMS[14]
    pair = Pair(10, P["p"], P["q"], P["t"], P["gamma"])
    for name in ["pqt", "mu_hi", "mu_lo", "psi", "psiinv", "n_inv", "n_inv_shoup", "halfTmodpqti", "psi_table",
                 "psiinv_table", "psi_shoup_table", "psiinv_shoup_table", "pHatVecModq", "pHatInvVecModp", "PModqt",
                 "PinvModq", "RiHatInv", "RiHatModT", "Rimodti", "QjHatInv", "QjHatModT", "Qjmodti", "THatInv",
                 "THatModRi", "Tmodpqi", "qiInvModql"]:
        assert np.array_equal(pair.dev.table(name), pair.orc.table(name)), name


def test_edge_cases_and_errors():
    from ckks_llm_amd import CkksError, Context_23
    pair = Pair(10, [], CFG2_Q[:2])
    d = to_dev(np.zeros((1, 2, pair.N), dtype=np.uint64))
    pair.dev.ToNTTInplace(d, 0, 0, 0, 2, 2)          # empty batch: no work, no error
    pair.dev.ToNTTInplace(d, 0, 0, 1, 0, 2)
    assert not from_dev(d, (2, pair.N)).any()
    pair.dev.ToNTTInplace(d, 0, 0, 1, 2, 2)          # NTT(0) = 0
    assert not from_dev(d, (2, pair.N)).any()
    with pytest.raises(CkksError):
        pair.dev.ToNTTInplace(d, 0, 1, 1, 2, 2)      # prime range outside the context
    with pytest.raises(CkksError):
        Context_23(10, [], [CFG2_Q[0] + 2])          # not 1 mod 2N
    with pytest.raises(CkksError):
        Context_23(17, [], CFG2_Q[:1])               # unsupported ring size
    # maximal residues q-1 everywhere
    data = np.stack([np.full(pair.N, q - 1, dtype=np.uint64) for q in CFG2_Q[:2]])[None]
    want = data.copy()
    pair.orc.ToNTTInplace(want.reshape(-1), 0, 0, 1, 2, 2)
    d.upload(data)
    pair.dev.ToNTTInplace(d, 0, 0, 1, 2, 2)
    assert np.array_equal(from_dev(d, data.shape), want)


def test_marks_between_launches():
    """ckks_timer_mark / ckks_timer_between: marks recorded between launches queued back to back give each launch's duration
    afterwards; the intervals add up, and a slot that was never marked or lies outside the range is refused."""
    from ckks_llm_amd import CkksError
    pair = Pair(16, [], CFG2_Q[:4])
    d = to_dev(limbs_uniform(5, CFG2_Q[:4], 2, pair.N))
    for i in range(4):
        pair.dev.timer_mark(i)
        (pair.dev.ToNTTInplace if i % 2 == 0 else pair.dev.FromNTTInplace)(d, 0, 0, 2, 4, 4)
    pair.dev.timer_mark(4)
    parts = [pair.dev.timer_between(i, i + 1) for i in range(4)]
    assert all(0.0 < t < 50.0 for t in parts), parts
    assert abs(sum(parts) - pair.dev.timer_between(0, 4)) < 0.02 * len(parts) + 0.05 * sum(parts)
    with pytest.raises(CkksError):
        pair.dev.timer_between(0, 9)                 # never marked
    with pytest.raises(CkksError):
        pair.dev.timer_mark(4096)                    # outside 0 .. 4095
    with pytest.raises(CkksError):
        pair.dev.timer_mark(-1)


def test_full_size_properties_batch32():
    """BASELINE config 2 at batch 32 (768 MiB): size-independent properties instead of a full oracle run:
    round trip, linearity on a sampled pair, and oracle parity on one sampled ciphertext."""
    pair = Pair(16, [], CFG2_Q)
    N, L1, B = pair.N, 24, 32
    rng = np.random.default_rng(2)
    data = np.empty((2 * B, L1, N), dtype=np.uint64)
    for j, q in enumerate(CFG2_Q):
        data[:, j, :] = rng.integers(0, q, size=(2 * B, N), dtype=np.uint64)
    d = to_dev(data)
    pair.dev.ToNTTInplace(d, 0, 0, 2 * B, L1, L1)
    got = from_dev(d, data.shape)
    # parity on one sampled ciphertext (2 polys)
    y = 17
    want = data[y:y + 2].copy()
    pair.orc.ToNTTInplace(want.reshape(-1), 0, 0, 2, L1, L1)
    assert np.array_equal(got[y:y + 2], want)
    # linearity: NTT(a) + NTT(b) == NTT(a + b) for polys 0 and 1 (checked on the device transform of the sum)
    s = np.empty((1, L1, N), dtype=np.uint64)
    for j, q in enumerate(CFG2_Q):
        s[0, j] = (data[0, j] + data[1, j]) % np.uint64(q)
    ds = to_dev(s)
    pair.dev.ToNTTInplace(ds, 0, 0, 1, L1, L1)
    fs = from_dev(ds, s.shape)
    for j, q in enumerate(CFG2_Q):
        assert np.array_equal(fs[0, j], (got[0, j] + got[1, j]) % np.uint64(q))
    pair.dev.FromNTTInplace(d, 0, 0, 2 * B, L1, L1)
    pair.dev.check()
    assert np.array_equal(from_dev(d, data.shape), data)
    # the other launch forms give the same residues on the whole batch (the paired form far beyond what the chip holds at once)
    for m in (1, 4, 5) + ((2, 3) if pair.dev.info("ntt_extra_forms") else ()):
        pair.dev.set_ntt_mode(m)
        pair.dev.ToNTTInplace(d, 0, 0, 2 * B, L1, L1)
        assert np.array_equal(from_dev(d, data.shape), got), m
        pair.dev.FromNTTInplace(d, 0, 0, 2 * B, L1, L1)
