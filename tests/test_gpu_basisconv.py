"""GPU parity: RNS basis conversions, ModDown, external / inner product, rescale and both key-switch chains
through the C ABI against the CPU oracle, bit-exact on every residue."""
import numpy as np
import pytest

from ckks_llm_amd import DeviceBuffer
from tests.gpu_common import Pair, to_dev, from_dev
from tests.helpers import limbs_uniform
from tests.params import CFG2_Q, CFG3_P, REF_PARAMS

pytestmark = pytest.mark.gpu


def ref_pair(params, logN):
    P = REF_PARAMS[params]
    return Pair(logN, P["p"], P["q"], P["t"], P["gamma"])


@pytest.mark.parametrize("params,logN", [(13, 10), (14, 12), (15, 11), (16, 10)])
def test_four_conversion_maps(params, logN):
    pair = ref_pair(params, logN)
    o, d, N = pair.orc, pair.dev, pair.N
    K, Q, T, RB, QB = o.p_num, o.q_num, o.t_num, o.Ri_blockNum, o.Qj_blockNum
    pq = o.p + o.q
    for l in sorted({o.L, o.L - 1, o.L // 2, 0}):
        batch = 2
        # [P|Q] -> T  (modUpPQtoT_23)
        inp = limbs_uniform(100 + l, pq, batch, N)
        want = np.zeros((batch, RB * T, N), dtype=np.uint64)
        o.modUpPQtoT_23(want.reshape(-1), inp.reshape(-1), l, batch)
        dout = to_dev(np.zeros_like(want))
        din = to_dev(inp)
        d.modUpPQtoT_23(dout, din, l, batch)
        assert np.array_equal(from_dev(dout, want.shape), want), ("pq_to_t", l)
        # Q digit -> T  (modUpQjtoT_23); corner values in the first columns
        inq = limbs_uniform(200 + l, o.q, batch, N)
        inq[:, :, 0] = 0
        for j, q in enumerate(o.q):
            inq[:, j, 1] = q - 1
            inq[:, j, 2] = 1
        want = np.zeros((batch, QB * T, N), dtype=np.uint64)
        o.modUpQjtoT_23(want.reshape(-1), inq.reshape(-1), l, batch)
        dout2 = to_dev(np.zeros_like(want))
        d.modUpQjtoT_23(dout2, to_dev(inq), l, batch)
        assert np.array_equal(from_dev(dout2, want.shape), want), ("qj_to_t", l)
        # T -> [P|Q_l]  (modUpTtoPQl_23), then ModDown (modDownPQltoQl_23)
        int_ = np.zeros((batch, RB * T, N), dtype=np.uint64)
        rng = np.random.default_rng(300 + l)
        for k in range(RB * T):
            int_[:, k, :] = rng.integers(0, o.t[k % T], size=(batch, N), dtype=np.uint64)
        int_[:, :, 0] = 0
        want = np.zeros((batch, RB * T, N), dtype=np.uint64)
        o.modUpTtoPQl_23(want.reshape(-1), int_.reshape(-1), l, batch)
        dbuf = to_dev(np.zeros_like(want))
        d.modUpTtoPQl_23(dbuf, to_dev(int_), l, batch)
        got = from_dev(dbuf, want.shape)
        assert np.array_equal(got[:, :K + l + 1], want[:, :K + l + 1]), ("t_to_pql", l)
        wdown = np.zeros((batch, Q, N), dtype=np.uint64)
        o.modDownPQltoQl_23(wdown.reshape(-1), want.reshape(-1), l, batch)
        ddown = to_dev(np.zeros_like(wdown))
        d.modDownPQltoQl_23(ddown, to_dev(want), l, batch)
        assert np.array_equal(from_dev(ddown, wdown.shape)[:, :l + 1], wdown[:, :l + 1]), ("moddown", l)


@pytest.mark.parametrize("params", [14, 15])
def test_external_product_swk_reuse(params):
    """Context_23::external_product_T_swk_reuse (ExternalProduct.cuh:103-162) against the oracle for 1, 3 and 8 digit sets."""
    pair = ref_pair(params, 12)
    o, d, N = pair.orc, pair.dev, pair.N
    K, T, RB, QB, dnum, L = o.p_num, o.t_num, o.Ri_blockNum, o.Qj_blockNum, o.dnum, o.L
    swk = limbs_uniform(70, o.t, 2 * dnum * RB, N)
    dswk = to_dev(swk)
    for l, batch in ((L, 3), (L - 1, 8), (1, 1)):
        cT = limbs_uniform(71 + l, o.t, batch * QB, N)
        want = np.zeros((2 * batch, RB * T, N), dtype=np.uint64)
        o.external_product_T_swk_reuse(want.reshape(-1), cT.reshape(-1), swk.reshape(-1), l, batch)
        dout = to_dev(np.zeros_like(want))
        d.external_product_T_swk_reuse(dout, to_dev(cT), dswk, l, batch)
        nblk = -(-(K + l + 1) // o.gamma)
        got = from_dev(dout, want.shape)
        assert np.array_equal(got[:, :nblk * T], want[:, :nblk * T]), (l, batch)
        assert not got[:, nblk * T:].any()                                    # blocks beyond the level stay untouched
    with pytest.raises(Exception):
        d.external_product_T_swk_reuse(dout, to_dev(cT), dswk, 1, 9)
    with pytest.raises(Exception):
        d.external_product_T_swk_reuse(dout, to_dev(cT), dswk, 1, 0)


@pytest.mark.parametrize("params", [14, 15])
def test_external_product_and_keyswitch_23(params):
    pair = ref_pair(params, 12)
    o, d, N = pair.orc, pair.dev, pair.N
    K, Q, T, RB, QB, dnum, L = o.p_num, o.q_num, o.t_num, o.Ri_blockNum, o.Qj_blockNum, o.dnum, o.L
    swk = limbs_uniform(7, o.t, 2 * dnum * RB, N)                     # [2][dnum][RB][T][N] uniform in T
    dswk = to_dev(swk)
    for l in (L, L - 1, 1):
        cT = limbs_uniform(8 + l, o.t, QB, N)
        want = np.zeros((2, RB * T, N), dtype=np.uint64)
        o.external_product_T(want.reshape(-1), cT.reshape(-1), swk.reshape(-1), l)
        dout = to_dev(np.zeros_like(want))
        d.external_product_T(dout, to_dev(cT), dswk, l)
        nblk = -(-(K + l + 1) // o.gamma)
        got = from_dev(dout, want.shape)
        assert np.array_equal(got[:, :nblk * T], want[:, :nblk * T]), ("external_product", l)
        # whole chain (steps 2..9 of mult_23)
        d2 = np.zeros((Q, N), dtype=np.uint64)
        d2[:l + 1] = limbs_uniform(20 + l, o.q[:l + 1], 1, N)[0]
        wout = np.zeros((2, Q, N), dtype=np.uint64)
        o.keyswitch_23(wout.reshape(-1), d2.reshape(-1), swk.reshape(-1), l)
        dd2, do = to_dev(d2), to_dev(np.zeros_like(wout))
        s1 = DeviceBuffer(8 * N * T * QB)
        s2 = DeviceBuffer(8 * N * T * RB * 2)
        s3 = DeviceBuffer(8 * N * T * RB * 2)
        s1.zero(); s2.zero(); s3.zero()
        d.keyswitch_23(do, dd2, dswk, l, s1, s2, s3)
        assert np.array_equal(from_dev(do, wout.shape)[:, :l + 1], wout[:, :l + 1]), ("keyswitch_23", l)


@pytest.mark.parametrize("primes", ["36", "49"])
def test_keyswitch_23_full_ring(primes):
    """The T-basis switch at N = 2^16 with the reference's 60-bit T primes over P and Q primes below 2^39 (36- and 37-bit) and over
    the reference's own 49- and 50-bit P and Q primes: at this size its external product runs in one launch with the row pass of
    the sums' inverse transform, and its ModDown inside the first pass of the final transform (handing over 5-byte values below
    2^39, whole limbs on the wide FP64 arithmetic above); same words as the oracle's separate steps, and as the device's own
    separate steps (ntt mode 1); the same for a whole multiplication, whose additions then leave with the last launch.  Three T primes here: the launch's numbering of its workgroups is exercised away from the
    eight primes it is laid out for."""
    q, p, t = CFG2_Q[:6], CFG3_P[:2], REF_PARAMS[16]["t"][:3]      # q_num a multiple of p_num, as in every set of the reference
    if primes == "49":
        q, p = REF_PARAMS[16]["q"][:6], REF_PARAMS[16]["p"][:2]
    pair = Pair(16, p, q, t, 3)
    o, d, N = pair.orc, pair.dev, pair.N
    Q, T, RB, QB, dnum, L = o.q_num, o.t_num, o.Ri_blockNum, o.Qj_blockNum, o.dnum, o.L
    swk = limbs_uniform(7, t, 2 * dnum * RB, N)
    dswk = to_dev(swk)
    for l in (L, 2, 1):                                            # three digits, two, one (the product's two-deep read-ahead at its ends)
        d2 = np.zeros((Q, N), dtype=np.uint64)
        d2[:l + 1] = limbs_uniform(20 + l, q[:l + 1], 1, N)[0]
        wout = np.zeros((2, Q, N), dtype=np.uint64)
        o.keyswitch_23(wout.reshape(-1), d2.copy().reshape(-1), swk.reshape(-1), l)
        for mode in (0, 1):
            d.set_ntt_mode(mode)
            dd2, do = to_dev(d2), to_dev(np.zeros_like(wout))
            s1, s2, s3 = DeviceBuffer(8 * N * T * QB), DeviceBuffer(8 * N * T * RB * 2), DeviceBuffer(8 * N * T * RB * 2)
            s1.zero(); s2.zero(); s3.zero()
            d.keyswitch_23(do, dd2, dswk, l, s1, s2, s3)
            assert np.array_equal(from_dev(do, wout.shape)[:, :l + 1], wout[:, :l + 1]), (l, mode)
        # the whole multiplication (KeySwitch_23.cuh:192-236): at this size its two closing additions ride on the last launch of
        # the key switch (mode 0) or run as a launch of their own (mode 1)
        c1, c2 = limbs_uniform(40 + l, q, 2, N), limbs_uniform(50 + l, q, 2, N)
        wm = np.zeros((2, Q, N), dtype=np.uint64)
        o.mult_23(wm.reshape(-1), c1.reshape(-1), c2.reshape(-1), swk.reshape(-1), l)
        dc1, dc2 = to_dev(c1), to_dev(c2)
        for mode in (0, 1):
            d.set_ntt_mode(mode)
            dm, work = to_dev(np.zeros_like(wm)), DeviceBuffer(8 * N * Q * 3)
            assert d.L_.ckks_mult_23(d.h, dm.ptr, dc1.ptr, dc2.ptr, dswk.ptr, l, work.ptr, s1.ptr, s2.ptr, s3.ptr) == 0
            assert np.array_equal(from_dev(dm, wm.shape)[:, :l + 1], wm[:, :l + 1]), ("mult_23", l, mode)
    # a context whose q_num is no multiple of p_num has keys of q_num / p_num digits (Context_23.cuh:29): levels that need more are refused
    odd = Pair(10, p, CFG2_Q[:5], t, 3)
    with pytest.raises(Exception):
        odd.dev.external_product_T(to_dev(np.zeros((2, odd.orc.Ri_blockNum * 3, 1024), dtype=np.uint64)),
                                   to_dev(np.zeros((3, 3, 1024), dtype=np.uint64)), to_dev(np.zeros((2, 2, odd.orc.Ri_blockNum, 3, 1024), dtype=np.uint64)), 4)


def test_rescale():
    pair = ref_pair(14, 12)
    o, d, N = pair.orc, pair.dev, pair.N
    L = o.L
    for l in (L, 1):
        c = limbs_uniform(30 + l, o.q, 2, N)
        want = c.copy()
        o.rescaleAndEqual(want.reshape(-1), l)
        dc = to_dev(c)
        scratch = DeviceBuffer(8 * 2 * (L + 1) * N)
        d.rescaleAndEqual(dc, scratch, l)
        got = from_dev(dc, c.shape)
        assert np.array_equal(got[:, :l + 1], want[:, :l + 1])
        assert np.array_equal(got[:, l + 1:], c[:, l + 1:])
    with pytest.raises(ValueError):
        d.rescaleAndEqual(dc, scratch, 0)                   # level-0 operand (Scheme_23.cuh:192-194 behaviour)


@pytest.mark.parametrize("primes", ["36", "49", "mixed"])
def test_rescale_full_ring(primes):
    """rescaleAndEqual at N = 2^16 with a special prime in front (limb i is modulo prime K + i): there the reduction of the last
    limb and the final subtraction run inside the two passes of the forward transform; same words as the oracle and as the
    device's separate steps (ntt mode 1), the last limb left in coefficient form, higher limbs untouched.  On 36-bit primes (5-byte
    form between the passes), on the reference's 49-bit primes and on a chain that mixes both (whole limbs between the passes)."""
    q, p = CFG2_Q[:7], CFG3_P[:1]
    if primes == "49":
        q, p = REF_PARAMS[16]["q"][:7], REF_PARAMS[16]["p"][:1]
    elif primes == "mixed":
        q = CFG2_Q[:2] + REF_PARAMS[16]["q"][:2] + CFG2_Q[2:4] + REF_PARAMS[16]["q"][2:3]
    pair = Pair(16, p, q)
    o, d, N = pair.orc, pair.dev, pair.N
    for l in (6, 3, 1):
        c = limbs_uniform(60 + l, q, 2, N)
        c[:, :, :4] = 0
        for j, qq in enumerate(q):
            c[:, j, 4] = qq - 1
        want = c.copy()
        o.rescaleAndEqual(want.reshape(-1), l)
        for mode in (0, 1):
            d.set_ntt_mode(mode)
            dc = to_dev(c)
            scratch = DeviceBuffer(8 * 2 * len(q) * N)
            d.rescaleAndEqual(dc, scratch, l)
            got = from_dev(dc, c.shape)
            assert np.array_equal(got[:, :l + 1], want[:, :l + 1]), (l, mode)
            assert np.array_equal(got[:, l + 1:], c[:, l + 1:]), (l, mode)


@pytest.mark.parametrize("arith_mode", [0, 1])
@pytest.mark.parametrize("logN,nq,np_", [(12, 6, 2), (10, 7, 3), (12, 24, 6), (10, 3, 1)])
def test_hybrid_keyswitch_stages(logN, nq, np_, arith_mode):
    """Textbook hybrid switch over [P|Q_l] (BASELINE config 3 shape at reduced N): every stage and the whole chain, with the
    FP64 conversion / ModDown kernels (arith_mode 0: these primes are below 2^41) and with the integer ones (arith_mode 1)."""
    q, p = CFG2_Q[:nq], CFG3_P[:np_]
    pair = Pair(logN, p, q)
    pair.dev.set_arith_mode(arith_mode)
    o, d, N = pair.orc, pair.dev, pair.N
    W = np_ + nq
    dnum = -(-nq // np_)
    evk = limbs_uniform(3, p + q, 2 * dnum, N)                          # [2][dnum][W][N], seed 3
    devk = to_dev(evk)
    for l in (nq - 1, nq - 2, 0):
        dn = -(-(l + 1) // np_)
        inp = np.zeros((nq, N), dtype=np.uint64)
        inp[:l + 1] = limbs_uniform(40 + l, q[:l + 1], 1, N)[0]
        wdig = np.zeros((dn, W, N), dtype=np.uint64)
        o.hybrid_modup(wdig.reshape(-1), inp.reshape(-1), l)
        ddig = to_dev(np.zeros_like(wdig))
        d.hybrid_modup(ddig, to_dev(inp), l)
        assert np.array_equal(from_dev(ddig, wdig.shape)[:, :np_ + l + 1], wdig[:, :np_ + l + 1]), ("modup", l)
        wip = np.zeros((2, W, N), dtype=np.uint64)
        o.hybrid_inner_product(wip.reshape(-1), wdig.reshape(-1), evk.reshape(-1), l)
        dip = to_dev(np.zeros_like(wip))
        d.hybrid_inner_product(dip, to_dev(wdig), devk, l)
        assert np.array_equal(from_dev(dip, wip.shape)[:, :np_ + l + 1], wip[:, :np_ + l + 1]), ("inner", l)
        wout = np.zeros((2, nq, N), dtype=np.uint64)
        o.hybrid_moddown(wout.reshape(-1), wip.reshape(-1), l)
        dout = to_dev(np.zeros_like(wout))
        d.hybrid_moddown(dout, to_dev(wip), l)
        assert np.array_equal(from_dev(dout, wout.shape)[:, :l + 1], wout[:, :l + 1]), ("moddown", l)
        # whole switch
        wks = np.zeros((2, nq, N), dtype=np.uint64)
        o.hybrid_keyswitch(wks.reshape(-1), inp.reshape(-1), evk.reshape(-1), l)
        dks = to_dev(np.zeros_like(wks))
        scratch = DeviceBuffer(8 * (dn + 2) * W * N)
        scratch.zero()
        d.hybrid_keyswitch(dks, to_dev(inp), devk, l, scratch)
        assert np.array_equal(from_dev(dks, wks.shape)[:, :l + 1], wks[:, :l + 1]), ("keyswitch", l)


@pytest.mark.parametrize("nq,np_,l,primes", [(24, 6, 23, "36"), (24, 6, 9, "36"), (5, 2, 4, "36"), (3, 1, 2, "36"), (3, 1, 0, "36"), (7, 3, 3, "36"),
                                             (5, 2, 4, "49"), (3, 1, 2, "49"), (8, 4, 7, "49"), (4, 2, 3, "mixed")])
def test_config3_full_size_keyswitch(nq, np_, l, primes):
    """BASELINE config 3 at full size: N = 2^16, 24 Q + 6 P primes, dnum = 4, seed 3; parity with the oracle on the
    whole switch output (every residue), at the top level and at a level whose last digit is partial (10 limbs in digits of 6);
    then smaller prime sets at the same ring size: a partial last digit at the top level, one special prime (digits of one prime, the
    ModDown's single-prime branch), level 0, and a level that leaves whole digits unused.
    At this ring size the middle of the switch (row passes of both transforms around the inner product) is one launch; the
    same call with the transforms forced to two launches each (ntt mode 1) takes the separate steps and must give the same words.
    On the reference's 49- and 50-bit primes (and on a chain that mixes widths) only the end of the switch is fused: the ModDown
    inside the first pass of the last transform, on the wide FP64 arithmetic."""
    q, p = CFG2_Q[:nq], CFG3_P[:np_]
    if primes == "49":
        q, p = REF_PARAMS[16]["q"][:nq], REF_PARAMS[16]["p"][:np_]
    elif primes == "mixed":
        q, p = CFG2_Q[:2] + REF_PARAMS[16]["q"][:nq - 2], [CFG3_P[0]] + REF_PARAMS[16]["p"][:np_ - 1]
    pair = Pair(16, p, q)
    o, d, N = pair.orc, pair.dev, pair.N
    W = nq + np_
    dn = -(-(l + 1) // np_)
    evk = limbs_uniform(3, p + q, 2 * -(-nq // np_), N)
    inp = np.zeros((nq, N), dtype=np.uint64)
    inp[:l + 1] = limbs_uniform(33, q[:l + 1], 1, N)[0]
    wks = np.zeros((2, nq, N), dtype=np.uint64)
    o.hybrid_keyswitch(wks.reshape(-1), inp.copy().reshape(-1), evk.reshape(-1), l)
    devk = to_dev(evk)
    for mode in (0, 1):
        d.set_ntt_mode(mode)
        dks = to_dev(np.zeros_like(wks))
        scratch = DeviceBuffer(8 * (dn + 2) * W * N)
        d.hybrid_keyswitch(dks, to_dev(inp), devk, l, scratch)
        assert np.array_equal(from_dev(dks, wks.shape)[:, :l + 1], wks[:, :l + 1]), mode


def test_hybrid_keyswitch_and_paired_transform_replayed_from_a_graph():
    """The fused key switch (five launches with waits between workgroups of one launch) and a paired transform captured into a HIP
    graph and replayed: no launch depends on host-side state, so every replay on fresh inputs gives the oracle's words.  Eager work
    and synchronisations lie between the replays."""
    import ctypes
    hip = ctypes.CDLL("libamdhip64.so")
    nq, np_, l = 6, 2, 5
    q, p = CFG2_Q[:nq], CFG3_P[:np_]
    pair = Pair(16, p, q)
    o, d, N = pair.orc, pair.dev, pair.N
    W, dn = nq + np_, -(-(l + 1) // np_)
    evk = limbs_uniform(3, p + q, 2 * -(-nq // np_), N)
    devk = to_dev(evk)
    stream = ctypes.c_void_p()
    assert hip.hipStreamCreate(ctypes.byref(stream)) == 0
    d.set_stream(stream)
    dks, dinp, scratch = to_dev(np.zeros((2, nq, N), dtype=np.uint64)), to_dev(np.zeros((nq, N), dtype=np.uint64)), DeviceBuffer(8 * (dn + 2) * W * N)
    d.hybrid_keyswitch(dks, dinp, devk, l, scratch)              # eager once: the inter-pass area is allocated before the capture
    d.FromNTTInplace(dinp, 0, np_, 1, l + 1, nq)
    d.check()
    graph, gexec = ctypes.c_void_p(), ctypes.c_void_p()
    assert hip.hipStreamBeginCapture(stream, 0) == 0
    d.hybrid_keyswitch(dks, dinp, devk, l, scratch)
    d.FromNTTInplace(dks, 0, np_, 2, l + 1, nq)                   # a paired transform of the result, 12 limbs
    assert hip.hipStreamEndCapture(stream, ctypes.byref(graph)) == 0
    assert hip.hipGraphInstantiate(ctypes.byref(gexec), graph, None, None, ctypes.c_size_t(0)) == 0
    for rep in range(3):
        inp = np.zeros((nq, N), dtype=np.uint64)
        inp[:l + 1] = limbs_uniform(70 + rep, q[:l + 1], 1, N)[0]
        want = np.zeros((2, nq, N), dtype=np.uint64)
        o.hybrid_keyswitch(want.reshape(-1), inp.copy().reshape(-1), evk.reshape(-1), l)
        o.FromNTTInplace(want.reshape(-1), 0, np_, 2, l + 1, nq)
        dinp.upload(inp)
        assert hip.hipGraphLaunch(gexec, stream) == 0
        d.check()
        assert np.array_equal(from_dev(dks, want.shape)[:, :l + 1], want[:, :l + 1]), rep
        d.ToNTTInplace(dks, 0, np_, 2, l + 1, nq)                  # eager work between the replays
        d.check()
    assert hip.hipGraphExecDestroy(gexec) == 0 and hip.hipGraphDestroy(graph) == 0
    d.set_stream(None)
    assert hip.hipStreamDestroy(stream) == 0
