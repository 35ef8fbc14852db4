"""Order of work of the chained transform (host logic, no GPU): every (pass, limb, tile) of a chain appears in exactly one slot,
a limb's second pass comes after its whole first pass, and first passes run at most `skew` limbs ahead."""
import ctypes as C
import itertools

import pytest

from ckks_llm_amd import load_library


def slots(kmax, tiles, skew):
    L = load_library()
    n = L.ckks_ntt_chain_slots(kmax, tiles, skew)
    out = []
    for s in range(n):
        second, k, tile = C.c_uint(), C.c_uint(), C.c_uint()
        assert L.ckks_ntt_chain_slot(s, tiles, skew, C.byref(second), C.byref(k), C.byref(tile)) == 0
        out.append((second.value, k.value, tile.value))
    return out


@pytest.mark.parametrize("kmax,tiles,skew", [(1, 16, 1), (2, 16, 1), (2, 16, 2), (6, 16, 1), (7, 8, 3), (192, 16, 1), (192, 16, 4), (5, 16, 5)])
def test_every_tile_once_and_in_order(kmax, tiles, skew):
    sl = slots(kmax, tiles, skew)
    live = [(p, k, t) for (p, k, t) in sl if k < kmax]
    assert sorted(live) == sorted(itertools.product((0, 1), range(kmax), range(tiles)))      # each exactly once
    pos = {x: i for i, x in enumerate(sl) if x[1] < kmax}
    for k in range(kmax):
        last_first = max(pos[(0, k, t)] for t in range(tiles))
        first_second = min(pos[(1, k, t)] for t in range(tiles))
        assert last_first < first_second
        if k + skew + 1 < kmax:       # the first pass of limb k + skew + 1 does not start before the second pass of limb k is handed out
            assert max(pos[(1, k, t)] for t in range(tiles)) < min(pos[(0, k + skew + 1, t)] for t in range(tiles))
    # tiles of an entry are consecutive slots
    for i in range(0, len(sl), tiles):
        assert len({(p, k) for (p, k, _) in sl[i:i + tiles]}) == 1
        assert [t for (_, _, t) in sl[i:i + tiles]] == list(range(tiles))


def test_bad_arguments():
    L = load_library()
    x = C.c_uint()
    assert L.ckks_ntt_chain_slot(0, 0, 1, C.byref(x), C.byref(x), C.byref(x)) != 0
