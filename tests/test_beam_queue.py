"""BeamSearch.GetTopNBSS (Utils/BeamSearch.cs:36-46 over AdvUtils/FixedSizePriorityQueue.cs): the oracle's Python
restatement and the library's C++ restatement (TSHip_BeamTopN, host code: runs without a GPU) against each other and
against what the queue is for: the survivors are the top_n lowest scores (brute force), the best one comes out first."""
import ctypes as C

import numpy as np
import pytest


def _lib_top_n(scores, top_n):
    from seq2seqsharp_amd._lib import check, lib
    L = lib()
    L.TSHip_BeamTopN.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.POINTER(C.c_int)]
    sc = np.ascontiguousarray(scores, dtype=np.float32)
    kept = np.full((top_n,), -1, np.int32)
    n = C.c_int(0)
    check(L.TSHip_BeamTopN(sc.ctypes.data_as(C.c_void_p), sc.size, top_n, kept.ctypes.data_as(C.c_void_p), C.byref(n)))
    return [int(k) for k in kept[:n.value]]


@pytest.mark.parametrize("top_n", [1, 2, 3, 4, 5, 8, 13])
def test_survivors_are_the_lowest_scores(oracle, top_n):
    rng = np.random.default_rng(top_n)
    for n in (1, 2, top_n, top_n + 1, 3 * top_n, 50):
        for _ in range(20):
            s = rng.permutation(n).astype(np.float32) + rng.random(n).astype(np.float32) * 0.5      # no ties
            kept = oracle.get_top_n(s, top_n)
            assert sorted(kept) == sorted(np.argsort(s)[:min(n, top_n)].tolist())
            assert kept[0] == int(np.argmin(s))             # the better half's root is the best hypothesis
            assert _lib_top_n(s, top_n) == kept


def test_ties_and_order_agree_between_the_two_restatements(oracle):
    rng = np.random.default_rng(0)
    for _ in range(300):
        n, top_n = int(rng.integers(1, 30)), int(rng.integers(1, 9))
        s = rng.integers(0, 6, n).astype(np.float32)        # many equal scores
        a, b = oracle.get_top_n(s, top_n), _lib_top_n(s, top_n)
        assert a == b
        assert sorted(s[a].tolist()) == sorted(np.sort(s)[:min(n, top_n)].tolist())
    # an equal score does not displace a survivor (Better is strict)
    assert oracle.get_top_n([1.0, 1.0, 1.0], 2) == _lib_top_n([1.0, 1.0, 1.0], 2) == [0, 1]


def test_beam_picks_restates_the_pick_loop(oracle):
    """Decoder.cs:756-792 with Argmax: the picks are the n largest probabilities in order (first index among equals), each
    logged before it is zeroed."""
    rng = np.random.default_rng(1)
    p = oracle.softmax(rng.standard_normal((3, 40)).astype(np.float32))
    p[1, 7] = p[1, 3]                                       # a tie: the lower index goes first
    ids, logp = oracle.beam_picks(p, 4)
    for b in range(3):
        order = sorted(range(40), key=lambda j: (-p[b, j], j))[:4]
        assert ids[:, b].tolist() == order
        assert np.allclose(logp[:, b], np.log(p[b, order].astype(np.float64)), rtol=1e-6)
