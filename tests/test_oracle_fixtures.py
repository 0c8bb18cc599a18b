"""Pins the CPU oracle (oracle/ts_oracle.cpp) against the inputs the reference's own tests use
(Tests/Seq2SeqSharp.Tests/GgmlOpsComparison_Tests.cs, ComputeGraph_Tests.cs) with closed-form or
independently computed answers, against library routines, and against invariants chosen so that a dropped
term, a wrong sign or index, or a transposed operand fails one of them."""
import math

import numpy as np
import pytest


# ---- fixtures of GgmlOpsComparison_Tests.cs -----------------------------------------------------------------
def test_softmax_fixture(oracle):
    # GgmlOpsComparison_Tests.cs:419-426: rows [1,2,3,4], [5,6,7,8]; closed form e^(x-4)/(1+e^-1+e^-2+e^-3)
    x = np.array([[1, 2, 3, 4], [5, 6, 7, 8]], np.float32)
    z = sum(math.exp(-k) for k in range(4))
    want = np.array([[math.exp(k - 3) / z for k in range(4)]] * 2)
    got = oracle.softmax(x)
    assert np.allclose(got, want, rtol=2e-7, atol=0)
    assert np.allclose(got.sum(1), 1.0, atol=1e-6)
    # shift invariance (the max is subtracted first)
    assert np.array_equal(got[0], got[1])


def test_softmax_non_contiguous_fixture(oracle):
    # :429-436: the same values through a transposed [4,2] view
    base = np.arange(1, 9, dtype=np.float32).reshape(4, 2)
    got = oracle.softmax(oracle.copy_strided(base.T))
    want = np.exp(base.T.astype(np.float64) - base.T.max(1, keepdims=True))
    want /= want.sum(1, keepdims=True)
    assert np.allclose(got, want, rtol=3e-7)


def test_addmm_fixture_exact(oracle):
    # :439-447: 2x4 (1..8) times 4x3 (1..12), beta 0: integers, exact in fp32
    m1 = np.arange(1, 9, dtype=np.float32).reshape(2, 4)
    m2 = np.arange(1, 13, dtype=np.float32).reshape(4, 3)
    got = oracle.addmm(0.0, np.zeros((2, 3), np.float32), 1.0, m1, m2)
    assert np.array_equal(got, np.array([[70, 80, 90], [158, 184, 210]], np.float32))


def test_addmm_fixture_transposed_operand(oracle):
    # :450-457: m1 given as the transpose of a [4,2] tensor holding 1,5,2,6,3,7,4,8 -> same product
    base = np.array([1, 5, 2, 6, 3, 7, 4, 8], np.float32).reshape(4, 2)
    m2 = np.arange(1, 13, dtype=np.float32).reshape(4, 3)
    got = oracle.addmm(0.0, np.zeros((2, 3), np.float32), 1.0, base.T, m2)
    assert np.array_equal(got, np.array([[70, 80, 90], [158, 184, 210]], np.float32))


def test_addmmbatch_fixture_exact(oracle):
    # :461-470: 2 x (3x2 . 2x4) of 1..12 and 1..16
    m1 = np.arange(1, 13, dtype=np.float32).reshape(2, 3, 2)
    m2 = np.arange(1, 17, dtype=np.float32).reshape(2, 2, 4)
    got = oracle.addmmbatch(0.0, np.zeros((2, 3, 4), np.float32), 1.0, m1, m2)
    assert np.array_equal(got, np.einsum("bik,bkj->bij", m1, m2))
    # :473-481: m1 stored as [2,2,3] and transposed(1,2)
    base = np.arange(1, 13, dtype=np.float32).reshape(2, 2, 3)
    got2 = oracle.addmmbatch(0.0, np.zeros((2, 3, 4), np.float32), 1.0, np.ascontiguousarray(base.transpose(0, 2, 1)), m2)
    assert np.array_equal(got2, np.einsum("bik,bkj->bij", base.transpose(0, 2, 1), m2))


def test_argmax_fixture(oracle):
    # :525-532 -> [2, 1]; :535-542 (transposed [4,2] of 3,2,1,4,5,6,9,8) -> rows [3,1,5,9],[2,4,6,8] -> [3, 3]
    assert list(oracle.argmax(np.array([[3, 1, 4, 1], [5, 9, 2, 6]], np.float32))) == [2.0, 1.0]
    t = np.array([3, 2, 1, 4, 5, 6, 9, 8], np.float32).reshape(4, 2).T
    assert list(oracle.argmax(oracle.copy_strided(t))) == [3.0, 3.0]


def test_argmax_first_maximum_wins(oracle):
    # TensorApplyCPU.cs:345-355 uses a strict '>'
    assert list(oracle.argmax(np.array([[1, 7, 7, 2], [4, 4, 4, 4], [0, -1, 0, 0]], np.float32))) == [1.0, 0.0, 0.0]


def test_layernorm_fixture(oracle):
    # :545-555: rows 1..4 and 5..8, gamma 1, beta 0, eps 1e-5.  mean 2.5 / 6.5, variance 1.25 -> closed form
    x = np.arange(1, 9, dtype=np.float32).reshape(2, 4)
    got = oracle.layernorm(x, np.ones(4, np.float32), np.zeros(4, np.float32), 1e-5)
    want = np.array([-1.5, -0.5, 0.5, 1.5]) / math.sqrt(1.25 + 1e-5)
    assert np.allclose(got[0], want, rtol=3e-7) and np.allclose(got[1], want, rtol=3e-7)


def test_rmsnorm_fixture(oracle):
    # :570-580: rms of [1,2,3,4] = sqrt(30/4 + eps); of [5..8] = sqrt(174/4 + eps)
    x = np.arange(1, 9, dtype=np.float32).reshape(2, 4)
    got = oracle.rmsnorm(x, np.ones(4, np.float32), np.zeros(4, np.float32), 1e-5)
    assert np.allclose(got[0], x[0] / math.sqrt(7.5 + 1e-5), rtol=3e-7)
    assert np.allclose(got[1], x[1] / math.sqrt(43.5 + 1e-5), rtol=3e-7)
    # beta = null path of RMSNormalization (Layers/RMSNormalization.cs:33-37)
    assert np.array_equal(oracle.rmsnorm(x, np.ones(4, np.float32), None, 1e-5), got)


def test_norms_against_float64(oracle):
    rng = np.random.default_rng(0)
    x = rng.standard_normal((5, 67)).astype(np.float32) * 3 + 1
    g = rng.standard_normal(67).astype(np.float32)
    b = rng.standard_normal(67).astype(np.float32)
    x64 = x.astype(np.float64)
    mu = x64.mean(1, keepdims=True)
    ln = g * (x64 - mu) / np.sqrt(((x64 - mu) ** 2).mean(1, keepdims=True) + 1e-6) + b      # eps inside the sqrt
    assert np.allclose(oracle.layernorm(x, g, b, 1e-6), ln, rtol=2e-5, atol=2e-6)
    rn = g * x64 / np.sqrt((x64 ** 2).mean(1, keepdims=True) + 1e-6) + b
    assert np.allclose(oracle.rmsnorm(x, g, b, 1e-6), rn, rtol=2e-5, atol=2e-6)
    # eps really is inside the square root: with a huge eps the output collapses towards beta
    assert np.allclose(oracle.rmsnorm(x, g, b, 1e12), b, atol=1e-4)


def test_activation_fixtures(oracle):
    # GgmlOpsComparison_Tests.cs:271-288 / ComputeGraph_Tests.cs:229-253 style: values against the definitions
    x = np.array([-2, -1, -0.5, 0, 0.5, 1, 2, 3], np.float32)
    assert np.array_equal(oracle.unary("relu", x), np.maximum(x, 0))
    assert np.allclose(oracle.unary("silu", x), x / (1 + np.exp(-x.astype(np.float64))), rtol=2e-7)
    assert np.allclose(oracle.unary("leakyrelu", x), np.where(x < 0, np.float32(0.01) * x, x), rtol=0)


# ---- TopK (ComputeGraph_Tests.cs:256-329) ---------------------------------------------------------------------
def test_topk_multiset_like_reference_test(oracle):
    # the reference compares value and index multisets with a sorted-dictionary brute force
    rng = np.random.default_rng(1)
    x = rng.standard_normal((16, 2560)).astype(np.float32)
    k = 128
    v, i = oracle.topk(x, k)
    for r in range(x.shape[0]):
        order = np.argsort(-x[r], kind="stable")[:k]
        assert sorted(i[r].astype(int)) == sorted(order)
        assert np.array_equal(np.sort(v[r])[::-1], x[r][order])
        assert np.array_equal(v[r], np.sort(v[r])[::-1])          # descending


def test_topk_tie_rule_from_source(oracle):
    # replace_smaller (TensorApplyCPU.cs:1099-1119): an element equal to the k-th replaces it (later index wins at
    # the boundary); an element equal to a higher entry goes after it.
    v, i = oracle.topk(np.array([[5, 3, 5, 3, 3]], np.float32), 3)
    assert list(v[0]) == [5, 5, 3] and list(i[0]) == [0, 2, 4]
    v, i = oracle.topk(np.array([[1, 1, 1, 1]], np.float32), 2)
    assert list(i[0]) == [0, 3]        # first stays on top, the last equal one holds the boundary slot
    # brute-force restatement on random tied data
    rng = np.random.default_rng(2)
    for _ in range(50):
        row = rng.integers(0, 4, size=9).astype(np.float32)
        k = int(rng.integers(1, 6))
        arr, idx = [-1.70141e38] * k, [-1.70141e38] * k
        for c, d in enumerate(row):
            if d < arr[k - 1]:
                continue
            j = k - 2
            while j >= 0:
                if d > arr[j]:
                    arr[j + 1], idx[j + 1] = arr[j], idx[j]
                else:
                    arr[j + 1], idx[j + 1] = d, c
                    break
                j -= 1
            if j < 0:
                arr[0], idx[0] = d, c
        v, i = oracle.topk(row[None], k)
        assert list(v[0]) == arr and list(i[0]) == idx


# ---- RoPE (no reference test: closed form and invariants) ------------------------------------------------------
def test_rope_closed_form_and_invariants(oracle):
    rng = np.random.default_rng(3)
    cols, seq = 16, 5
    x = rng.standard_normal((2 * seq, cols)).astype(np.float32)
    off = 7
    got = oracle.rope(x, seq, off)
    want = np.empty_like(x, dtype=np.float64)
    for r in range(x.shape[0]):
        m = (r % seq) + off
        for i in range(cols // 2):
            th = np.float32(np.float32(500000.0 ** (-2.0 * i / cols)) * np.float32(m))     # float theta * float m
            c, s = math.cos(th), math.sin(th)
            want[r, 2 * i] = x[r, 2 * i] * c - x[r, 2 * i + 1] * s            # adjacent pairs, not half-split
            want[r, 2 * i + 1] = x[r, 2 * i + 1] * c + x[r, 2 * i] * s
    assert np.allclose(got, want, rtol=1e-6, atol=1e-6)
    # position 0 is the identity
    assert np.array_equal(oracle.rope(x[:1], 1, 0), x[:1])
    # rotations preserve the norm of every pair
    pn = lambda a: np.hypot(a[:, 0::2], a[:, 1::2])
    assert np.allclose(pn(got), pn(x), rtol=1e-6)
    # <rope(q,m), rope(k,n)> depends on m - n only
    q, k = x[:1], x[1:2]
    d1 = (oracle.rope(q, 1, 9) * oracle.rope(k, 1, 4)).sum()
    d2 = (oracle.rope(q, 1, 25) * oracle.rope(k, 1, 20)).sum()
    assert abs(d1 - d2) < 2e-4
    # a wrong base or a half-split pairing must not pass the closed form above
    assert not np.allclose(oracle.rope(x, seq, off, base=10000.0), want, rtol=1e-3, atol=1e-3)


# ---- gather / scatter / masks: brute force, bit exact ------------------------------------------------------------
def test_indexselect_and_indexupdate_bruteforce(oracle):
    rng = np.random.default_rng(4)
    src = rng.standard_normal((11, 6)).astype(np.float32)
    idx = np.array([3, 0, -1, 10, 3, 7], np.float32)
    got = oracle.indexselect(src, idx, result=np.full((6, 6), 9.0, np.float32))
    for j, s in enumerate(idx.astype(int)):
        assert np.array_equal(got[j], src[s] if s >= 0 else np.full(6, 9.0, np.float32))     # negative rows are skipped
    acc = oracle.indexselect(src, idx, result=np.ones((6, 6), np.float32), is_add=True)
    assert np.array_equal(acc[0], np.float32(1) + src[3])
    # IndexSelectGrad: out[idx[j]] += adj[j] in row order; rows 0 and 4 both hit row 3 -> (0 + a0) + a4
    adj = rng.standard_normal((6, 6)).astype(np.float32)
    g = oracle.indexselectgrad(np.zeros((11, 6), np.float32), adj, idx)
    assert np.array_equal(g[3], (np.float32(0) + adj[0]) + adj[4])
    assert np.array_equal(g[10], adj[3]) and not g[1].any()


def test_trimask(oracle):
    m = oracle.buildtrimask(4, 4)
    assert np.array_equal(m, np.where(np.tril(np.ones((4, 4))) > 0, 0.0, -30000.0).astype(np.float32))
    sm = oracle.buildselftrimask(np.array([2, 3], np.float32), 3)
    want = np.full((6, 3), -30000.0, np.float32)
    for b, ol in enumerate([2, 3]):
        for s in range(3):
            for c in range(3):
                if c < ol and s < ol and c <= s:
                    want[b * 3 + s, c] = 0.0
    assert np.array_equal(sm, want)


# ---- GEMM ---------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("layout", ["nn", "a_t", "b_t", "bias_broadcast"])
def test_gemm_against_numpy(oracle, layout):
    rng = np.random.default_rng(5)
    M, K, N = 7, 33, 19
    a = rng.standard_normal((M, K)).astype(np.float32)
    b = rng.standard_normal((K, N)).astype(np.float32)
    src = rng.standard_normal((M, N)).astype(np.float32)
    if layout == "a_t":
        a = np.ascontiguousarray(a.T).T
    if layout == "b_t":
        b = np.ascontiguousarray(b.T).T
    if layout == "bias_broadcast":
        src = np.broadcast_to(src[:1], (M, N))           # bias.Expand(n, d) of g.Affine
    got = oracle.addmm(0.5, src, 2.0, a, b)
    want = 0.5 * src.astype(np.float64) + 2.0 * (a.astype(np.float64) @ b.astype(np.float64))
    assert np.allclose(got, want, rtol=2e-5, atol=2e-5)


def test_gemm_k_sequential_order(oracle):
    # SGEMM.cs:482-549: C starts from beta*C (the bias) and adds alpha*x_l*w_l for l = 0..K-1, one rounding per
    # product and per sum.  Reproduce that order with float32 scalars.
    rng = np.random.default_rng(6)
    K = 50
    x = rng.standard_normal((1, K)).astype(np.float32)
    w = rng.standard_normal((K, 3)).astype(np.float32)
    bias = rng.standard_normal((1, 3)).astype(np.float32)
    got = oracle.addmm(1.0, bias, 1.0, x, w)
    want = bias.copy()
    for l in range(K):
        want = (want + (np.float32(1.0) * x[0, l]) * w[l]).astype(np.float32)
    assert np.array_equal(got, want)


# ---- half rounding ---------------------------------------------------------------------------------------------
def test_float2half_matches_ieee_rne(oracle):
    rng = np.random.default_rng(7)
    x = np.concatenate([rng.standard_normal(20000).astype(np.float32) * 0.02,
                        rng.standard_normal(2000).astype(np.float32) * 1e-6,
                        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e6, -1e6, 6.0e-8, 5.9e-8, 2.98e-8, 3.0e-8,
                                  np.inf, -np.inf, 1.0009765625, 1.00048828125, 1.00146484375], np.float32)])
    got = oracle.float2half_bits(x)
    assert np.array_equal(got, x.astype(np.float16).view(np.uint16))
    assert np.array_equal(oracle.half_bits2float(got), x.astype(np.float16).astype(np.float32))


# ---- top-p ----------------------------------------------------------------------------------------------------------
def _topp_python(p, top_p, u, seq=None, penalty=0.0):
    """ComputeGraphTensor.TopPSample (ComputeGraphTensor.cs:2305-2403) restated independently; `seq` = the row's
    decodedSequence (tokens already in it are decayed by pow(dist / len, penalty), :2320-2345)."""
    import math
    last = {}
    if seq is not None:
        for j, tok in enumerate(seq):
            last[int(tok)] = len(seq) - j                 # later occurrences overwrite: the last one counts
    items = []
    for j, w in enumerate(p):
        if not w > 0:
            continue
        w = np.float32(w)
        if j in last:
            ratio = np.float32(np.float32(last[j]) / np.float32(len(seq)))
            rp = np.float32(math.pow(float(ratio), float(np.float32(penalty))))
            w = np.float32(w * rp)
        items.append((float(w), j))
    items.sort(key=lambda t: (-t[0], t[1]))
    acc, cands, accp = np.float32(0), [], []
    for w, j in items:
        acc = np.float32(acc + np.float32(w))
        cands.append(j)
        accp.append(acc)
        if acc >= np.float32(top_p):
            break
    for k, a in enumerate(accp):
        if np.float32(a / acc) >= np.float32(u):
            return cands[k]
    return 0


def test_toppsample_bruteforce(oracle):
    rng = np.random.default_rng(8)
    for trial in range(40):
        K = int(rng.integers(3, 40))
        p = rng.random(K).astype(np.float32)
        if trial % 3 == 0:
            p[rng.integers(0, K, 3)] = p[0]               # exact ties -> ascending index inside a bucket
        if trial % 4 == 0:
            p[rng.integers(0, K)] = 0.0                   # masked entries are dropped
        p = (p / p.sum()).astype(np.float32)
        u = np.float32(rng.random())
        tp = float(rng.choice([0.1, 0.5, 0.9, 1.0]))
        got = oracle.toppsample(p[None], tp, 0.0, None, np.array([u], np.float32))
        assert int(got[0]) == _topp_python(p, tp, u)


def test_toppsample_repeat_penalty_bruteforce(oracle):
    rng = np.random.default_rng(18)
    for trial in range(40):
        K = int(rng.integers(3, 40))
        L = int(rng.integers(1, 30))
        p = rng.random(K).astype(np.float32)
        p = (p / p.sum()).astype(np.float32)
        seq = rng.integers(0, K, L).astype(np.int32)
        u = np.float32(rng.random())
        tp = float(rng.choice([0.1, 0.5, 0.9, 1.0]))
        pen = float(rng.choice([2.0, 1.0, 0.5, 1.5, 3.0]))
        got = oracle.toppsample(p[None], tp, pen, seq[None], np.array([u], np.float32))
        assert int(got[0]) == _topp_python(p, tp, u, seq, pen), trial


def test_toppsample_small_p_is_argmax(oracle):
    # cf. the commented GPT test that decodes with DecodingTopP = 0 (Seq2Seq_Tests.cs:135)
    rng = np.random.default_rng(9)
    p = oracle.softmax(rng.standard_normal((6, 50)).astype(np.float32))
    got = oracle.toppsample(p, 1e-6, 0.0, None, rng.random(6).astype(np.float32))
    assert np.array_equal(got, oracle.argmax(p))


def test_toppsample_repeat_penalty(oracle):
    # tokens already in the sequence are decayed by (distance / length) ^ penalty before sorting
    p = np.array([[0.5, 0.3, 0.2]], np.float32)
    seq = np.array([[0, 2, 0, 1]], np.int32)          # token 0 last seen at distance 2, token 1 at 1, token 2 at 3
    got = oracle.toppsample(p, 0.01, 2.0, seq, np.array([0.0], np.float32))
    w = np.array([0.5 * (2 / 4) ** 2, 0.3 * (1 / 4) ** 2, 0.2 * (3 / 4) ** 2])
    assert int(got[0]) == int(np.argmax(w))
