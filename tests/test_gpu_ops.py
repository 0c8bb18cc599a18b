"""Per-op parity on the GPU, in the pattern of the reference's cross-backend comparator
(Tests/Seq2SeqSharp.Tests/GgmlOpsComparison_Tests.cs:23-70): the same inputs through the CPU oracle and through the
C-ABI op, each op on a contiguous and on a transposed (non-contiguous) input.  Tolerance: the reference's 1e-4
for floating point (tighter where noted), bit-exact for index work."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

TOL = 1e-4      # GgmlOpsComparison_Tests.cs:19


@pytest.fixture(scope="module")
def T():
    from seq2seqsharp_amd import ops, tensor
    return tensor.HipTensor, ops


def _both_layouts(HT, a):
    """The array as a contiguous device tensor and as a transposed view of a transposed copy."""
    yield HT.from_numpy(a)
    yield HT.from_numpy(np.ascontiguousarray(a.T)).transpose(0, 1)


def test_copy_fill_and_views(T, oracle):
    HT, ops = T
    a = np.arange(24, dtype=np.float32).reshape(2, 3, 4)
    t = HT.from_numpy(a)
    assert np.array_equal(t.numpy(), a)
    assert np.array_equal(t.transpose(1, 2).numpy(), a.transpose(0, 2, 1))            # strided copy
    assert np.array_equal(t.narrow(2, 1, 2).numpy(), a[:, :, 1:3])
    assert np.array_equal(t.select(1, 2).numpy(), a[:, 2])
    e = HT.from_numpy(a[:, :1]).expand(2, 3, 4)                                       # stride-0 broadcast
    assert np.array_equal(e.numpy(), np.broadcast_to(a[:, :1], (2, 3, 4)))
    v5 = HT.from_numpy(np.arange(48, dtype=np.float32)).view(2, 2, 1, 3, 4).expand(2, 2, 3, 3, 4).transpose(3, 4)
    assert np.array_equal(v5.numpy(), oracle.copy_strided(
        np.broadcast_to(np.arange(48, dtype=np.float32).reshape(2, 2, 1, 3, 4), (2, 2, 3, 3, 4)).transpose(0, 1, 2, 4, 3)))
    f = ops.fill(HT([3, 5]), 2.5)
    assert np.array_equal(f.numpy(), np.full((3, 5), 2.5, np.float32))
    with pytest.raises(Exception):
        t.transpose(0, 1).view(24)                                                     # View needs a contiguous tensor


def test_float2half_roundtrip_is_rne(T, oracle):
    HT, ops = T
    x = (np.random.default_rng(0).standard_normal(4096) * 0.02).astype(np.float32)
    h = ops.float2half(None, HT.from_numpy(x))
    back = ops.half2float(None, h).numpy()
    assert np.array_equal(back, oracle.half_bits2float(oracle.float2half_bits(x)))


@pytest.mark.parametrize("op", ["add", "sub", "mul", "div"])
def test_binary_ops(T, op):
    HT, ops = T
    rng = np.random.default_rng(1)
    a = rng.standard_normal((6, 9)).astype(np.float32)
    b = (rng.standard_normal((6, 9)) + 3).astype(np.float32)
    f = {"add": np.add, "sub": np.subtract, "mul": np.multiply, "div": np.divide}[op]
    for ta in _both_layouts(HT, a):
        got = getattr(ops, op)(None, ta, HT.from_numpy(b)).numpy()
        assert np.array_equal(got, f(a, b))
        assert np.array_equal(getattr(ops, op)(None, ta, 3.0).numpy(), f(a, np.float32(3.0)))
    row = HT.from_numpy(b[:1]).expand(6, 9)
    assert np.array_equal(ops.add(None, HT.from_numpy(a), row).numpy(), a + b[:1])


@pytest.mark.parametrize("name", ["relu", "silu", "leakyrelu", "exp", "log", "sigmoid", "neg", "tanh", "sqrt", "abs"])
def test_unary_ops(T, oracle, name):
    HT, ops = T
    x = np.random.default_rng(2).standard_normal((5, 7)).astype(np.float32)
    if name in ("log", "sqrt"):
        x = np.abs(x) + 0.1
    ref = {"exp": np.exp, "log": np.log, "sigmoid": lambda v: 1 / (1 + np.exp(-v)), "neg": np.negative, "tanh": np.tanh, "sqrt": np.sqrt,
           "abs": np.abs}.get(name)
    want = oracle.unary(name, x) if ref is None else ref(x.astype(np.float64))
    for t in _both_layouts(HT, x):
        assert np.allclose(getattr(ops, name)(None, t).numpy(), want, rtol=2e-6, atol=1e-7)


def test_softmax(T, oracle):
    HT, ops = T
    fix = np.array([[1, 2, 3, 4], [5, 6, 7, 8]], np.float32)        # GgmlOpsComparison_Tests.cs:419-426
    big = np.random.default_rng(3).standard_normal((7, 3001)).astype(np.float32) * 4
    for a in (fix, big):
        for t in _both_layouts(HT, a):
            got = ops.softmax(None, t).numpy()
            assert np.allclose(got, oracle.softmax(a), rtol=1e-5, atol=1e-8)
            assert np.allclose(got.sum(1), 1, atol=1e-5)


def test_addmm(T, oracle):
    HT, ops = T
    m1 = np.arange(1, 9, dtype=np.float32).reshape(2, 4)
    m2 = np.arange(1, 13, dtype=np.float32).reshape(4, 3)
    for a in _both_layouts(HT, m1):                                   # GgmlOpsComparison_Tests.cs:439-457
        r = ops.addmm(None, 0.0, HT.from_numpy(np.zeros((2, 3), np.float32)), 1.0, a, HT.from_numpy(m2))
        assert np.array_equal(r.numpy(), np.array([[70, 80, 90], [158, 184, 210]], np.float32))
    rng = np.random.default_rng(4)
    M, K, N = 37, 129, 70
    x, w, b = (rng.standard_normal(s).astype(np.float32) for s in ((M, K), (K, N), (1, N)))
    want = oracle.addmm(1.0, np.broadcast_to(b, (M, N)), 1.0, x, w)
    for tw in _both_layouts(HT, w):
        bias = HT.from_numpy(b).expand(M, N)                          # g.Affine: Addmm(res, 1, bias.Expand, 1, x, W)
        got = ops.addmm(None, 1.0, bias, 1.0, HT.from_numpy(x), tw).numpy()
        assert np.allclose(got, want, rtol=TOL, atol=TOL)
        assert np.abs(got - want).max() < 2e-5
    with pytest.raises(Exception, match="Size mismatch"):
        ops.addmm(None, 0.0, HT([2, 3]), 1.0, HT([2, 4]), HT([5, 3]))


@pytest.mark.parametrize("M,K,N", [(1, 16, 4), (33, 24, 68), (130, 512, 256), (64, 2048, 96), (200, 40, 8)])
def test_addmm_fp16_on_the_matrix_cores(T, M, K, N):
    """Float16 operands with contiguous rows take the MFMA kernel (K a multiple of 8, N of 4): partial row, column and k
    tiles, alpha / beta, an expanded bias, result aliasing src, and the batched form.  Against float64 products of the same
    Float16 values; the result is rounded to Float16 once."""
    HT, ops = T
    from seq2seqsharp_amd.tensor import F16
    rng = np.random.default_rng(M + K + N)
    a = rng.standard_normal((M, K)).astype(np.float16)
    b = rng.standard_normal((K, N)).astype(np.float16)
    bias = rng.standard_normal((1, N)).astype(np.float16)
    want = a.astype(np.float64) @ b.astype(np.float64)
    tol = 2e-3 * np.sqrt(K) + 1e-2
    ta, tb = HT.from_numpy(a.astype(np.float32), F16), HT.from_numpy(b.astype(np.float32), F16)
    got = ops.addmm(None, 1.0, HT.from_numpy(bias.astype(np.float32), F16).expand(M, N), 1.0, ta, tb)
    assert got.dtype == F16
    assert np.abs(got.numpy() - (want + bias.astype(np.float64))).max() <= tol
    r = HT.from_numpy(np.ones((M, N), np.float32), F16)
    got = ops.addmm(r, 0.5, r, -2.0, ta, tb).numpy()                      # result aliases src
    assert np.abs(got - (0.5 - 2.0 * want)).max() <= 2 * tol
    # same product through the generic kernel (a transposed view of a transposed copy is not row-contiguous)
    tbt = HT.from_numpy(np.ascontiguousarray(b.T).astype(np.float32), F16).transpose(0, 1)
    gen = ops.addmm(None, 0.0, HT([M, N], F16), 1.0, ta, tbt).numpy()
    mf = ops.addmm(None, 0.0, HT([M, N], F16), 1.0, ta, tb).numpy()
    assert np.abs(gen - mf).max() <= tol
    # batched: attention weights x values (MulBatch(attn, Vs))
    q = rng.standard_normal((5, M, K)).astype(np.float16)
    v = rng.standard_normal((5, K, N)).astype(np.float16)
    z = HT([5, M, N], F16)
    got = ops.addmmbatch(z, 0.0, z, 1.0, HT.from_numpy(q.astype(np.float32), F16), HT.from_numpy(v.astype(np.float32), F16)).numpy()
    assert np.abs(got - np.einsum("bik,bkj->bij", q.astype(np.float64), v.astype(np.float64))).max() <= tol


def test_addmmbatch(T, oracle):
    HT, ops = T
    m1 = np.arange(1, 13, dtype=np.float32).reshape(2, 3, 2)
    m2 = np.arange(1, 17, dtype=np.float32).reshape(2, 2, 4)          # GgmlOpsComparison_Tests.cs:461-481
    src = HT.from_numpy(np.zeros((2, 3, 4), np.float32))
    assert np.array_equal(ops.addmmbatch(None, 0.0, src, 1.0, HT.from_numpy(m1), HT.from_numpy(m2)).numpy(), np.einsum("bik,bkj->bij", m1, m2))
    base = HT.from_numpy(np.ascontiguousarray(m1.transpose(0, 2, 1))).transpose(1, 2)
    assert np.array_equal(ops.addmmbatch(None, 0.0, src, 1.0, base, HT.from_numpy(m2)).numpy(), np.einsum("bik,bkj->bij", m1, m2))
    rng = np.random.default_rng(5)
    q, k = rng.standard_normal((6, 5, 16)).astype(np.float32), rng.standard_normal((6, 16, 33)).astype(np.float32)
    r = HT([6, 5, 33])
    got = ops.addmmbatch(r, 0.0, r, 0.25, HT.from_numpy(q), HT.from_numpy(k)).numpy()      # g.MulBatch with scale
    assert np.allclose(got, oracle.addmmbatch(0.0, np.zeros((6, 5, 33), np.float32), 0.25, q, k), rtol=TOL, atol=1e-5)


def test_norms(T, oracle):
    HT, ops = T
    fix = np.arange(1, 9, dtype=np.float32).reshape(2, 4)              # GgmlOpsComparison_Tests.cs:545-590
    one, zero = np.ones(4, np.float32), np.zeros(4, np.float32)
    for t in _both_layouts(HT, fix):
        assert np.allclose(ops.layernorm(None, t, HT.from_numpy(one), HT.from_numpy(zero), 1e-5).numpy(), oracle.layernorm(fix, one, zero, 1e-5), atol=1e-6)
        assert np.allclose(ops.rmsnorm(None, t, HT.from_numpy(one), HT.from_numpy(zero), 1e-5).numpy(), oracle.rmsnorm(fix, one, zero, 1e-5), atol=1e-6)
    rng = np.random.default_rng(6)
    x = rng.standard_normal((9, 2048)).astype(np.float32) * 2 + 0.5
    g, b = rng.standard_normal(2048).astype(np.float32), rng.standard_normal(2048).astype(np.float32)
    tg, tb = HT.from_numpy(g.reshape(1, -1)), HT.from_numpy(b.reshape(1, -1))
    assert np.allclose(ops.layernorm(None, HT.from_numpy(x), tg, tb, 1e-6).numpy(), oracle.layernorm(x, g, b, 1e-6), rtol=TOL, atol=2e-5)
    assert np.allclose(ops.rmsnorm(None, HT.from_numpy(x), tg, None, 1e-6).numpy(), oracle.rmsnorm(x, g, None, 1e-6), rtol=TOL, atol=2e-5)


def test_rope(T, oracle):
    HT, ops = T
    x = np.random.default_rng(7).standard_normal((3 * 4 * 5, 64)).astype(np.float32)
    for off in (0, 17, 1024):
        got = ops.rope(None, HT.from_numpy(x), 5, off).numpy()
        want = oracle.rope(x, 5, off)
        assert np.abs(got - want).max() <= 2e-6
    x3 = x.reshape(12, 5, 64)                                          # [B*H, Tq, d] as the layers pass it
    assert np.abs(ops.rope(None, HT.from_numpy(x3), 5, 3).numpy() - oracle.rope(x3, 5, 3)).max() <= 2e-6


def test_indexselect_bit_exact(T, oracle):
    HT, ops = T
    rng = np.random.default_rng(8)
    src = rng.standard_normal((50, 33)).astype(np.float32)
    idx = np.array([3, 0, -1, 49, 3, 7, 12], np.float32).reshape(-1, 1)
    init = rng.standard_normal((7, 33)).astype(np.float32)
    got = ops.indexselect(HT.from_numpy(init), HT.from_numpy(src), HT.from_numpy(idx)).numpy()
    assert np.array_equal(got, oracle.indexselect(src, idx, result=init))
    got = ops.indexselect(HT.from_numpy(init), HT.from_numpy(src), HT.from_numpy(idx), True).numpy()
    assert np.array_equal(got, oracle.indexselect(src, idx, result=init, is_add=True))
    with pytest.raises(Exception, match="out of range"):
        ops.indexselect(None, HT.from_numpy(src), HT.from_numpy(np.array([[50.0]], np.float32)))
    adj = rng.standard_normal((7, 33)).astype(np.float32)
    g = ops.indexselectgrad(ops.fill(HT([50, 33]), 0.0), HT.from_numpy(adj), HT.from_numpy(idx)).numpy()
    assert np.array_equal(g, oracle.indexselectgrad(np.zeros((50, 33), np.float32), adj, idx))     # duplicates add in row order


def test_argmax_and_topk_bit_exact(T, oracle):
    HT, ops = T
    fix = np.array([[3, 1, 4, 1], [5, 9, 2, 6]], np.float32)          # GgmlOpsComparison_Tests.cs:525-532
    assert list(ops.argmax(None, HT.from_numpy(fix), 1).numpy().reshape(-1)) == [2.0, 1.0]
    tv = HT.from_numpy(np.array([3, 2, 1, 4, 5, 6, 9, 8], np.float32).reshape(4, 2)).transpose(0, 1)
    assert list(ops.argmax(None, tv, 1).numpy().reshape(-1)) == [3.0, 3.0]
    rng = np.random.default_rng(9)
    x = rng.integers(0, 50, size=(17, 32000)).astype(np.float32)       # many exact ties: lowest index must win
    assert np.array_equal(ops.argmax(None, HT.from_numpy(x), 1).numpy().reshape(-1), oracle.argmax(x))
    assert np.array_equal(ops.argmax(None, HT.from_numpy(x), 0).numpy().reshape(-1), oracle.argmax(np.ascontiguousarray(x.T)))
    p = oracle.softmax(rng.standard_normal((64, 8)).astype(np.float32))
    p[5] = 0.125                                                        # all tied
    p[6, :4] = p[6, 4:]                                                 # pairwise ties
    for k in (1, 2, 3):
        ov, oi = ops.topk(None, None, HT.from_numpy(p), k)
        wv, wi = oracle.topk(p, k)
        assert np.array_equal(oi.numpy(), wi) and np.array_equal(ov.numpy(), wv)


def test_masks_and_iscorrupted(T, oracle):
    HT, ops = T
    assert np.array_equal(ops.buildtrimask(HT([6, 6]), 0.0, -30000.0).numpy(), oracle.buildtrimask(6, 6))
    lens = np.array([2, 5, 3], np.float32)
    got = ops.buildselftrimask(HT([15, 5]), HT.from_numpy(lens), 5, 0.0, -30000.0).numpy()
    assert np.array_equal(got, oracle.buildselftrimask(lens, 5))
    x = np.zeros((4, 9), np.float32)
    assert ops.iscorrupted(HT.from_numpy(x)) is False
    x[2, 3] = np.nan
    assert ops.iscorrupted(HT.from_numpy(x)) is True
    x[2, 3] = np.inf
    assert ops.iscorrupted(HT.from_numpy(x)) is True


def test_toppsample_bit_exact_given_probs(T, oracle):
    HT, ops = T
    rng = np.random.default_rng(10)
    p = oracle.softmax(rng.standard_normal((16, 32000)).astype(np.float32))
    p[3, 100:110] = p[3, 50]                                            # exact ties
    p[4, ::7] = 0.0                                                     # masked entries
    u = rng.random(16).astype(np.float32)
    for top_p in (0.1, 0.9, 1.0):
        got = ops.toppsample(None, HT.from_numpy(p), HT.from_numpy(u), top_p).numpy().reshape(-1)
        assert np.array_equal(got, oracle.toppsample(p, top_p, 0.0, None, u))
    small = oracle.softmax(rng.standard_normal((5, 97)).astype(np.float32))
    got = ops.toppsample(None, HT.from_numpy(small), HT.from_numpy(u[:5]), 1e-6).numpy().reshape(-1)
    assert np.array_equal(got, oracle.argmax(small))                    # topP -> 0 is greedy


def test_toppsample_running_sum_is_the_sequential_one(T, oracle):
    """The device evaluates the running sum with block-wide scans in integer arithmetic; the values must be those of
    the reference's one-by-one fp32 additions.  Inputs that stress it: flat rows walked to the end over many binades,
    exact powers of two and equal values (ties of the rounding), sums that never reach top_p, tiny and subnormal
    weights, one candidate, none."""
    HT, ops = T
    rng = np.random.default_rng(12)
    rows = []
    K = 32000
    rows.append(np.full(K, 1.0 / K))                                    # flat
    rows.append(rng.random(K) / K * 2)                                   # flat-ish, sum about 1
    rows.append(2.0 ** rng.integers(-24, -10, K).astype(np.float64))     # powers of two only
    rows.append(rng.integers(1, 4, K) * 2.0 ** -17)                      # few distinct values, many ties
    rows.append(np.where(rng.random(K) < 0.5, 2.0 ** -16, 3 * 2.0 ** -17))
    rows.append(rng.random(K) * 1e-9)                                    # never reaches top_p
    rows.append(np.concatenate([[0.5, 0.25, 0.125], np.full(K - 3, 2.0 ** -30)]))
    rows.append(np.concatenate([rng.random(50) * 1e-41, np.zeros(K - 50)]))          # subnormal weights only
    rows.append(np.concatenate([[0.7], np.zeros(K - 1)]))                # one candidate
    rows.append(np.zeros(K))                                             # none
    rows.append(np.exp(rng.standard_normal(K) * 4) / 1e4)                # wide dynamic range
    rows.append(np.concatenate([rng.random(2047) * 1e-3, [2.0 ** -9], rng.random(K - 2048) * 1e-4]))
    p = np.stack(rows).astype(np.float32)
    for seed in range(8):
        u = np.random.default_rng(100 + seed).random(len(rows)).astype(np.float32)
        for top_p in (0.5, 0.9, 1.0, 1e30):
            got = ops.toppsample(None, HT.from_numpy(p), HT.from_numpy(u), top_p).numpy().reshape(-1)
            want = oracle.toppsample(p, top_p, 0.0, None, u)
            assert np.array_equal(got, want), (seed, top_p, np.nonzero(got != want)[0])
    # small vocabularies: fewer elements than one tile, and an odd size
    for K in (1, 2, 97, 2049, 4100):
        q = oracle.softmax(rng.standard_normal((6, K)).astype(np.float32))
        u = rng.random(6).astype(np.float32)
        for top_p in (0.3, 1.0):
            got = ops.toppsample(None, HT.from_numpy(q), HT.from_numpy(u), top_p).numpy().reshape(-1)
            assert np.array_equal(got, oracle.toppsample(q, top_p, 0.0, None, u)), (K, top_p)


def test_toppsample_repeat_penalty(T, oracle):
    """decodedSequences given (ComputeGraphTensor.cs:2320-2345): tokens already in the row's sequence are decayed by
    pow(dist / len, penalty) before the sort.  Penalty 2 (the reference's default) squares exactly in double; 1.5 and
    0.5 go through pow proper."""
    HT, ops = T
    rng = np.random.default_rng(11)
    rows, K, L = 8, 5000, 40
    p = oracle.softmax((3.0 * rng.standard_normal((rows, K))).astype(np.float32))
    seqs = rng.integers(0, K, size=(rows, L)).astype(np.int32)
    top = np.argsort(-p, axis=1)[:, :12]
    seqs[:, 5:17] = top                                                 # the likeliest tokens have been generated before
    seqs[:, 30:34] = top[:, :4]                                         # some of them twice: the last occurrence counts
    p[2, top[2, 0]] = p[2, top[2, 1]]                                   # a tie that the decay breaks or keeps
    u = rng.random(rows).astype(np.float32)
    for penalty in (2.0, 1.5, 0.5):
        for top_p in (0.3, 0.9, 1.0):
            got = ops.toppsample(None, HT.from_numpy(p), HT.from_numpy(u), top_p, penalty, seqs).numpy().reshape(-1)
            assert np.array_equal(got, oracle.toppsample(p, top_p, penalty, seqs, u)), (penalty, top_p)
    # the decay changes the outcome on this input (otherwise the test would pass without it)
    assert not np.array_equal(oracle.toppsample(p, 0.9, 2.0, seqs, u), oracle.toppsample(p, 0.9, 0.0, None, u))
    # rows of different lengths: every row against the oracle on its own sequence; an empty sequence decays nothing
    lens = np.array([40, 1, 0, 17, 33, 40, 2, 9], np.int32)
    got = ops.toppsample(None, HT.from_numpy(p), HT.from_numpy(u), 0.9, 2.0, seqs, lens).numpy().reshape(-1)
    for i in range(rows):
        want = oracle.toppsample(p[i:i + 1], 0.9, 2.0, seqs[i:i + 1, :lens[i]] if lens[i] else None, u[i:i + 1])
        assert got[i] == want[0], i
    # penalty 0 with sequences = no decay (pow(x, 0) = 1)
    got = ops.toppsample(None, HT.from_numpy(p), HT.from_numpy(u), 0.9, 0.0, seqs).numpy().reshape(-1)
    assert np.array_equal(got, oracle.toppsample(p, 0.9, 0.0, None, u))


def test_error_paths(T):
    HT, ops = T
    from seq2seqsharp_amd._lib import TSHipError
    with pytest.raises(TSHipError):
        ops.softmax(HT([2, 3]), HT([2, 4]))                            # wrong result size
    with pytest.raises(TSHipError):
        ops.add(None, HT([2, 3]), HT([3, 2]))
    with pytest.raises(TSHipError):
        ops.topk(None, None, HT([2, 3]), 4)


def test_gather_and_scatter_fill(T):
    """The two indexing ops of the beam search loop (Decoder.cs:766 Gather(probs, idx, 1), :788 ScatterFill(probs, 0, idx, 1)),
    on contiguous and strided tensors, against NumPy's take_along_axis / put_along_axis; an index outside the dimension fails."""
    HT, ops = T
    rng = np.random.default_rng(30)
    p = rng.random((5, 97)).astype(np.float32)
    idx = rng.integers(0, 97, size=(5, 1)).astype(np.float32)
    got = ops.gather(None, HT.from_numpy(p), 1, HT.from_numpy(idx)).numpy()
    assert np.array_equal(got, np.take_along_axis(p, idx.astype(np.int64), 1))
    t = HT.from_numpy(p)
    ops.scatter_fill(t, 0.0, 1, HT.from_numpy(idx))
    want = p.copy()
    np.put_along_axis(want, idx.astype(np.int64), 0.0, 1)
    assert np.array_equal(t.numpy(), want)
    a = rng.random((4, 6, 7)).astype(np.float32)
    for dim in range(3):
        shape = list(a.shape)
        shape[dim] = 3
        ix = rng.integers(0, a.shape[dim], size=shape).astype(np.float32)
        for src in (HT.from_numpy(a), HT.from_numpy(np.ascontiguousarray(a.transpose(0, 2, 1))).transpose(1, 2)):
            assert np.array_equal(ops.gather(None, src, dim, HT.from_numpy(ix)).numpy(), np.take_along_axis(a, ix.astype(np.int64), dim))
    with pytest.raises(Exception, match="outside"):
        ops.gather(None, HT.from_numpy(p), 1, HT.from_numpy(np.full((5, 1), 97, np.float32)))


def test_toppsample_wide_rows(T, oracle):
    """Rows of 200 000 and 262 144 probabilities (vocabularies beyond 16 bits): nearly flat, so that the running sum walks
    most of the row and the pick lands far beyond index 65 535 of the sorted order; bit-exact against the oracle."""
    HT, ops = T
    rng = np.random.default_rng(11)
    for K in (200000, 262144):
        p = rng.random((3, K)).astype(np.float32) + 0.5
        p[1, :1000] = 0.0                                        # some non-candidates
        p /= p.sum(1, keepdims=True)
        u = np.array([0.999, 0.5, 0.93], np.float32)
        want = oracle.toppsample(p, 0.97, 0.0, None, u)
        got = ops.toppsample(None, HT.from_numpy(p), HT.from_numpy(u.reshape(-1, 1)), 0.97).numpy().reshape(-1)
        assert np.array_equal(got, want), K
    with pytest.raises(Exception):
        ops.toppsample(None, HT.from_numpy(np.ones((1, 262145), np.float32)), HT.from_numpy(np.array([[0.5]], np.float32)), 0.9)
