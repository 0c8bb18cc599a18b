"""ctypes binding of the CPU oracle (oracle/ts_oracle.cpp).

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke check and by the benchmark's
cpu_baseline leg as the checker / reported baseline.  The product package never imports it.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libts_oracle.so")

f32p = np.ctypeslib.ndpointer(dtype=np.float32, flags="C_CONTIGUOUS")
i32p = np.ctypeslib.ndpointer(dtype=np.int32, flags="C_CONTIGUOUS")
u16p = np.ctypeslib.ndpointer(dtype=np.uint16, flags="C_CONTIGUOUS")
i64p = np.ctypeslib.ndpointer(dtype=np.int64, flags="C_CONTIGUOUS")


def build(force=False):
    """Compile the oracle with g++ (a checker build, not a product build)."""
    src = os.path.join(_HERE, "ts_oracle.cpp")
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libts_oracle.so"], stdout=subprocess.DEVNULL)
    return _SO


class OrcConfig(C.Structure):
    _fields_ = [
        ("n_layers", C.c_int), ("hidden", C.c_int), ("n_heads", C.c_int), ("n_kv_heads", C.c_int),
        ("ffn_dim", C.c_int), ("vocab", C.c_int), ("attn_type", C.c_int), ("norm_type", C.c_int),
        ("act", C.c_int), ("n_experts", C.c_int), ("experts_per_token", C.c_int),
        ("norm_eps", C.c_float), ("rope_base", C.c_float), ("use_rope", C.c_int),
        ("max_segments", C.c_int), ("sep_token_id", C.c_int),
    ]


_lib = None


def lib():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_SO):
        build()
    L = C.CDLL(_SO)
    L.orc_last_error.restype = C.c_char_p
    L.orc_set_threads.argtypes = [C.c_int]
    L.orc_get_threads.restype = C.c_int
    L.orc_addmm.argtypes = [f32p, C.c_float, f32p, C.c_long, C.c_long, C.c_float, f32p, C.c_long, C.c_long,
                            f32p, C.c_long, C.c_long, C.c_long, C.c_long, C.c_long]
    L.orc_addmmbatch.argtypes = [f32p, C.c_float, f32p, C.c_float, f32p, f32p, C.c_long, C.c_long, C.c_long, C.c_long, C.c_int]
    L.orc_softmax.argtypes = [f32p, f32p, C.c_long, C.c_long]
    L.orc_layernorm.argtypes = [f32p, f32p, f32p, C.c_void_p, C.c_float, C.c_long, C.c_long]
    L.orc_rmsnorm.argtypes = [f32p, f32p, f32p, C.c_void_p, C.c_float, C.c_long, C.c_long]
    L.orc_rope.argtypes = [f32p, f32p, C.c_long, C.c_long, C.c_int, C.c_int, C.c_double]
    L.orc_indexselect.argtypes = [f32p, f32p, f32p, C.c_long, C.c_long, C.c_int]
    L.orc_indexselectgrad.argtypes = [f32p, f32p, f32p, C.c_long, C.c_long]
    L.orc_topk.argtypes = [f32p, f32p, f32p, C.c_int, C.c_long, C.c_long]
    L.orc_argmax.argtypes = [f32p, f32p, C.c_long, C.c_long]
    L.orc_buildtrimask.argtypes = [f32p, C.c_long, C.c_long, C.c_float, C.c_float]
    L.orc_buildselftrimask.argtypes = [f32p, f32p, C.c_long, C.c_long, C.c_int, C.c_float, C.c_float]
    L.orc_unary.argtypes = [C.c_int, f32p, f32p, C.c_long]
    L.orc_iscorrupted.argtypes = [f32p, C.c_long]
    L.orc_float2half.argtypes = [u16p, f32p, C.c_long]
    L.orc_half2float.argtypes = [f32p, u16p, C.c_long]
    L.orc_toppsample.argtypes = [f32p, f32p, C.c_long, C.c_long, C.c_float, C.c_float, C.c_void_p, C.c_long, f32p]
    L.orc_copy_strided.argtypes = [f32p, f32p, C.c_long, C.c_int, i64p, i64p]
    L.orc_gpt_create.restype = C.c_void_p
    L.orc_gpt_create.argtypes = [C.POINTER(OrcConfig)]
    L.orc_gpt_destroy.argtypes = [C.c_void_p]
    L.orc_gpt_set_weight.argtypes = [C.c_void_p, C.c_char_p, f32p, C.c_int, i64p]
    L.orc_gpt_reset_cache.argtypes = [C.c_void_p]
    L.orc_gpt_cache_len.argtypes = [C.c_void_p]
    L.orc_gpt_cache_len.restype = C.c_long
    L.orc_gpt_step.argtypes = [C.c_void_p, i32p, C.c_long, C.c_long, C.c_int, C.c_float, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p]
    L.orc_gpt_step_padded.argtypes = [C.c_void_p, i32p, C.c_long, C.c_long, f32p, C.c_int, C.c_float, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p]
    L.orc_gpt_get_cache.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_long]
    L.orc_gpt_get_cache.restype = C.c_long
    L.orc_gpt_set_cache.argtypes = [C.c_void_p, C.c_int, C.c_int, f32p, C.c_long, C.c_long, C.c_long]
    L.orc_gpt_moe_trace.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_long]
    L.orc_gpt_moe_trace.restype = C.c_long
    L.orc_moe_layer.argtypes = [C.c_void_p, C.c_int, f32p, C.c_long, f32p, C.c_void_p, C.c_void_p, C.c_void_p]
    L.orc_attn_layer.argtypes = [C.c_void_p, C.c_int, f32p, C.c_long, C.c_long, C.c_int, C.c_int, f32p]
    L.orc_ffn_layer.argtypes = [C.c_void_p, C.c_int, f32p, C.c_long, f32p]
    _lib = L
    return L


def _chk(rc):
    if rc != 1:
        raise RuntimeError("oracle: " + lib().orc_last_error().decode())


def set_threads(n):
    lib().orc_set_threads(int(n))


def _f(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _vp(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


# ---- ops (numpy in, numpy out) ---------------------------------------------------------------
def addmm(beta, src, alpha, m1, m2):
    """src/m1/m2 may be numpy views with arbitrary 2-D strides (in the sense of the reference's Tensor views)."""
    M, K = m1.shape
    N = m2.shape[1]
    out = np.zeros((M, N), np.float32)

    def spans(a):
        a = np.asarray(a, dtype=np.float32)
        s0, s1 = (a.strides[0] // 4, a.strides[1] // 4)
        if s0 < 0 or s1 < 0:
            a = np.ascontiguousarray(a)
            s0, s1 = a.shape[1], 1
        span = (a.shape[0] - 1) * s0 + (a.shape[1] - 1) * s1 + 1
        base = np.lib.stride_tricks.as_strided(a, shape=(span,), strides=(4,))
        return np.ascontiguousarray(base), s0, s1

    sb, ss0, ss1 = spans(np.broadcast_to(src, (M, N)) if src.shape != (M, N) else src)
    ab, as0, as1 = spans(m1)
    bb, bs0, bs1 = spans(m2)
    _chk(lib().orc_addmm(out, beta, sb, ss0, ss1, alpha, ab, as0, as1, bb, bs0, bs1, M, K, N))
    return out


def addmmbatch(beta, src, alpha, m1, m2, m2_transposed=False):
    nb, M, K = m1.shape
    N = m2.shape[1] if m2_transposed else m2.shape[2]
    out = np.zeros((nb, M, N), np.float32)
    _chk(lib().orc_addmmbatch(out, beta, _f(src), alpha, _f(m1), _f(m2), nb, M, K, N, int(m2_transposed)))
    return out


def softmax(x):
    x = _f(x)
    out = np.empty_like(x)
    lib().orc_softmax(out, x, x.size // x.shape[-1], x.shape[-1])
    return out


def layernorm(x, gamma, beta, eps):
    x = _f(x)
    out = np.empty_like(x)
    b = None if beta is None else _f(beta)
    lib().orc_layernorm(out, x, _f(gamma), _vp(b), eps, x.size // x.shape[-1], x.shape[-1])
    return out


def rmsnorm(x, gamma, beta, eps):
    x = _f(x)
    out = np.empty_like(x)
    b = None if beta is None else _f(beta)
    lib().orc_rmsnorm(out, x, _f(gamma), _vp(b), eps, x.size // x.shape[-1], x.shape[-1])
    return out


def rope(x, seq_len, row_offset, base=500000.0):
    x = _f(x)
    out = np.empty_like(x)
    lib().orc_rope(out, x, x.size // x.shape[-1], x.shape[-1], seq_len, row_offset, base)
    return out


def indexselect(src, idx, result=None, is_add=False):
    src = _f(src)
    idx = _f(idx).reshape(-1)
    out = np.zeros((idx.size, src.shape[-1]), np.float32) if result is None else _f(result).copy()
    lib().orc_indexselect(out, src, idx, idx.size, src.shape[-1], int(is_add))
    return out


def indexselectgrad(grad, adj, idx):
    grad = _f(grad).copy()
    adj = _f(adj)
    idx = _f(idx).reshape(-1)
    lib().orc_indexselectgrad(grad, adj, idx, idx.size, adj.shape[-1])
    return grad


def topk(x, k):
    x = _f(x)
    rows = x.size // x.shape[-1]
    ov = np.empty((rows, k), np.float32)
    oi = np.empty((rows, k), np.float32)
    lib().orc_topk(ov, oi, x, k, rows, x.shape[-1])
    return ov, oi


def argmax(x):
    x = _f(x)
    rows = x.size // x.shape[-1]
    oi = np.empty((rows,), np.float32)
    lib().orc_argmax(oi, x, rows, x.shape[-1])
    return oi


def buildtrimask(rows, cols, value=0.0, masked=-30000.0):
    out = np.empty((rows, cols), np.float32)
    lib().orc_buildtrimask(out, rows, cols, value, masked)
    return out


def buildselftrimask(lens, padded, value=0.0, masked=-30000.0):
    lens = _f(lens)
    rows = lens.size * padded
    out = np.empty((rows, padded), np.float32)
    lib().orc_buildselftrimask(out, lens, rows, padded, padded, value, masked)
    return out


def unary(op, x):
    code = {"relu": 0, "silu": 1, "leakyrelu": 2}[op]
    x = _f(x)
    out = np.empty_like(x)
    lib().orc_unary(code, out, x, x.size)
    return out


def iscorrupted(x):
    x = _f(x)
    return bool(lib().orc_iscorrupted(x, x.size))


def float2half_bits(x):
    x = _f(x)
    out = np.empty(x.shape, np.uint16)
    lib().orc_float2half(out, x, x.size)
    return out


def half_bits2float(h):
    h = np.ascontiguousarray(h, dtype=np.uint16)
    out = np.empty(h.shape, np.float32)
    lib().orc_half2float(out, h, h.size)
    return out


def toppsample(probs, top_p, repeat_penalty, seqs, uniforms):
    probs = _f(probs)
    rows, K = probs.shape
    out = np.empty((rows,), np.float32)
    if seqs is None:
        sp, sl = None, 0
    else:
        seqs = np.ascontiguousarray(seqs, dtype=np.int32)
        sp, sl = seqs.ctypes.data_as(C.c_void_p), seqs.shape[1]
    lib().orc_toppsample(out, probs, rows, K, top_p, repeat_penalty, sp, sl, _f(uniforms))
    return out


def copy_strided(view):
    """Ops.AsContiguous of a numpy view (non-negative strides)."""
    view = np.asarray(view, dtype=np.float32)
    sizes = np.array(view.shape, np.int64)
    strides = np.array([s // 4 for s in view.strides], np.int64)
    span = int(((sizes - 1) * strides).sum() + 1)
    base = np.ascontiguousarray(np.lib.stride_tricks.as_strided(view, shape=(span,), strides=(4,)))
    out = np.empty(view.shape, np.float32)
    _chk(lib().orc_copy_strided(out, base, span, view.ndim, sizes, strides))
    return out


# ---- model -----------------------------------------------------------------------------------
ACT = {"relu": 0, "silu": 1, "leakyrelu": 2, "swiglu": 3, "swiglu_silu": 4}


class OracleGpt:
    """GPTDecoder on the CPU oracle: literal concat cache, expanded GQA heads, [B*H,Tq,T] scores."""

    def __init__(self, cfg, weights):
        """cfg: dict with the Config fields; weights: dict name -> float32 array (reference names)."""
        L = lib()
        self.cfg = dict(cfg)
        c = OrcConfig(cfg["n_layers"], cfg["hidden"], cfg["n_heads"], cfg["n_kv_heads"], cfg["ffn_dim"], cfg["vocab"],
                      cfg["attn_type"], cfg["norm_type"], cfg["act"], cfg.get("n_experts", 1), cfg.get("experts_per_token", 1),
                      cfg.get("norm_eps", 1e-6), cfg.get("rope_base", 500000.0), cfg.get("use_rope", 1),
                      cfg.get("max_segments", 0), cfg.get("sep_token_id", 3))
        self.h = L.orc_gpt_create(C.byref(c))
        for name, w in weights.items():
            w = _f(w)
            _chk(L.orc_gpt_set_weight(self.h, name.encode(), w, w.ndim, np.array(w.shape, np.int64)))

    def __del__(self):
        try:
            lib().orc_gpt_destroy(self.h)
        except Exception:
            pass

    def reset(self):
        lib().orc_gpt_reset_cache(self.h)

    def cache_len(self):
        return lib().orc_gpt_cache_len(self.h)

    def step(self, seqs, use_cache=True, temperature=1.0, sampling=False, want_hidden=False, lens=None):
        """seqs: int array [B, len] (whole sequences so far).  Returns (probs, logits[, hidden]).
        lens: original lengths of sequences that were padded to `len` (the reference's PadSentences + BuildSelfTriMask
        branch); only the first, full-sequence call looks at them."""
        seqs = np.ascontiguousarray(seqs, dtype=np.int32)
        B, ln = seqs.shape
        V = self.cfg["vocab"]
        probs = np.empty((B, V), np.float32)
        logits = np.empty((B, V), np.float32)
        hidden = np.empty((B, self.cfg["hidden"]), np.float32) if want_hidden else None
        if lens is not None:
            _chk(lib().orc_gpt_step_padded(self.h, seqs, B, ln, _f(lens), int(use_cache), temperature, int(sampling),
                                           _vp(probs), _vp(logits), _vp(hidden)))
            return (probs, logits, hidden) if want_hidden else (probs, logits)
        _chk(lib().orc_gpt_step(self.h, seqs, B, ln, int(use_cache), temperature, int(sampling),
                                _vp(probs), _vp(logits), _vp(hidden)))
        return (probs, logits, hidden) if want_hidden else (probs, logits)

    def get_cache(self, layer, which):
        n = lib().orc_gpt_get_cache(self.h, layer, which, None, 0)
        if n == 0:
            return None
        out = np.empty((n,), np.float32)
        lib().orc_gpt_get_cache(self.h, layer, which, _vp(out), n)
        return out

    def set_cache(self, layer, which, data, BH, T, d):
        _chk(lib().orc_gpt_set_cache(self.h, layer, which, _f(data), BH, T, d))

    def moe_trace(self, ordinal, R=None):
        """Routing of MoE layer number `ordinal` at the last step, for all rows that step fed (B at a cached step, B * len
        at a full-sequence step).  R, when given, must be that row count."""
        k, E = self.cfg["experts_per_token"], self.cfg["n_experts"]
        n = lib().orc_gpt_moe_trace(self.h, ordinal, None, None, None, 0)
        if n < 0:
            raise IndexError("no such MoE layer trace")
        rows = n // k
        if R is not None and R != rows:
            raise ValueError("the last step routed %d rows, not %d" % (rows, R))
        ti = np.empty((rows, k), np.float32)
        tv = np.empty((rows, k), np.float32)
        pr = np.empty((rows, E), np.float32)
        lib().orc_gpt_moe_trace(self.h, ordinal, _vp(ti), _vp(tv), _vp(pr), rows * k)
        return ti, tv, pr

    def moe_layer(self, layer, x):
        x = _f(x)
        R = x.shape[0]
        k, E = self.cfg["experts_per_token"], self.cfg["n_experts"]
        y = np.empty_like(x)
        ti = np.empty((R, k), np.float32)
        tv = np.empty((R, k), np.float32)
        pr = np.empty((R, E), np.float32)
        _chk(lib().orc_moe_layer(self.h, layer, x, R, y, _vp(ti), _vp(tv), _vp(pr)))
        return y, ti, tv, pr

    def attn_layer(self, layer, x, B, Tq, causal, use_cache):
        x = _f(x)
        y = np.empty_like(x)
        _chk(lib().orc_attn_layer(self.h, layer, x, B, Tq, int(causal), int(use_cache), y))
        return y

    def ffn_layer(self, layer, x):
        x = _f(x)
        y = np.empty_like(x)
        _chk(lib().orc_ffn_layer(self.h, layer, x, x.shape[0], y))
        return y


# ---- beam search (pure Python: small cases only) ------------------------------------------------
class FixedSizePriorityQueue:
    """AdvUtils/FixedSizePriorityQueue.cs:10-341 with ComparableItemComparer(false) (Seq2SeqSharp/Tools/ComparableItem.cs:31-50),
    as BeamSearch.GetTopNBSS uses it (Utils/BeamSearch.cs:36-46).  Items are (score, payload); lower scores are better.
    Two array heaps: `top` (better half, best at the root) and `bottom` (worst at the root); enumeration = top in array
    order, then bottom in reverse array order."""

    def __init__(self, capacity):
        assert capacity >= 1
        self.cap, self.count, self.nb, self.nt = capacity, 0, 0, 0
        bcap = max(capacity // 2, 1)
        self.top = [None] * max(capacity - bcap, 1)
        self.bottom = [None] * bcap

    @staticmethod
    def _better(a, b, f_top):
        d = np.float32(a[0]) - np.float32(b[0])
        c = -(1 if d > 0 else (-1 if d < 0 else 0))         # Compare(x, y) = -Math.Sign(x.Score - y.Score)
        return c > 0 if f_top else c < 0

    def _up(self, arr, i, f_top):                           # UpHeapify :198-208
        while i > 0:
            p = (i - 1) // 2
            if not self._better(arr[i], arr[p], f_top):
                return i
            arr[i], arr[p] = arr[p], arr[i]
            i = p
        return i

    def _down(self, arr, i, size, f_top):                   # DownHeapify :210-224
        while True:
            l, r, best = 2 * i + 1, 2 * i + 2, i
            if l < size and self._better(arr[l], arr[best], f_top):
                best = l
            if r < size and self._better(arr[r], arr[best], f_top):
                best = r
            if best == i:
                return i
            arr[i], arr[best] = arr[best], arr[i]
            i = best

    def _top1(self, i):                                     # TopNode1 :176-182
        return 2 * i + 1 if self.nb <= 2 * i + 1 < self.nt else i

    def _top2(self, i):                                     # TopNode2 :184-195
        if i == self.nb - 1 and i % 2 == 1 and self.nt > self.nb:
            return i + 1
        return 2 * i + 1 if self.nb <= 2 * i + 1 < self.nt else i

    def _boundary_up(self, bpos):                           # CheckBoundaryUpwards :226-249
        t1, t2, b = self._top1(bpos), self._top2(bpos), -1
        if self._better(self.bottom[bpos], self.top[t1], True):
            b = t1
        if self._better(self.bottom[bpos], self.top[t2], True) and (b == -1 or self._better(self.top[t1], self.top[t2], True)):
            b = t2
        if b == -1:
            return -1
        self.top[b], self.bottom[bpos] = self.bottom[bpos], self.top[b]
        return b

    def _boundary_down(self, tpos):                         # CheckBoundaryDownwards :251-268, BottomNode :163-174
        if tpos < self.nb:
            bpos = tpos
        else:
            bpos = (tpos - 1) // 2 if tpos % 2 == 1 else tpos - 1
        if bpos == -1:
            return -1
        if bpos >= self.nb or not self._better(self.bottom[bpos], self.top[tpos], True):
            return -1
        self.top[tpos], self.bottom[bpos] = self.bottom[bpos], self.top[tpos]
        return bpos

    def enqueue(self, item):                                # Enqueue :56-149
        if self.cap == self.count:
            if self.cap == 1:
                if not self._better(item, self.top[0], True):
                    return False
                self.top[0] = item
                return True
            if not self._better(item, self.bottom[0], True):
                return False
            self.bottom[0] = item
            upd = self._down(self.bottom, 0, self.nb, False)
            if not (2 * upd + 2 >= self.nb):                # SemiLeaf
                return True
            it = self._boundary_up(upd)
            if it == -1:
                return True
            self._up(self.top, it, True)
            return True
        self.count += 1
        if self.nb < self.nt:
            pos = self.nb
            self.nb += 1
            self.bottom[pos] = item
            up = self._boundary_up(pos)
            if up == -1:
                self._up(self.bottom, pos, False)
            else:
                self._up(self.top, up, True)
            return True
        pos = self.nt
        self.nt += 1
        self.top[pos] = item
        bt = self._boundary_down(pos)
        if bt == -1:
            self._up(self.top, pos, True)
        else:
            self._up(self.bottom, bt, False)
        return True

    def items(self):                                        # GetEnumerator :306-312
        return [self.top[i] for i in range(self.nt)] + [self.bottom[i] for i in range(self.nb - 1, -1, -1)]


def get_top_n(scores, top_n):
    """BeamSearch.GetTopNBSS on a list of scores: indices of the survivors in the queue's enumeration order."""
    q = FixedSizePriorityQueue(top_n)
    for i, s in enumerate(scores):
        q.enqueue((np.float32(s), i))
    return [it[1] for it in q.items()]


def beam_picks(probs, n_picks, top_p=None, repeat_penalty=0.0, seqs=None, uniforms=None):
    """The pick loop of Decoder.GPTDecode (Applications/Decoder.cs:756-792): Argmax (top_p None) or TopPSample, Gather + Log of
    the picked probability, ScatterFill(probs, 0) at the pick before the next one.  probs [B, V] (blocked tokens already
    lowered by 1).  Returns (ids [n_picks, B], log p [n_picks, B])."""
    p = _f(probs).copy()
    B = p.shape[0]
    ids = np.zeros((n_picks, B), np.int32)
    logp = np.zeros((n_picks, B), np.float32)
    for i in range(n_picks):
        if top_p is None:
            pick = argmax(p).astype(np.int32)
        else:
            pick = toppsample(p, top_p, repeat_penalty, seqs, uniforms[i]).astype(np.int32)
        ids[i] = pick
        with np.errstate(divide="ignore"):
            logp[i] = np.log(p[np.arange(B), pick].astype(np.float64)).astype(np.float32)      # (float)Math.Log
        p[np.arange(B), pick] = 0.0
    return ids, logp


def gpt_beam_search(orc, prompts, beam_size, max_len, eos_id=0, top_p=None, repeat_penalty=0.0, uniforms=None, temperature=1.0):
    """GPT.RunForwardOnSingleDevice for BeamSearchSize > 1 (Applications/GPT.cs:264-302) on an OracleGpt: no KV cache (the
    dictionary only exists for beam size 1, :238-241), every beam's batch recomputed from its first token each step.
    uniforms [steps, beam_size picks, beams * batch] (beam-major rows).  Returns (hypotheses [batch][beam], scores)."""
    prompts = np.ascontiguousarray(prompts, dtype=np.int32)
    B, T0 = prompts.shape
    beams = [[(list(map(int, prompts[b])), np.float32(1.0)) for b in range(B)]]       # beam2batchStatus; Score starts at 1.0f
    step = 0
    for _ in range(T0, max_len):
        per_batch = [[] for _ in range(B)]
        for j, batch_status in enumerate(beams):
            seqs = np.array([h[0] for h in batch_status], np.int32)
            p, _ = orc.step(seqs, use_cache=False, temperature=temperature, sampling=top_p is not None)
            u = None if uniforms is None else [uniforms[step][i][j * B:(j + 1) * B] for i in range(beam_size)]
            ids, logp = beam_picks(p, beam_size, top_p, repeat_penalty, seqs if top_p is not None else None, u)
            for b in range(B):
                for i in range(beam_size):
                    per_batch[b].append((batch_status[b][0] + [int(ids[i, b])], np.float32(batch_status[b][1] + np.float32(-1.0) * logp[i, b])))
        if beam_size > 1:
            per_batch = [[c[k] for k in get_top_n([h[1] for h in c], beam_size)] for c in per_batch]
        beams = [[per_batch[b][j] for b in range(B)] for j in range(len(per_batch[0]))]
        step += 1
        if all(h[0][-1] == eos_id for bs in beams for h in bs):
            break
    hyp = [[beams[j][b][0] for j in range(len(beams))] for b in range(B)]
    sc = [[float(beams[j][b][1]) for j in range(len(beams))] for b in range(B)]
    return hyp, sc
