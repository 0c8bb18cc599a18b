"""The reference's layer code replayed, op for op, on the per-op C-ABI surface.

`ComputeGraph` mirrors the inference half of Seq2SeqSharp's IComputeGraph / ComputeGraphTensor
(Seq2SeqSharp/Tools/ComputeGraphTensor.cs): every method allocates its result and issues the same TensorSharp
op the reference issues.  The layer functions below are line-by-line replays of
GroupQueryAttention.Perform (Seq2SeqSharp/Layers/GroupQueryAttention.cs:114-233),
MultiHeadAttention.PerformClassic (Layers/MultiHeadAttention.cs:125-240) and
PositionwiseFeedForward.Process (Layers/PositionwiseFeedForward.cs:72-98), concat KV cache included.
They exist to show that the unmodified layer code runs on this backend; the fast path is seq2seqsharp_amd.gpt.
"""
import math

import numpy as np

from . import ops
from .tensor import F16, F32, HipTensor


class ComputeGraph:
    def Affine(self, x, W, b):                    # ComputeGraphTensor.cs:1848-1880
        n, d = x.sizes[0], W.sizes[1]
        be = b.expand(n, d)
        r = ops.addmm(HipTensor([n, d], x.dtype), 1.0, be, 1.0, x, W)
        be.dispose()
        return r

    def Mul(self, a, b, alpha=1.0):               # ComputeGraphTensor.cs:1752-1763
        if isinstance(b, HipTensor):
            r = HipTensor([a.sizes[0], b.sizes[1]], a.dtype)
            return ops.addmm(r, 0.0, r, alpha, a, b)
        return ops.mul(None, a, b)

    def MulBatch(self, a, b, alpha=1.0):          # ComputeGraphTensor.cs:1659-1666
        r = HipTensor([a.sizes[0], a.sizes[1], b.sizes[2]], a.dtype)
        return ops.addmmbatch(r, 0.0, r, alpha, a, b)

    def View(self, t, dims):                      # ComputeGraphTensor.cs:3094-3134
        return t.view(list(dims))

    def Transpose(self, t, d1, d2):
        return t.transpose(d1, d2)

    def Expand(self, t, dims):
        return t.expand(list(dims))

    def Select(self, t, dim, idx):
        return t.select(dim, idx)

    def AsContiguous(self, t):                    # ComputeGraphTensor.cs:3038-3057
        return ops.as_contiguous(t)

    def RoPE(self, t, seq_len, offset):           # ComputeGraphTensor.cs:490-497
        return ops.rope(None, t, seq_len, offset)

    def Concate(self, dim, a, b):                 # ComputeGraphTensor.cs:2838-2873
        return ops.concat(dim, [a, b])

    def Softmax(self, t, in_place=False):         # ComputeGraphTensor.cs:2444-2460
        return ops.softmax(t if in_place else None, t)

    def Add(self, a, b, in_place=False):          # ComputeGraphTensor.cs:895-919
        return ops.add(a if in_place else None, a, b)

    def EltMul(self, a, b):
        return ops.mul(None, a, b)

    def RMSNorm(self, x, alpha, beta, eps):       # ComputeGraphTensor.cs:3471-3483
        return ops.rmsnorm(None, x, alpha, beta, eps)

    def LayerNorm(self, x, alpha, beta, eps):     # ComputeGraphTensor.cs:3352-3361
        return ops.layernorm(None, x, alpha, beta, eps)

    def IndexSelect(self, src, idx):              # ComputeGraphTensor.cs:2791-2831
        return ops.indexselect(None, src, idx)

    def Act(self, act, t):                        # RunActivateFunction, PositionwiseFeedForward.cs:100-116
        if act == 1:
            return ops.silu(t, t)
        if act == 0:
            return ops.relu(t, t)
        if act == 2:
            return ops.leakyrelu(t, t)
        return t


class DeviceWeights:
    """The model's parameters as device tensors under the reference's names."""

    def __init__(self, weights, dtype=F32):
        """dtype F16: the model as the reference holds it with AMP (every parameter Float16, Applications/GPT.cs:122-130)."""
        self.dtype = dtype
        self.t = {k: HipTensor.from_numpy(np.asarray(v, np.float32), dtype) for k, v in weights.items()}

    def __getitem__(self, k):
        return self.t[k]


def _norm(g, cfg, W, prefix, x):
    if cfg["norm_type"] == 1:
        return g.LayerNorm(x, W[prefix + ".m_alpha"], W[prefix + ".m_beta"], cfg["norm_eps"])
    return g.RMSNorm(x, W[prefix + ".m_alpha"], None, cfg["norm_eps"])


def _attn_tail(g, cfg, W, name, Qs, Ks, Vs, mask, B, Tq, H, d, inputQ, cache):
    kn, vn = name + "_cached_K", name + "_cached_V"
    if cache is not None:
        if kn in cache:
            Ks = g.Concate(2, cache[kn], Ks)
        cache[kn] = Ks
        if vn in cache:
            Vs = g.Concate(1, cache[vn], Vs)
        cache[vn] = Vs
    Tkv = Ks.sizes[2]
    scale = np.float32(1.0) / np.float32(math.sqrt(d))
    use_f16 = Qs.dtype == F16                     # GroupQueryAttention.cs:196-201: scores, mask and softmax run in Float32
    if use_f16:
        Qs, Ks = ops.half2float(None, Qs), ops.half2float(None, Ks)
    attn = g.MulBatch(Qs, Ks, float(scale))
    attn = g.View(attn, [B, H, Tq, Tkv])
    if mask is not None:
        if use_f16:
            mask = ops.half2float(None, mask)     # :209-212 (the expanded view is materialised by the conversion)
        attn = g.Add(attn, mask, in_place=True)
    attn = g.Softmax(attn, in_place=True)
    if use_f16:
        attn = ops.float2half(None, attn)         # :216-219
    attn = g.View(attn, [B * H, Tq, Tkv])
    o = g.View(g.MulBatch(attn, Vs), [B, H, Tq, d])
    Wt = g.View(g.AsContiguous(g.Transpose(o, 1, 2)), [B * Tq, H * d])
    fin = g.Affine(Wt, W[name + ".W0"], W[name + ".b0"])
    return g.Add(fin, inputQ)


def group_query_attention(g, cfg, W, layer, inputQ, mask, B, cache):
    name = "GPTDecoder.SelfAttn_%d" % layer
    H, G = cfg["n_heads"], cfg["n_kv_heads"]
    d = cfg["hidden"] // H
    Tq = inputQ.sizes[0] // B
    n = _norm(g, cfg, W, name + ".layerNormQ", inputQ)
    allQ = g.View(g.Affine(n, W[name + ".Q"], W[name + ".Qb"]), [B, Tq, H, d])
    allK = g.View(g.Affine(n, W[name + ".K"], W[name + ".Kb"]), [B, Tq, G, d])
    allV = g.View(g.Affine(n, W[name + ".V"], W[name + ".Vb"]), [B, Tq, G, d])
    off = cache[name + "_cached_K"].sizes[2] if cache is not None and name + "_cached_K" in cache else 0
    Qs = g.View(g.AsContiguous(g.Transpose(allQ, 1, 2)), [B * H, Tq, d])
    Qs = g.RoPE(Qs, Tq, off)
    gs = H // G
    Ks = g.View(g.AsContiguous(g.Transpose(allK, 1, 2)), [B * G, Tq, d])
    Ks = g.RoPE(Ks, Tq, off)
    Ks = g.View(Ks, [B, G, 1, Tq, d])
    Ks = g.Expand(Ks, [B, G, gs, Tq, d])
    Ks = g.Transpose(Ks, 3, 4)
    Ks = g.View(g.AsContiguous(Ks), [B * H, d, Tq])
    Vs = g.AsContiguous(g.Transpose(allV, 1, 2))
    Vs = g.View(Vs, [B, G, 1, Tq, d])
    Vs = g.Expand(Vs, [B, G, gs, Tq, d])
    Vs = g.View(g.AsContiguous(Vs), [B * H, Tq, d])
    return _attn_tail(g, cfg, W, name, Qs, Ks, Vs, mask, B, Tq, H, d, inputQ, cache)


def multi_head_attention(g, cfg, W, layer, inputQ, mask, B, cache):
    name = "GPTDecoder.SelfAttn_%d" % layer
    H = cfg["n_heads"]
    d = cfg["hidden"] // H
    Tq = inputQ.sizes[0] // B
    n = _norm(g, cfg, W, name + ".layerNormQ", inputQ)
    qkv = g.View(g.Affine(n, W[name + ".QKV"], W[name + ".QKVb"]), [B, Tq, 3, H, d])
    allQ, allK, allV = g.Select(qkv, 2, 0), g.Select(qkv, 2, 1), g.Select(qkv, 2, 2)
    off = cache[name + "_cached_K"].sizes[2] if cache is not None and name + "_cached_K" in cache else 0
    Qs = g.View(g.AsContiguous(g.Transpose(allQ, 1, 2)), [B * H, Tq, d])
    Qs = g.RoPE(Qs, Tq, off)
    Ks = g.View(g.AsContiguous(g.Transpose(allK, 1, 2)), [B * H, -1, d])
    Ks = g.RoPE(Ks, Tq, off)
    Ks = g.View(g.AsContiguous(g.Transpose(Ks, 1, 2)), [B * H, d, -1])
    Vs = g.View(g.AsContiguous(g.Transpose(allV, 1, 2)), [B * H, -1, d])
    return _attn_tail(g, cfg, W, name, Qs, Ks, Vs, mask, B, Tq, H, d, inputQ, cache)


def positionwise_feed_forward(g, cfg, W, layer, x):
    name = "GPTDecoder.PosFFN_%d" % layer
    n = _norm(g, cfg, W, name + ".layerNorm2", x)
    a = g.Affine(n, W[name + ".feedForwardLayer1.m_Whd"], W[name + ".feedForwardLayer1.m_Bd"])
    a = g.Act(cfg["act"], a)
    if cfg["act"] in (3, 4):
        c = g.Affine(n, W[name + ".feedForwardLayer3.m_Whd"], W[name + ".feedForwardLayer3.m_Bd"])
        a = g.EltMul(a, c)
    y = g.Affine(a, W[name + ".feedForwardLayer2.m_Whd"], W[name + ".feedForwardLayer2.m_Bd"])
    return g.Add(y, x)


def gpt_decode_step(g, cfg, W, seqs, cache):
    """Decoder.GPTDecode up to the probabilities (Seq2SeqSharp/Applications/Decoder.cs:648-732), dense layers only.
    seqs: int array [B, len].  Returns (probs, logits) as device tensors.  With Float16 weights (DeviceWeights(..., F16))
    this is the AMP run: every tensor Float16 except the attention scores and the logits handed to the softmax."""
    amp = getattr(W, "dtype", F32) == F16
    seqs = np.asarray(seqs)
    B, ln = seqs.shape
    H = cfg["n_heads"]
    mask = None
    if cache:
        Tq, ids = 1, seqs[:, -1].astype(np.float32)
    else:
        Tq, ids = ln, seqs.reshape(-1).astype(np.float32)
        m = ops.buildtrimask(HipTensor([Tq, Tq], F16 if amp else F32), 0.0, -30000.0)      # Decoder.cs:685: the mask has the model's type
        mask = m.view(1, 1, Tq, Tq).expand(B, H, Tq, Tq)
    idx = HipTensor.from_numpy(ids.reshape(-1, 1))
    x = g.IndexSelect(W["TgtEmbeddings"], idx)
    x = ops.mul(x, x, float(np.float32(math.sqrt(cfg["hidden"]))))
    for k in range(cfg["n_layers"]):
        attn = group_query_attention if cfg["attn_type"] == 1 else multi_head_attention
        x2 = attn(g, cfg, W, k, x, mask, B, cache)
        x = positionwise_feed_forward(g, cfg, W, k, x2)
    x = _norm(g, cfg, W, "GPTDecoder.layerNorm", x)
    last = HipTensor.from_numpy(np.array([Tq * (i + 1) - 1 for i in range(B)], np.float32).reshape(-1, 1))
    x = g.IndexSelect(x, last)
    logits = g.Affine(x, W["FeedForward_Decoder_0.m_Whd"], W["FeedForward_Decoder_0.m_Bd"])
    if amp:
        logits = ops.half2float(None, logits)     # Decoder.cs:725-730
    probs = ops.softmax(None, logits)
    return probs, logits
