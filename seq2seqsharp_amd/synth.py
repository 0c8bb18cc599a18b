"""Synthetic GPTDecoder models: the benchmark configurations and seeded random weights.

Weight names and shapes follow the reference's saved parameter names
(Seq2SeqSharp/Networks/GPTDecoder.cs:90-132, Layers/GroupQueryAttention.cs:76-95,
Layers/MultiHeadAttention.cs:89-90, Layers/PositionwiseFeedForward.cs:44-59,
Layers/MoEFeedForward.cs:49-55, Applications/GPT.cs:125-130).  The reference never random-initialises
inference-mode tensors (Tools/WeightTensor.cs:181-204), so the harness supplies N(0, 0.02) itself.
"""
import numpy as np

MHA, GQA = 0, 1
RMSNORM, LAYERNORM = 0, 1
RELU, SILU, LEAKYRELU, SWIGLU, SWIGLU_SILU = 0, 1, 2, 3, 4


def _cfg(**kw):
    base = dict(n_experts=1, experts_per_token=1, norm_eps=1e-6, rope_base=500000.0, use_rope=1, dtype="f32")
    base.update(kw)
    return base


# The five configurations of the benchmark contract.  rope_base is the reference's literal 500000
# (TensorSharp/TensorApplyCPU.cs:1161) and "SwiGLU" is the reference's gate without SiLU
# (Layers/PositionwiseFeedForward.cs:80-94).
CONFIGS = {
    "cfg0_tiny_mha_f32": _cfg(n_layers=6, hidden=512, n_heads=8, n_kv_heads=8, ffn_dim=2048, vocab=32000,
                              attn_type=MHA, norm_type=RMSNORM, act=SWIGLU, batch=1, prompt=64, steps=128),
    "cfg1_gpt2small_f32": _cfg(n_layers=12, hidden=768, n_heads=12, n_kv_heads=12, ffn_dim=3072, vocab=32000,
                               attn_type=MHA, norm_type=LAYERNORM, act=RELU, batch=8, prompt=512, steps=256),
    "cfg1_gpt2small_f16": _cfg(n_layers=12, hidden=768, n_heads=12, n_kv_heads=12, ffn_dim=3072, vocab=32000,
                               attn_type=MHA, norm_type=LAYERNORM, act=RELU, batch=8, prompt=512, steps=256, dtype="f16"),
    "cfg2_1b_gqa_f16": _cfg(n_layers=16, hidden=2048, n_heads=32, n_kv_heads=8, ffn_dim=5632, vocab=32000,
                            attn_type=GQA, norm_type=RMSNORM, act=SWIGLU, batch=32, prompt=1024, steps=256, dtype="f16"),
    "cfg3_moe_f16": _cfg(n_layers=12, hidden=1024, n_heads=16, n_kv_heads=4, ffn_dim=4096, vocab=32000,
                         attn_type=GQA, norm_type=LAYERNORM, act=RELU, n_experts=8, experts_per_token=2,
                         batch=64, prompt=256, steps=128, dtype="f16"),
    "cfg4_7b_longctx_f16": _cfg(n_layers=32, hidden=4096, n_heads=32, n_kv_heads=8, ffn_dim=11008, vocab=32000,
                                attn_type=GQA, norm_type=RMSNORM, act=SWIGLU, batch=16, prompt=8192, steps=128, dtype="f16"),
}


def tiny_config(**kw):
    """A model small enough for the CPU oracle to run in milliseconds."""
    c = _cfg(n_layers=2, hidden=64, n_heads=4, n_kv_heads=2, ffn_dim=128, vocab=97,
             attn_type=GQA, norm_type=RMSNORM, act=SWIGLU, batch=2, prompt=8, steps=8)
    c.update(kw)
    return c


def weight_shapes(cfg):
    """Ordered list of (name, shape, kind); kind in {'normal','ones','zeros'}."""
    h, H, G, F, V, L = cfg["hidden"], cfg["n_heads"], cfg["n_kv_heads"], cfg["ffn_dim"], cfg["vocab"], cfg["n_layers"]
    d = h // H
    ln = cfg["norm_type"] == LAYERNORM
    out = [("TgtEmbeddings", (V, h), "normal")]
    if cfg.get("max_segments", 0) > 0:          # Misc.CreateAuxEmbeddings: "SegmentEmbedding" [MaxSegmentNum, EncoderEmbeddingDim]
        out.append(("SegmentEmbedding", (cfg["max_segments"], h), "normal"))

    def norm(prefix):
        out.append((prefix + ".m_alpha", (1, h), "ones"))
        if ln:
            out.append((prefix + ".m_beta", (1, h), "zeros"))

    for i in range(L):
        a = f"GPTDecoder.SelfAttn_{i}"
        norm(a + ".layerNormQ")
        if cfg["attn_type"] == GQA:
            out += [(a + ".Q", (h, H * d), "normal"), (a + ".Qb", (1, H * d), "zeros"),
                    (a + ".K", (h, G * d), "normal"), (a + ".Kb", (1, G * d), "zeros"),
                    (a + ".V", (h, G * d), "normal"), (a + ".Vb", (1, G * d), "zeros")]
        else:
            out += [(a + ".QKV", (h, 3 * h), "normal"), (a + ".QKVb", (1, 3 * h), "zeros")]
        out += [(a + ".W0", (h, h), "normal"), (a + ".b0", (1, h), "zeros")]
        if cfg["n_experts"] > 1 and i > 1:
            f = f"GPTDecoder.MoEFFN_{i}"
            E = cfg["n_experts"]
            out += [(f + ".layerNorm.m_alpha", (1, h), "ones"), (f + ".layerNorm.m_beta", (1, h), "zeros"),
                    (f + ".m_Router", (h, E), "normal"), (f + ".m_RouterBias", (1, E), "zeros"),
                    (f + ".m_Whd1", (E, h, 4 * h), "normal"), (f + ".m_Whd2", (E, 4 * h, h), "normal")]
        else:
            f = f"GPTDecoder.PosFFN_{i}"
            norm(f + ".layerNorm2")
            out += [(f + ".feedForwardLayer1.m_Whd", (h, F), "normal"), (f + ".feedForwardLayer1.m_Bd", (1, F), "zeros")]
            if cfg["act"] in (SWIGLU, SWIGLU_SILU):
                out += [(f + ".feedForwardLayer3.m_Whd", (h, F), "normal"), (f + ".feedForwardLayer3.m_Bd", (1, F), "zeros")]
            out += [(f + ".feedForwardLayer2.m_Whd", (F, h), "normal"), (f + ".feedForwardLayer2.m_Bd", (1, h), "zeros")]
    norm("GPTDecoder.layerNorm")
    out += [("FeedForward_Decoder_0.m_Whd", (h, V), "normal"), ("FeedForward_Decoder_0.m_Bd", (1, V), "zeros")]
    return out


def n_params(cfg):
    return sum(int(np.prod(s)) for _, s, _ in weight_shapes(cfg))


def iter_weights(cfg, seed=0, std=0.02, random_bias=False, round_f16=None):
    """Yield (name, float32 array) in a fixed order from one seeded stream.

    round_f16: round every tensor to the nearest half (RNE) and back, so that an fp32 consumer sees exactly
    the values an fp16 device copy holds.  Defaults to cfg['dtype'] == 'f16'.
    random_bias: draw biases and norm gains/offsets at random too (tests use it so that a dropped bias shows).
    """
    if round_f16 is None:
        round_f16 = cfg.get("dtype", "f32") == "f16"
    rng = np.random.default_rng(seed)
    for name, shape, kind in weight_shapes(cfg):
        if kind == "normal":
            w = rng.standard_normal(shape, dtype=np.float32) * np.float32(std)
        elif kind == "ones":
            w = np.ones(shape, np.float32)
            if random_bias:
                w = w + rng.standard_normal(shape, dtype=np.float32) * np.float32(0.1)
        else:
            w = np.zeros(shape, np.float32)
            if random_bias:
                w = rng.standard_normal(shape, dtype=np.float32) * np.float32(std)
        if round_f16:
            w = w.astype(np.float16).astype(np.float32)
        yield name, w


def make_weights(cfg, seed=0, **kw):
    return dict(iter_weights(cfg, seed, **kw))


def make_prompts(cfg, seed=1, batch=None, length=None):
    """Uniform ids in [4, vocab): ids 0-3 are EOS/BOS/UNK/SEP in the reference (Utils/Vocab.cs:23-30)."""
    rng = np.random.default_rng(seed)
    B = batch or cfg["batch"]
    T = length or cfg["prompt"]
    return rng.integers(4, cfg["vocab"], size=(B, T), dtype=np.int32)


def make_uniforms(seed, batch, steps):
    """The shared uniform stream for top-p: one draw per row per step, row-major inside a step."""
    return np.random.default_rng(seed).random((steps, batch), dtype=np.float32)
