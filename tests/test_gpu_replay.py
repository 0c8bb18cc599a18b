"""The reference's layer code replayed op by op on the per-op C-ABI surface (seq2seqsharp_amd.graph) against the
oracle's literal restatement of the same layers: same op sequence, concat KV cache, expanded GQA heads."""
import numpy as np
import pytest

from seq2seqsharp_amd import synth

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("kw", [dict(), dict(attn_type=synth.MHA, n_kv_heads=4, norm_type=synth.LAYERNORM, act=synth.RELU),
                                dict(act=synth.SILU, hidden=128, n_heads=4, n_kv_heads=1)])
def test_decode_loop_through_the_op_registry_surface(oracle, kw):
    from seq2seqsharp_amd import graph
    cfg = synth.tiny_config(**kw)
    w = synth.make_weights(cfg, 5, random_bias=True)
    orc = oracle.OracleGpt(cfg, w)
    W = graph.DeviceWeights(w)
    g = graph.ComputeGraph()
    cache = {}
    cur = synth.make_prompts(cfg, 6)
    for step in range(4):
        p, lg = orc.step(cur, use_cache=True)
        probs, logits = graph.gpt_decode_step(g, cfg, W, cur, cache)
        assert np.abs(logits.numpy() - lg).max() / np.abs(lg).max() <= 1e-4
        nxt = oracle.argmax(p).astype(np.int32)
        from seq2seqsharp_amd import ops
        assert np.array_equal(ops.argmax(None, probs, 1).numpy().reshape(-1), nxt.astype(np.float32))
        cur = np.concatenate([cur, nxt[:, None]], 1)
    # the concat cache has the reference's layout: K [B*H, d, T], V [B*H, T, d]
    k = cache["GPTDecoder.SelfAttn_0_cached_K"]
    B, H, d = cfg["batch"], cfg["n_heads"], cfg["hidden"] // cfg["n_heads"]
    assert k.sizes == [B * H, d, cfg["prompt"] + 3]
    assert np.abs(k.numpy().reshape(-1) - orc.get_cache(0, 0)).max() <= 1e-5


@pytest.mark.parametrize("kw", [dict(hidden=128, n_heads=4, n_kv_heads=2, ffn_dim=256, vocab=200),
                                dict(attn_type=synth.MHA, n_kv_heads=4, norm_type=synth.LAYERNORM, act=synth.RELU, vocab=96)])
def test_amp_decode_loop_through_the_op_registry_surface(oracle, kw):
    """The same replay with every parameter Float16, as the reference runs with AMP: Float16 Affine (the matrix-core GEMM
    where rows are contiguous), norms, RoPE, copies and adds; scores, mask and softmax in Float32 between Half2Float and
    Float2Half (GroupQueryAttention.cs:196-220).  Every intermediate is rounded to Float16 here, the residual stream
    included, so the distance to the fp32 oracle (on the same fp16-rounded weights) is larger than the fused path's."""
    from seq2seqsharp_amd import graph, ops
    from seq2seqsharp_amd.tensor import F16
    cfg = synth.tiny_config(dtype="f16", **kw)
    w = synth.make_weights(cfg, 5, random_bias=True)
    orc = oracle.OracleGpt(cfg, w)
    W = graph.DeviceWeights(w, F16)
    g = graph.ComputeGraph()
    cache = {}
    cur = synth.make_prompts(cfg, 6)
    for step in range(4):
        p, lg = orc.step(cur, use_cache=True)
        probs, logits = graph.gpt_decode_step(g, cfg, W, cur, cache)
        assert logits.dtype == 0 and cache["GPTDecoder.SelfAttn_0_cached_K"].dtype == F16
        assert np.abs(logits.numpy() - lg).max() <= 3e-2
        cur = np.concatenate([cur, oracle.argmax(p).astype(np.int32)[:, None]], 1)
