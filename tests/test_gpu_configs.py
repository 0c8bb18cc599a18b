"""The benchmark contract's configurations at their own layer shapes, against the CPU oracle where it finishes in
seconds (reduced depth, short prompts) and through size-independent properties at full context.

Bars: fp32 logits max relative error <= 1e-4 with identical greedy tokens; fp16 logits max absolute error <= 3e-2 with
>= 99 % per-step top-1 agreement, where a row whose winner differs only counts as a miss when the oracle's own gap
between the two candidates exceeds what the measured logit error can explain (twice the row's max |dlogit|): two
logits closer than the fp16 path's error are a tie in everything but name."""
import numpy as np
import pytest

from parity_util import top1_agreement
from seq2seqsharp_amd import synth

pytestmark = pytest.mark.gpu

FP32_REL = 1e-4
FP16_ABS = 3e-2


@pytest.fixture(scope="module")
def G():
    from seq2seqsharp_amd import gpt
    return gpt


def teacher_forced(G, oracle, cfg, seed, steps, max_batch=None, prompt_seed=None):
    w = synth.make_weights(cfg, seed, random_bias=True)
    orc = oracle.OracleGpt(cfg, w)
    gpu = G.HipGpt(cfg, w, max_batch=max_batch or cfg["batch"], max_seq_len=cfg["prompt"] + steps + 2)
    seqs = synth.make_prompts(cfg, seed + 100 if prompt_seed is None else prompt_seed)
    p, lg = orc.step(seqs, use_cache=True)
    gpu.prefill(seqs)
    out = [(lg, gpu.logits())]
    cur = seqs
    for _ in range(steps):
        nxt = oracle.argmax(p).astype(np.int32)
        cur = np.concatenate([cur, nxt[:, None]], 1)
        p, lg = orc.step(cur, use_cache=True)
        gpu.decode(nxt)
        out.append((lg, gpu.logits()))
    return orc, gpu, out, cur


def check_fp16(out):
    fr = []
    for lg, gl in out:
        assert np.abs(gl - lg).max() <= FP16_ABS
        fr.append(top1_agreement(gl, lg)[0])
    assert np.mean(fr) >= 0.99


def test_cfg0_full_run_greedy_tokens(G, oracle):
    """Configuration 0 as the contract states it: 6 layers, hidden 512, 8 heads, gated FFN 2048, RMSNorm, vocab 32000, fp32,
    batch 1, prompt 64, 128 greedy steps.  Identical tokens at every step; final logits within 1e-4 relative."""
    cfg = dict(synth.CONFIGS["cfg0_tiny_mha_f32"])
    w = synth.make_weights(cfg, 0)
    orc = oracle.OracleGpt(cfg, w)
    gpu = G.HipGpt(cfg, w, max_batch=1, max_seq_len=64 + 130)
    seqs = synth.make_prompts(cfg, 1)
    gpu.prefill(seqs)
    ids, _ = gpu.generate(128)
    cur = seqs
    for s in range(128):
        p, lg = orc.step(cur, use_cache=True)
        nxt = oracle.argmax(p).astype(np.int32)
        assert nxt[0] == ids[s, 0], "step %d" % s
        cur = np.concatenate([cur, nxt[:, None]], 1)
    _, lg = orc.step(cur, use_cache=True)
    gl = gpu.logits()
    assert float(np.abs(gl - lg).max() / np.abs(lg).max()) <= FP32_REL
    gpu.close()


def test_cfg1_fp32_full_depth_greedy_tokens(G, oracle):
    """Configuration 1 at its full depth and width (12 layers, hidden 768, 12 heads, FFN 3072 ReLU, LayerNorm, fused QKV,
    vocab 32000, fp32, batch 8, prompt 512): 16 greedy steps (the budget the CPU reference is given on this
    configuration), identical tokens, logits within 1e-4 relative at the first and the last step."""
    cfg = dict(synth.CONFIGS["cfg1_gpt2small_f32"])
    w = synth.make_weights(cfg, 0)
    orc = oracle.OracleGpt(cfg, w)
    gpu = G.HipGpt(cfg, w, max_batch=cfg["batch"], max_seq_len=cfg["prompt"] + 20)
    seqs = synth.make_prompts(cfg, 1)
    gpu.prefill(seqs)
    p, lg = orc.step(seqs, use_cache=True)
    assert float(np.abs(gpu.logits() - lg).max() / np.abs(lg).max()) <= FP32_REL
    ids, _ = gpu.generate(16)
    cur = seqs
    for s in range(16):
        nxt = oracle.argmax(p).astype(np.int32)
        assert np.array_equal(nxt, ids[s]), "step %d" % s
        cur = np.concatenate([cur, nxt[:, None]], 1)
        p, lg = orc.step(cur, use_cache=True)
    assert float(np.abs(gpu.logits() - lg).max() / np.abs(lg).max()) <= FP32_REL
    gpu.close()


def test_cfg1_fp16_full_width(G, oracle):
    """Configuration 1's fp16 variant at full width, 4 layers, batch 8, prompt 96 (768 prompt rows: the LDS-tiled GEMMs)."""
    cfg = dict(synth.CONFIGS["cfg1_gpt2small_f16"], n_layers=4, prompt=96)
    _, gpu, out, _ = teacher_forced(G, oracle, cfg, 3, 4)
    check_fp16(out)
    gpu.close()


@pytest.mark.parametrize("kw", [dict(), dict(hidden=128, n_heads=2, n_kv_heads=2, ffn_dim=320), dict(act=synth.SWIGLU, attn_type=synth.GQA, n_kv_heads=2)])
def test_deferred_layernorm_with_a_large_row_mean(G, oracle, kw):
    """fp16 LayerNorm models take the five-launch decode step: the producers of the residual stream store half(gamma x) and
    the tiles' sums of x and x^2, the consumers rebuild mean and 1 / sigma and take the mean's share out of their products
    (folded constants c, d per output column).  Here every embedding carries an offset of about twice its spread and gamma,
    beta and the biases are random, so that a wrong mean term, a dropped beta or a transposed fold would move the logits far
    beyond the bar; the generate loop (sampling kernel + embedding in one launch) must give the step-wise tokens."""
    cfg = synth.tiny_config(dtype="f16", norm_type=synth.LAYERNORM, **{**dict(attn_type=synth.MHA, n_kv_heads=4, act=synth.RELU), **kw})
    w = synth.make_weights(cfg, 21, random_bias=True)
    rng = np.random.default_rng(5)
    w = {k: np.array(v, np.float32) for k, v in w.items()}
    w["TgtEmbeddings"] = w["TgtEmbeddings"] + np.float32(0.04)
    for k in w:
        if k.endswith("m_alpha"):
            w[k] = (1.0 + 0.3 * rng.standard_normal(w[k].shape)).astype(np.float32)
        elif k.endswith("m_beta"):
            w[k] = (0.2 * rng.standard_normal(w[k].shape)).astype(np.float32)
    orc = oracle.OracleGpt(cfg, w)
    gpu = G.HipGpt(cfg, w, max_batch=cfg["batch"], max_seq_len=cfg["prompt"] + 12)
    seqs = synth.make_prompts(cfg, 3)
    p, lg = orc.step(seqs, use_cache=True)
    gpu.prefill(seqs)
    assert np.abs(gpu.logits() - lg).max() <= FP16_ABS
    cur, agree = seqs, []
    for _ in range(5):
        nxt = oracle.argmax(p).astype(np.int32)
        cur = np.concatenate([cur, nxt[:, None]], 1)
        p, lg = orc.step(cur, use_cache=True)
        gpu.decode(nxt)
        gl = gpu.logits()
        assert np.abs(gl - lg).max() <= FP16_ABS
        agree.append(top1_agreement(gl, lg)[0])
    hid = gpu.hidden()
    assert np.isfinite(hid).all()
    assert np.mean(agree) >= 0.99
    # the graph-captured loop against step-by-step decoding from the same state
    gpu.reset()
    gpu.prefill(seqs)
    ids, _ = gpu.generate(4)
    gpu.reset()
    gpu.prefill(seqs)
    for s in range(4):
        nxt = gpu.sample()
        assert np.array_equal(nxt, ids[s])
        gpu.decode(nxt)
    gpu.close()


@pytest.mark.parametrize("dtype", ["f32", "f16"])
def test_cfg3_moe_layer_shape(G, oracle, dtype):
    """Configuration 3's layer shape: hidden 1024, 16 / 4 heads, 8 experts of width 4096 with 2 per token, batch 64, at
    three layers (layers 0-1 dense, layer 2 MoE) with a short prompt and a small vocabulary.  fp32 model: routing indices
    bit-exact and logits within 1e-4.  fp16 model: the router sees activations that differ from the oracle's by the fp16
    path's rounding, so a token whose k-th and (k+1)-th expert probabilities are closer than that can be routed to the
    other expert; such rows (few, and only with a margin below 2e-3 in the oracle's own probabilities) are checked for
    that margin instead of the logit bar, every other row meets the fp16 bars.  The margin: the reference adds -65000 to the
    router's logits (MoEFeedForward.cs:83), which rounds them to multiples of 2^-8, the float32 spacing there; an input
    difference far below one such step can move a logit across a rounding boundary, by one step.  The choice may differ from
    the oracle's only where the oracle's own two logits are one step (2^-8) apart or tied (measured here: 1 row of 256,
    at exactly one step).  The logit gap is the log of the probability ratio."""
    cfg = dict(synth.CONFIGS["cfg3_moe_f16"], n_layers=3, vocab=2048, prompt=6, dtype=dtype)
    B, k = cfg["batch"], cfg["experts_per_token"]
    w = synth.make_weights(cfg, 5, random_bias=True)
    orc = oracle.OracleGpt(cfg, w)
    gpu = G.HipGpt(cfg, w, max_batch=B, max_seq_len=cfg["prompt"] + 6)
    cur = synth.make_prompts(cfg, 105)
    gpu.prefill(cur)
    hit = set()
    agree, flipped, worst_gap = [], 0, 0.0
    for step in range(4):
        p, lg = orc.step(cur, use_cache=True)
        gl = gpu.logits()
        ti, tv, pr = gpu.moe_routing(2)                     # the only MoE layer: last position of every sequence
        oi, ov, op = orc.moe_trace(0)                        # all rows the oracle's step fed: the whole prompt at step 0
        if step == 0:
            last = cfg["prompt"] * (np.arange(B) + 1) - 1
            oi, ov, op = oi[last], ov[last], op[last]
        hit |= set(np.unique(oi).astype(int))
        if dtype == "f32":
            assert np.array_equal(ti, oi)
            assert np.allclose(tv, ov, rtol=1e-6) and np.allclose(pr, op, rtol=1e-6)
            assert float(np.abs(gl - lg).max() / np.abs(lg).max()) <= FP32_REL
            assert np.array_equal(gl.argmax(1), lg.argmax(1))
        else:
            same = np.array([set(ti[r]) == set(oi[r]) for r in range(B)])
            srt = -np.sort(-op, axis=1)
            # the oracle's own gap between the last expert in and the first out, in steps of the -65000 quantisation
            gap_steps = (np.log(srt[:, k - 1].astype(np.float64)) - np.log(srt[:, k].astype(np.float64))) / 2.0 ** -8
            assert (gap_steps[~same] <= 1.0 + 0.05).all(), gap_steps[~same]
            flipped += int((~same).sum())
            worst_gap = max(worst_gap, float(gap_steps[~same].max()) if (~same).any() else 0.0)
            assert np.abs(gl[same] - lg[same]).max() <= FP16_ABS
            assert np.abs(pr - op).max() <= 2e-3
            agree.append(top1_agreement(gl[same], lg[same])[0])
        nxt = oracle.argmax(p).astype(np.int32)
        cur = np.concatenate([cur, nxt[:, None]], 1)
        gpu.decode(nxt)
    assert hit == set(range(8))                             # every expert is hit at batch 64
    if dtype == "f16":
        print("fp16 MoE routing at cfg3's layer shape: %d of %d rows routed differently from the fp32 oracle, largest oracle gap among them %.2f steps of 2^-8"
              % (flipped, 4 * B, worst_gap))
        assert np.mean(agree) >= 0.99 and flipped <= 0.05 * 4 * B
    gpu.close()


def test_cfg4_layer_shape_against_oracle(G, oracle):
    """Configuration 4's layer shape: hidden 4096, 32 / 8 heads of 128, FFN 11008 gated, RMSNorm, batch 16, at two
    layers with a short prompt: 16-row partial tiles, three column tiles per block in the FFN up projection (688 tiles)."""
    cfg = dict(synth.CONFIGS["cfg4_7b_longctx_f16"], n_layers=2, vocab=2048, prompt=40)
    _, gpu, out, _ = teacher_forced(G, oracle, cfg, 7, 3)
    check_fp16(out)
    gpu.close()


def test_cfg4_long_context_properties(G):
    """Configuration 4 at its real context (batch 16, prompt 8192, two layers): prefill(P) + decode(3) must reproduce
    prefill(P + 3); generate() equals step-by-step decoding.  At this length the decode attention splits a (row, head)
    pair over several blocks by itself and the rotary table is read beyond position 8192."""
    cfg = dict(synth.CONFIGS["cfg4_7b_longctx_f16"], n_layers=2, vocab=4096)
    B, Tp = cfg["batch"], cfg["prompt"]
    w = synth.make_weights(cfg, 0)
    seqs = synth.make_prompts(cfg, 1, length=Tp + 3)
    a = G.HipGpt(cfg, w, max_batch=B, max_seq_len=Tp + 16)
    a.prefill(seqs[:, :Tp])
    for t in range(Tp, Tp + 3):
        a.decode(seqs[:, t])
    la = a.logits()
    assert a.seq_len() == Tp + 3
    b = G.HipGpt(cfg, w, max_batch=B, max_seq_len=Tp + 16)
    b.prefill(seqs)
    lb = b.logits()
    assert np.abs(la - lb).max() <= FP16_ABS
    assert top1_agreement(la, lb)[0] >= 0.99
    for which in (0, 1):
        ka, kb = a.get_kv(1, which), b.get_kv(1, which)
        assert ka.shape == (B, cfg["n_kv_heads"], Tp + 3, 128)
        assert np.abs(ka - kb).max() <= 2e-2
    del ka, kb
    b.close()
    g1, _ = a.generate(4)
    a.set_seq_len(B, Tp + 2)
    a.decode(seqs[:, Tp + 2])
    assert np.array_equal(a.logits(), la)
    steps = []
    for _ in range(4):
        nxt = a.sample()
        steps.append(nxt)
        a.decode(nxt)
    assert np.array_equal(g1, np.stack(steps))
    a.close()


@pytest.mark.parametrize("hidden,heads,kv_heads,batch", [(512, 4, 1, 2), (256, 4, 2, 3)])
def test_decode_across_position_8192_against_oracle(G, oracle, hidden, heads, kv_heads, batch):
    """A narrow one-layer model with a cache of 8190 random positions installed on both sides: decode steps at positions
    8190 .. 8194 against the oracle (rotary angles at m > 8000, split attention chosen by the library itself, the
    appended rows landing in the last chunks of a long cache).  head_dim 128 and 64."""
    T0 = 8190
    cfg = synth.tiny_config(dtype="f16", n_layers=1, hidden=hidden, n_heads=heads, n_kv_heads=kv_heads, ffn_dim=2 * hidden, vocab=300,
                            batch=batch, prompt=T0)
    d = hidden // heads
    w = synth.make_weights(cfg, 3, random_bias=True)
    for k in list(w):                                        # widen Q and K so that the scores are far from uniform
        if k.endswith((".Q", ".K")):
            w[k] = (w[k] * np.float32(8.0)).astype(np.float16).astype(np.float32)
    rng = np.random.default_rng(9)
    keys = rng.standard_normal((batch, kv_heads, T0, d)).astype(np.float16).astype(np.float32)
    vals = rng.standard_normal((batch, kv_heads, T0, d)).astype(np.float16).astype(np.float32)
    orc = oracle.OracleGpt(cfg, w)
    g = heads // kv_heads
    # the reference keeps keys as [B*H, d, T] and values as [B*H, T, d], heads expanded
    orc.set_cache(0, 0, np.ascontiguousarray(np.repeat(keys, g, axis=1).transpose(0, 1, 3, 2)).reshape(batch * heads, d, T0), batch * heads, T0, d)
    orc.set_cache(0, 1, np.ascontiguousarray(np.repeat(vals, g, axis=1)).reshape(batch * heads, T0, d), batch * heads, T0, d)
    gpu = G.HipGpt(cfg, w, max_batch=batch, max_seq_len=T0 + 8)
    gpu.set_kv(0, 0, keys)
    gpu.set_kv(0, 1, vals)
    gpu.set_seq_len(batch, T0)
    toks = synth.make_prompts(cfg, 4, length=6)
    cur = np.zeros((batch, T0), np.int32)                    # (only the last token of a row is read when a cache exists)
    for s in range(5):
        cur = np.concatenate([cur, toks[:, s:s + 1]], 1)
        _, lg = orc.step(cur, use_cache=True)
        gpu.decode(toks[:, s])
        gl = gpu.logits()
        assert np.abs(gl - lg).max() <= FP16_ABS, "position %d" % (T0 + s)
    assert gpu.seq_len() == T0 + 5 == orc.cache_len()
    kg = gpu.get_kv(0, 0)[:, :, T0:]
    ko = orc.get_cache(0, 0).reshape(batch, heads, d, T0 + 5)[:, ::g, :, T0:].transpose(0, 1, 3, 2)
    assert np.abs(kg - ko).max() <= 2e-2                     # appended keys: rotated at positions beyond 8190
    gpu.close()


@pytest.mark.parametrize("max_batch,batch", [(48, 48), (100, 100), (100, 37)])
def test_dense_fp16_rmsnorm_batches_above_32(G, oracle, max_batch, batch):
    """The deferred-norm decode path with two and four 32-row tiles per block (max_batch 33-64 and 65-128), including a
    batch that leaves the last tiles partly or wholly empty."""
    cfg = synth.tiny_config(dtype="f16", hidden=256, n_heads=4, n_kv_heads=2, ffn_dim=512, vocab=300, batch=batch, prompt=7)
    _, gpu, out, _ = teacher_forced(G, oracle, cfg, 11, 3, max_batch=max_batch)
    check_fp16(out)
    gpu.close()


def test_wide_model_more_than_eight_qkv_splits(G, oracle):
    """hidden 4608 at max_batch 70: the QKV projection's K is split nine ways, one more than the attention prologue keeps
    in registers."""
    cfg = synth.tiny_config(dtype="f16", n_layers=1, hidden=4608, n_heads=36, n_kv_heads=9, ffn_dim=256, vocab=300, batch=70, prompt=3)
    _, gpu, out, _ = teacher_forced(G, oracle, cfg, 13, 2)
    check_fp16(out)
    gpu.close()


def test_cfg3_full_depth_graph_replay_equals_stepwise(G):
    """Configuration 3 at its full depth (12 layers, 10 of them MoE) and batch: the captured step graph (router with the
    counter-based places, expert GEMMs over the pointer tables, combine) gives the tokens and the logits of explicit
    decode calls, and a second model object repeats them bit for bit -- the places rows take in their experts' batches
    differ from run to run, the results must not."""
    cfg = dict(synth.CONFIGS["cfg3_moe_f16"], vocab=4096, prompt=24)
    B = cfg["batch"]
    w = synth.make_weights(cfg, 21, random_bias=True)
    ids = synth.make_prompts(cfg, 4)
    runs = []
    for rep in range(2):
        gpu = G.HipGpt(cfg, w, max_batch=B, max_seq_len=cfg["prompt"] + 12)
        gpu.prefill(ids)
        toks, _ = gpu.generate(6)
        runs.append((toks, gpu.logits()))
        gpu.close()
    assert np.array_equal(runs[0][0], runs[1][0]) and np.array_equal(runs[0][1], runs[1][1])
    step = G.HipGpt(cfg, w, max_batch=B, max_seq_len=cfg["prompt"] + 12)
    step.prefill(ids)
    for s in range(6):
        nxt = step.sample()
        assert np.array_equal(nxt, runs[0][0][s])
        step.decode(nxt)
    assert np.array_equal(step.logits(), runs[0][1])
    ti, tv, pr = step.moe_routing(5)
    assert ti.shape == (B, cfg["experts_per_token"]) and np.allclose(pr.sum(1), 1.0, atol=1e-5)
    step.close()


@pytest.mark.parametrize("batch,prompt,hidden,heads,kv,ffn,act", [
    (3, 200, 192, 3, 3, 256, synth.SWIGLU),        # 600 rows: partial 256-row tiles; 6 and 8 column tiles (partial groups of four)
    (2, 300, 256, 4, 2, 264, synth.SWIGLU_SILU),   # odd number of k-tiles in the down projection (the register-staged kernel)
    (5, 128, 512, 8, 2, 1024, synth.SWIGLU),       # 640 rows, whole 64-row blocks, whole groups of four column tiles (line stores)
    (9, 64, 128, 2, 1, 512, synth.RELU),           # 576 rows, ungated activation
])
def test_prefill_tile_edges_against_oracle(G, oracle, batch, prompt, hidden, heads, kv, ffn, act):
    """Prompts of 512 rows and more take the LDS-tiled prefill GEMMs, whose epilogues write whole 64 x 128-byte blocks
    through LDS where a wavefront's block is complete and element-wise elsewhere: row counts that are no multiple of
    the tile sizes and widths that leave partial column groups, against the oracle."""
    cfg = synth._cfg(n_layers=2, hidden=hidden, n_heads=heads, n_kv_heads=kv, ffn_dim=ffn, vocab=211, attn_type=synth.GQA,
                     norm_type=synth.RMSNORM, act=act, batch=batch, prompt=prompt, steps=2, dtype="f16")
    _, gpu, out, _ = teacher_forced(G, oracle, cfg, 31, 2)
    check_fp16(out)
    gpu.close()


@pytest.mark.parametrize("dtype,hidden,heads,kv,batch,prompt", [
    ("f16", 512, 8, 1, 5, 70),        # head size 64, eight query heads on one KV head: the MFMA attention kernels
    ("f16", 1024, 8, 1, 33, 40),      # head size 128
    ("f16", 1024, 16, 2, 3, 530),     # two KV heads; 530 rows of prompt take the LDS-tiled prefill GEMMs
    ("f32", 256, 8, 1, 4, 37),        # the fp32 (VALU) attention kernels
    ("f16", 256, 8, 1, 2, 33),        # head size 32: VALU kernels on an fp16 cache
])
def test_eight_query_heads_per_kv_head(G, oracle, dtype, hidden, heads, kv, batch, prompt):
    """Group size 8 (Llama-3-70B-like head layouts), prefill and decode, both cache layouts."""
    cfg = synth._cfg(n_layers=2, hidden=hidden, n_heads=heads, n_kv_heads=kv, ffn_dim=2 * hidden, vocab=173, attn_type=synth.GQA,
                     norm_type=synth.RMSNORM, act=synth.SWIGLU, batch=batch, prompt=prompt, steps=3, dtype=dtype)
    _, gpu, out, _ = teacher_forced(G, oracle, cfg, 41, 3)
    if dtype == "f16":
        check_fp16(out)
    else:
        for lg, gl in out:
            assert float(np.abs(gl - lg).max() / np.abs(lg).max()) <= FP32_REL
    gpu.close()


@pytest.mark.parametrize("hidden,heads,kv,batch,prompt", [
    (512, 8, 2, 5, 128),       # head size 64, 640 rows: the last 256-row tile holds one 64-row block and a half
    (1024, 8, 2, 3, 192),      # head size 128: a wavefront's 128 columns are one head, written in two passes
    (512, 8, 4, 1, 544),       # one sequence of 17 chunks: the last wavefront's second chunk lies beyond the rows
])
def test_projection_writes_the_cache_like_the_separate_kernel(G, oracle, monkeypatch, hidden, heads, kv, batch, prompt):
    """From 512 rows on, with whole 32-position chunks, the QKV projection's epilogue rotates the keys and writes keys and
    values into the fragment-major cache itself.  Same cache contents and logits as with the separate cache-write kernel
    (TSHIP_NO_KV_FUSE=1), and the cache against the oracle's keys and values."""
    cfg = synth._cfg(n_layers=2, hidden=hidden, n_heads=heads, n_kv_heads=kv, ffn_dim=2 * hidden, vocab=157, attn_type=synth.GQA,
                     norm_type=synth.RMSNORM, act=synth.SWIGLU, batch=batch, prompt=prompt, steps=2, dtype="f16")
    w = synth.make_weights(cfg, 77, random_bias=True)
    seqs = synth.make_prompts(cfg, 78)
    gpu = G.HipGpt(cfg, w, max_batch=batch, max_seq_len=prompt + 136)
    gpu.prefill(seqs)
    fused = [(gpu.get_kv(l, 0), gpu.get_kv(l, 1)) for l in range(2)]
    lg_fused = gpu.logits()
    monkeypatch.setenv("TSHIP_NO_KV_FUSE", "1")
    gpu.reset()
    gpu.prefill(seqs)
    monkeypatch.delenv("TSHIP_NO_KV_FUSE")
    for l in range(2):
        k, v = gpu.get_kv(l, 0), gpu.get_kv(l, 1)
        assert np.array_equal(fused[l][0], k), "keys of layer %d" % l
        assert np.array_equal(fused[l][1], v), "values of layer %d" % l
    assert np.array_equal(lg_fused, gpu.logits())
    # appended tokens behind the fused prefill continue the same cache: 128 more per sequence (with three or five sequences
    # again 512 rows or more, written by the projection at a cache offset; with one sequence by the separate kernel)
    more = synth.make_prompts(dict(cfg, prompt=128), 79)
    gpu.reset()
    gpu.prefill(seqs)
    gpu.prefill(more)
    lg_app = gpu.logits()
    k_app = gpu.get_kv(1, 0)
    orc = oracle.OracleGpt(cfg, w)
    _, lg = orc.step(np.concatenate([seqs, more], 1), use_cache=True)
    assert np.abs(lg_app - lg).max() <= FP16_ABS
    monkeypatch.setenv("TSHIP_NO_KV_FUSE", "1")
    gpu.reset()
    gpu.prefill(seqs)
    gpu.prefill(more)
    monkeypatch.delenv("TSHIP_NO_KV_FUSE")
    assert np.array_equal(lg_app, gpu.logits()) and np.array_equal(k_app, gpu.get_kv(1, 0))
    gpu.close()


@pytest.mark.parametrize("patch_rows", ["1", "2", "4", "8"])
def test_prefill_tile_patch_heights_give_the_same_bits(G, monkeypatch, patch_rows):
    """The LDS-tiled prefill GEMM maps its blocks to tiles in patches of (8, 4, 2 or 1) x 4 tiles per XCD, chosen from the
    launch size; the mapping must not change any result.  1536 rows x 512 columns: 6 x 2 tiles, fewer than eight patches at
    every height, against the height the launch code picks."""
    cfg = synth._cfg(n_layers=2, hidden=512, n_heads=8, n_kv_heads=2, ffn_dim=1024, vocab=157, attn_type=synth.GQA,
                     norm_type=synth.RMSNORM, act=synth.SWIGLU, batch=3, prompt=512, steps=1, dtype="f16")
    w = synth.make_weights(cfg, 91, random_bias=True)
    seqs = synth.make_prompts(cfg, 92)
    gpu = G.HipGpt(cfg, w, max_batch=3, max_seq_len=520)
    gpu.prefill(seqs)
    want = gpu.logits()
    monkeypatch.setenv("TSHIP_PATCH_ROWS", patch_rows)
    gpu.reset()
    gpu.prefill(seqs)
    monkeypatch.delenv("TSHIP_PATCH_ROWS")
    assert np.array_equal(want, gpu.logits())
    gpu.close()


@pytest.mark.parametrize("head_dim", [64, 128])
def test_prefill_attention_column_groups_agree(G, monkeypatch, head_dim):
    """The prefill attention gives a wavefront one or two groups of 16 MFMA columns (4 or 8 query positions at four query
    heads per KV head), chosen from the head size and the launch size.  The grouping changes which chunks move a column's
    reference, hence the rounding, not the result: logits and the second layer's cache must agree within the fp16 bar,
    for a plain and for a padded batch, and large scores (which move the reference often) must not overflow."""
    cfg = synth._cfg(n_layers=2, hidden=8 * head_dim, n_heads=8, n_kv_heads=2, ffn_dim=1024, vocab=157, attn_type=synth.GQA,
                     norm_type=synth.RMSNORM, act=synth.SWIGLU, batch=3, prompt=200, steps=1, dtype="f16")
    w = synth.make_weights(cfg, 93, random_bias=True)
    for name in w:
        if name.endswith(".Q") or name.endswith(".K"):
            w[name] = w[name] * 6.0          # peaked attention: scores far apart, so that the reference moves often
    seqs = synth.make_prompts(cfg, 94)
    lens = np.array([200, 37, 129], np.int32)
    out = {}
    for nq in ("1", "2"):
        monkeypatch.setenv("TSHIP_ATTN_NQ", nq)
        for padded in (False, True):
            gpu = G.HipGpt(cfg, w, max_batch=3, max_seq_len=224)
            gpu.prefill(seqs, lens if padded else None)
            out[nq, padded] = (gpu.logits(), gpu.get_kv(1, 0), gpu.get_kv(1, 1))
            gpu.close()
    monkeypatch.delenv("TSHIP_ATTN_NQ")
    for padded in (False, True):
        for a, b in zip(out["1", padded], out["2", padded]):
            assert np.isfinite(a).all() and np.isfinite(b).all()
            assert np.abs(a - b).max() <= FP16_ABS


def test_full_size_prefill_repeats_bit_for_bit(G):
    """The benchmark configuration's prefill (16 layers, 32 x 1024 tokens, 8192 attention blocks per layer) six times on
    one model: finite and the same bits every time.  The prefill kernels hand data between wavefronts through LDS under
    hand-counted waits; a wait that is one short shows as a row that differs in some launches, not in all."""
    cfg = dict(synth.CONFIGS["cfg2_1b_gqa_f16"])
    B, Tp, last = cfg["batch"], cfg["prompt"], cfg["n_layers"] - 1
    w = synth.make_weights(cfg, 0)
    seqs = synth.make_prompts(cfg, 1, length=Tp)
    gpu = G.HipGpt(cfg, w, max_batch=B, max_seq_len=Tp + 16)
    first = None
    for _ in range(6):
        gpu.reset()
        gpu.prefill(seqs)
        cur = (gpu.logits().copy(), gpu.get_kv(last, 0).copy(), gpu.get_kv(last, 1).copy())
        assert all(np.isfinite(x).all() for x in cur)
        if first is None:
            first = cur
        else:
            assert all(np.array_equal(a, b) for a, b in zip(first, cur))
    gpu.close()
