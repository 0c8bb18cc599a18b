"""Batches of sequences of different lengths through the fused path, as the reference runs them when padding is allowed
(Decoder.cs:656 PadSentences, :687-690 BuildSelfTriMask): padded with the END tag to the longest, masked per row, logits
read at every row's last padded position, decoding continued on the padded sequences.  Against the oracle's restatement
of that branch (pinned on the CPU by tests/test_oracle_layers_numpy.py)."""
import numpy as np
import pytest

from parity_util import top1_agreement
from seq2seqsharp_amd import synth

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def G():
    from seq2seqsharp_amd import gpt
    return gpt


def _run(G, oracle, cfg, lens, seed, steps=3):
    w = synth.make_weights(cfg, seed, random_bias=True)
    for k in list(w):                                        # widen Q and K: attention far from uniform, so that a wrong mask shows
        if k.endswith((".Q", ".K", ".QKV")):
            w[k] = (w[k] * np.float32(6.0)).astype(np.float16 if cfg["dtype"] == "f16" else np.float32).astype(np.float32)
    rng = np.random.default_rng(seed)
    seqs = [list(rng.integers(4, cfg["vocab"], size=int(n))) for n in lens]
    ids, ln = G.HipGpt.pad_sentences(seqs, pad_id=0)
    assert np.array_equal(ln, lens)
    orc = oracle.OracleGpt(cfg, w)
    gpu = G.HipGpt(cfg, w, max_batch=len(lens), max_seq_len=ids.shape[1] + steps + 2)
    p, lg = orc.step(ids, use_cache=True, lens=lens.astype(np.float32))
    gpu.prefill(ids, lens=lens)
    out = [(lg, gpu.logits())]
    cur = ids
    for _ in range(steps):
        nxt = oracle.argmax(p).astype(np.int32)
        cur = np.concatenate([cur, nxt[:, None]], 1)
        p, lg = orc.step(cur, use_cache=True)
        gpu.decode(nxt)
        out.append((lg, gpu.logits()))
    assert gpu.seq_len() == ids.shape[1] + steps == orc.cache_len()
    return orc, gpu, out, ids


@pytest.mark.parametrize("kw", [dict(), dict(attn_type=synth.MHA, n_kv_heads=4, norm_type=synth.LAYERNORM, act=synth.RELU)])
def test_padded_batch_fp32(G, oracle, kw):
    cfg = synth.tiny_config(batch=4, **kw)
    lens = np.array([5, 8, 1, 8], np.int32)
    orc, gpu, out, ids = _run(G, oracle, cfg, lens, 7)
    for lg, gl in out:
        assert float(np.abs(gl - lg).max() / np.abs(lg).max()) <= 1e-4
        assert np.array_equal(gl.argmax(1), lg.argmax(1))
    # the masking matters on this input: a plain causal prefill of the same padded ids differs on the short rows only
    gpu.reset()
    gpu.prefill(ids)
    plain = gpu.logits()
    padded = out[0][1]
    gpu.reset()
    gpu.prefill(ids, lens=lens)
    assert np.array_equal(gpu.logits(), padded)
    assert np.abs(plain[[1, 3]] - padded[[1, 3]]).max() <= 1e-5 * np.abs(padded).max()
    assert np.abs(plain[[0, 2]] - padded[[0, 2]]).max() > 1e-3 * np.abs(padded).max()
    gpu.close()


@pytest.mark.parametrize("hidden,heads,kv_heads,lens", [(256, 4, 2, [70, 33, 1, 64, 2]), (512, 4, 1, [40, 9, 31]), (256, 4, 4, [130, 129, 5, 64]),
                                                        # 9 x 64 = 576 padded rows in whole 32-position chunks: the LDS-tiled GEMMs, and the QKV
                                                        # projection writes the cache (padding positions included) from its epilogue
                                                        (512, 8, 4, [64, 17, 1, 33, 64, 50, 2, 31, 48]), (512, 4, 2, [64, 3, 40, 64, 20, 9, 33, 1, 60])])
def test_padded_batch_fp16_mfma_attention(G, oracle, hidden, heads, kv_heads, lens):
    """head_dim 64 and 128 (the MFMA prefill attention): lengths on both sides of 32-position chunk boundaries, a row of
    length 1, rows of full length."""
    lens = np.array(lens, np.int32)
    cfg = synth.tiny_config(dtype="f16", hidden=hidden, n_heads=heads, n_kv_heads=kv_heads, ffn_dim=2 * hidden, vocab=300, batch=len(lens))
    orc, gpu, out, ids = _run(G, oracle, cfg, lens, 9)
    fr = []
    for lg, gl in out:
        assert np.abs(gl - lg).max() <= 3e-2
        fr.append(top1_agreement(gl, lg)[0])
    assert np.mean(fr) >= 0.99
    # cached keys of the padded positions too (they stay visible to every later step)
    H, d = heads, hidden // heads
    T = gpu.seq_len()
    last = cfg["n_layers"] - 1
    ko = orc.get_cache(last, 0).reshape(len(lens), H, d, T)[:, ::H // kv_heads].transpose(0, 1, 3, 2)
    assert np.abs(gpu.get_kv(last, 0) - ko).max() <= 2e-2
    gpu.close()


def test_padded_prefill_argument_errors(G):
    from seq2seqsharp_amd._lib import TSHipError
    cfg = synth.tiny_config(batch=2)
    gpu = G.HipGpt(cfg, synth.make_weights(cfg, 0), max_batch=2, max_seq_len=24)
    ids = synth.make_prompts(cfg, 1)
    with pytest.raises(TSHipError, match="length"):
        gpu.prefill(ids, lens=np.array([3, ids.shape[1] + 1], np.int32))
    gpu.prefill(ids)
    with pytest.raises(TSHipError, match="Reset"):
        gpu.prefill(ids, lens=np.array([3, 4], np.int32))
    gpu.close()
