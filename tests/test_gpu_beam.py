"""Beam search and sentence scores through the fused path (TSHip_GptBeamPick / TSHip_GptReorderRows / TSHip_BeamTopN and
the loop in seq2seqsharp_amd.gpt.HipGpt.beam_search) against the oracle's restatement of the reference's loop, which
recomputes every hypothesis without a KV cache (GPT.cs:238-241, 264-302; Decoder.cs:756-792)."""
import numpy as np
import pytest

from seq2seqsharp_amd import synth

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def G():
    from seq2seqsharp_amd import gpt
    return gpt


def _sharp(cfg, seed):
    """Weights with a head wide enough that the probabilities are far from uniform (scores of hypotheses then differ by much
    more than fp32 noise, so that pruning cannot flip on rounding)."""
    w = synth.make_weights(cfg, seed, random_bias=True)
    w["FeedForward_Decoder_0.m_Whd"] = (w["FeedForward_Decoder_0.m_Whd"] * np.float32(40.0)).astype(np.float32)
    return w


@pytest.mark.parametrize("beam,kw", [(3, dict()), (4, dict(attn_type=synth.MHA, n_kv_heads=4, norm_type=synth.LAYERNORM, act=synth.RELU)), (2, dict(batch=3)),
                                     (3, dict(hidden=160, n_heads=10, n_kv_heads=1))])      # ten heads on one KV head: two groups of five
def test_greedy_beam_search_matches_the_reference_loop(G, oracle, beam, kw):
    cfg = synth.tiny_config(prompt=5, vocab=61, **kw)
    w = _sharp(cfg, 3)
    B = cfg["batch"]
    prompts = synth.make_prompts(cfg, 4)
    gpu = G.HipGpt(cfg, w, max_batch=B * beam, max_seq_len=32)
    hyp, sc = gpu.beam_search(prompts, beam, max_len=5 + 7)
    orc = oracle.OracleGpt(cfg, w)
    ohyp, osc = oracle.gpt_beam_search(orc, prompts, beam, max_len=5 + 7)
    assert hyp == ohyp
    assert np.allclose(np.array(sc), np.array(osc), rtol=1e-5, atol=1e-5)
    # hypotheses of one sequence are distinct and the best one leads (the queue's better half has its best at the root)
    for b in range(B):
        assert len({tuple(h) for h in hyp[b]}) == beam
        assert sc[b][0] == min(sc[b])
    gpu.close()


def test_top_p_beam_search_with_repeat_penalty(G, oracle):
    cfg = synth.tiny_config(prompt=6, vocab=80, batch=2)
    w = _sharp(cfg, 5)
    prompts = synth.make_prompts(cfg, 6)
    prompts[:, 2] = prompts[:, 0]
    beam, steps = 3, 5
    u = np.random.default_rng(7).random((steps, beam, beam * 2), dtype=np.float32)
    gpu = G.HipGpt(cfg, w, max_batch=2 * beam, max_seq_len=32)
    gpu.set_repeat_penalty(2.0)
    hyp, sc = gpu.beam_search(prompts, beam, max_len=6 + steps, mode=G.TOPP, top_p=0.9, uniforms=u)
    orc = oracle.OracleGpt(cfg, w)
    ohyp, osc = oracle.gpt_beam_search(orc, prompts, beam, max_len=6 + steps, top_p=0.9, repeat_penalty=2.0, uniforms=u)
    assert hyp == ohyp
    assert np.allclose(np.array(sc), np.array(osc), rtol=1e-5, atol=1e-5)
    gpu.close()


def test_beam_search_stops_when_every_hypothesis_ends(G, oracle):
    cfg = synth.tiny_config(prompt=4, vocab=9, batch=2)
    w = _sharp(cfg, 8)
    w["FeedForward_Decoder_0.m_Bd"] = w["FeedForward_Decoder_0.m_Bd"].copy()
    w["FeedForward_Decoder_0.m_Bd"][0, 0] = 30.0             # the END tag wins everywhere: all hypotheses end at once
    prompts = synth.make_prompts(cfg, 9)
    gpu = G.HipGpt(cfg, w, max_batch=4, max_seq_len=32)
    orc = oracle.OracleGpt(cfg, w)
    # one hypothesis per sequence: its first pick is the END tag, the loop ends after one step
    hyp, sc = gpu.beam_search(prompts, 1, max_len=20, eos_id=0)
    ohyp, osc = oracle.gpt_beam_search(orc, prompts, 1, max_len=20, eos_id=0)
    assert hyp == ohyp and all(len(h[0]) == 5 and h[0][-1] == 0 for h in hyp)
    assert np.allclose(np.array(sc), np.array(osc), rtol=1e-5, atol=1e-5)
    # two hypotheses: the second pick of a step is never the END tag, so some hypothesis may stay open; same loop either way
    hyp, sc = gpu.beam_search(prompts, 2, max_len=12, eos_id=0)
    ohyp, osc = oracle.gpt_beam_search(orc, prompts, 2, max_len=12, eos_id=0)
    assert hyp == ohyp
    gpu.close()


def test_pick_scores_and_row_gather(G, oracle):
    """One pick = the greedy token with its log probability (the sentence score of a beam-size-1 run); rows gathered with
    repeats continue their parents exactly."""
    cfg = synth.tiny_config(prompt=7, vocab=120, batch=3, dtype="f16", hidden=256, n_heads=4, n_kv_heads=2, ffn_dim=512)
    w = synth.make_weights(cfg, 11, random_bias=True)
    prompts = synth.make_prompts(cfg, 12)
    gpu = G.HipGpt(cfg, w, max_batch=6, max_seq_len=48)
    gpu.prefill(prompts)
    lg = gpu.logits().astype(np.float64)
    lp = lg - lg.max(1, keepdims=True)
    lp = lp - np.log(np.exp(lp).sum(1, keepdims=True))
    ids, logp = gpu.beam_pick(2)
    assert np.array_equal(ids[0], gpu.sample())
    assert np.allclose(logp[0], lp[np.arange(3), ids[0]], atol=1e-5)
    second = np.argsort(-lg, axis=1)[:, 1]
    assert np.array_equal(ids[1], second) and np.allclose(logp[1], lp[np.arange(3), second], atol=1e-5)
    # rows 0,0,2,1,1,2 continue with different tokens; each must equal a fresh model fed the same sequence
    src = np.array([0, 0, 2, 1, 1, 2], np.int32)
    toks = np.array([5, 9, 11, 5, 17, 11], np.int32)
    gpu.reorder_rows(src)
    gpu.decode(toks)
    got = gpu.logits()
    k_got = gpu.get_kv(1, 0)
    ref = G.HipGpt(cfg, w, max_batch=6, max_seq_len=48)
    ref.prefill(np.concatenate([prompts[src], toks[:, None]], 1))
    want = ref.logits()
    assert np.abs(got - want).max() <= 2e-2
    assert np.abs(k_got - ref.get_kv(1, 0)).max() <= 2e-2
    assert np.array_equal(got[2], got[5])                    # identical parents and tokens: identical rows
    gpu.close()
    ref.close()
