"""Features of the fused path in combination, each checked against another route through the library that must give the
same answer bit for bit (the single features are checked against the oracle elsewhere): padded prompts, MoE layers, the
captured step graph, top-p with the repeat penalty, appended prefills and beam reordering."""
import numpy as np
import pytest

from seq2seqsharp_amd import synth

pytestmark = pytest.mark.gpu


def _moe_cfg(dtype):
    return synth.tiny_config(dtype=dtype, n_layers=3, hidden=128, n_heads=4, n_kv_heads=2, ffn_dim=256, vocab=211, n_experts=4, experts_per_token=2,
                             norm_type=synth.LAYERNORM, act=synth.RELU, batch=5, prompt=12)


@pytest.mark.parametrize("dtype", ["f32", "f16"])
def test_padded_moe_model_graph_replay_equals_explicit_steps(dtype):
    from seq2seqsharp_amd.gpt import HipGpt, TOPP
    cfg = _moe_cfg(dtype)
    w = synth.make_weights(cfg, 3, random_bias=True)
    seqs = [list(range(5, 5 + n)) for n in (12, 7, 1, 12, 9)]
    ids, lens = HipGpt.pad_sentences(seqs)
    u = synth.make_uniforms(9, cfg["batch"], 6)
    a = HipGpt(cfg, w, max_batch=5, max_seq_len=32)
    a.set_repeat_penalty(2.0)
    a.prefill(ids, lens)
    toks, _ = a.generate(6, mode=TOPP, top_p=0.8, temperature=1.0, uniforms=u)
    b = HipGpt(cfg, w, max_batch=5, max_seq_len=32)
    b.set_repeat_penalty(2.0)
    b.prefill(ids, lens)
    for s in range(6):
        nxt = b.sample(mode=TOPP, top_p=0.8, temperature=1.0, uniforms=u[s])
        assert np.array_equal(nxt, toks[s]), s
        b.decode(nxt)
    assert np.array_equal(a.logits(), b.logits())
    a.close()
    b.close()


def test_appended_prefill_on_a_moe_model_equals_one_prefill():
    """Prompt-prefix reuse (the cached text is extended by new tokens) through MoE layers: fp32, so that both routes see the
    same routing inputs to the last bit."""
    from seq2seqsharp_amd.gpt import HipGpt
    cfg = _moe_cfg("f32")
    w = synth.make_weights(cfg, 4, random_bias=True)
    ids = synth.make_prompts(cfg, 8)
    one = HipGpt(cfg, w, max_batch=5, max_seq_len=32)
    one.prefill(ids)
    two = HipGpt(cfg, w, max_batch=5, max_seq_len=32)
    two.prefill(ids[:, :7])
    two.prefill(ids[:, 7:])
    assert np.abs(one.logits() - two.logits()).max() <= 1e-5 * np.abs(one.logits()).max()
    assert np.array_equal(one.generate(4)[0], two.generate(4)[0])
    one.close()
    two.close()


def test_reordered_rows_continue_like_their_sources():
    """TSHip_GptReorderRows with repeated and dropped rows (what beam pruning does): every new row decodes exactly like the
    row it was copied from."""
    from seq2seqsharp_amd.gpt import HipGpt
    cfg = synth.tiny_config(dtype="f16", batch=4, prompt=9)
    w = synth.make_weights(cfg, 6)
    ids = synth.make_prompts(cfg, 2)
    ref = HipGpt(cfg, w, max_batch=6, max_seq_len=32)
    ref.prefill(ids)
    src = np.array([2, 2, 0, 3, 2, 1], np.int32)
    tok = np.array([7, 8, 9, 10, 7, 11], np.int32)
    want = []
    for r, t in zip(src, tok):                      # row by row on a model of its own
        one = HipGpt(cfg, w, max_batch=1, max_seq_len=32)
        one.prefill(ids[r:r + 1])
        one.decode(np.array([t], np.int32))
        want.append(one.logits()[0])
        one.close()
    ref.reorder_rows(src)
    ref.decode(tok)
    got = ref.logits()
    assert got.shape[0] == 6
    assert np.abs(got - np.stack(want)).max() <= 2e-3       # (batch 1 and batch 6 take different GEMM tilings: fp16 rounding apart)
    assert np.array_equal(got[0], got[4])                    # same source, same token: identical rows
    ref.close()


def test_vocabulary_beyond_sixteen_bits(oracle):
    """A vocabulary of 70 000 entries: greedy and top-p picks index past 65 535 (every probability gets a 32-bit index in the
    sort keys), against the oracle with the shared uniform stream."""
    from seq2seqsharp_amd.gpt import HipGpt, TOPP
    cfg = synth.tiny_config(dtype="f32", n_layers=1, hidden=32, n_heads=2, n_kv_heads=1, ffn_dim=48, vocab=70000, batch=3, prompt=5)
    w = synth.make_weights(cfg, 8)
    w["FeedForward_Decoder_0.m_Bd"] = np.linspace(-2.0, 6.0, 70000, dtype=np.float32).reshape(1, -1)      # favour the high indices
    ids = synth.make_prompts(cfg, 3)
    orc = oracle.OracleGpt(cfg, w)
    gpu = HipGpt(cfg, w, max_batch=3, max_seq_len=16)
    p, lg = orc.step(ids, use_cache=True)
    gpu.prefill(ids)
    assert np.abs(gpu.logits() - lg).max() <= 1e-4 * np.abs(lg).max()
    assert np.array_equal(gpu.sample(), oracle.argmax(p).astype(np.int32)) and gpu.sample().min() > 65535
    u = synth.make_uniforms(4, 3, 1)[0]
    want = oracle.toppsample(p, 0.9, 0.0, None, u)
    got = gpu.sample(mode=TOPP, top_p=0.9, temperature=1.0, uniforms=u)
    assert np.array_equal(got, want.astype(np.int32))
    gpu.close()
