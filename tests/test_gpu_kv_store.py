"""Parked conversations: device-side snapshots of the cache rows (TSHip_GptSaveRows / TSHip_GptRestoreRows), the
counterpart of the reference's text-keyed MemoryCache of KV tensors (Applications/GPT.cs:153-173, 236-247, 312-328)."""
import numpy as np
import pytest

from seq2seqsharp_amd import synth

pytestmark = pytest.mark.gpu

CASES = [
    dict(),                                                                     # fp32, row-major cache
    dict(dtype="f16"),                                                          # fp16, row-major cache (head size 16)
    dict(dtype="f16", hidden=128, n_heads=2, n_kv_heads=1, ffn_dim=256),        # fp16, head size 64: fragment-major cache, MFMA attention
    dict(dtype="f16", norm_type=synth.LAYERNORM, act=synth.RELU, attn_type=synth.MHA, n_kv_heads=4),
    dict(dtype="f16", hidden=768, n_heads=12, n_kv_heads=1, ffn_dim=128),       # twelve query heads on one KV head: two groups of six
]


@pytest.mark.parametrize("kw", CASES)
def test_park_run_another_conversation_resume(kw):
    """Save after turn 1, run another conversation on the same model, restore, continue: logits and tokens are bit-equal to
    an uninterrupted run."""
    from seq2seqsharp_amd.gpt import HipGpt
    cfg = synth.tiny_config(**kw)
    w = synth.make_weights(cfg, 3, random_bias=True)
    a = synth.make_prompts(dict(cfg, batch=2, prompt=40), 5)
    other = synth.make_prompts(dict(cfg, batch=3, prompt=70), 6)
    cont = synth.make_prompts(dict(cfg, batch=2, prompt=6), 7)          # tokens of turn 2

    def turn1(g):
        g.prefill(a)
        ids, _ = g.generate(5)
        return ids

    ref = HipGpt(cfg, w, max_batch=4, max_seq_len=128)
    ids_ref = turn1(ref)
    lg1_ref = ref.logits()
    ref.prefill(cont)                       # turn 2 appends to the cached turn 1
    lg2_ref = ref.logits()
    ids2_ref, _ = ref.generate(4)
    lg3_ref = ref.logits()
    ref.close()

    g = HipGpt(cfg, w, max_batch=4, max_seq_len=128)
    ids1 = turn1(g)
    assert np.array_equal(ids1, ids_ref)
    snap = g.save_rows()
    b, n, nbytes = snap.info()
    assert (b, n) == (2, 45) and nbytes > 0
    g.reset()
    g.prefill(other)                        # another conversation overwrites rows 0..2 far beyond the saved length
    g.generate(9)
    g.restore_rows(snap)
    assert g.seq_len() == 45 and g.batch == 2
    assert np.array_equal(g.logits(), lg1_ref)
    g.prefill(cont)
    assert np.array_equal(g.logits(), lg2_ref)
    ids2, _ = g.generate(4)
    assert np.array_equal(ids2, ids2_ref) and np.array_equal(g.logits(), lg3_ref)
    # the snapshot is still whole: a second resume gives the same continuation
    g.restore_rows(snap)
    g.prefill(cont)
    assert np.array_equal(g.logits(), lg2_ref)
    snap.close()
    g.close()


def test_snapshot_keeps_the_token_history_of_top_p():
    """With a repeat penalty the model keeps every token's last position; a resumed conversation samples the same tokens."""
    from seq2seqsharp_amd.gpt import TOPP, HipGpt
    cfg = synth.tiny_config(dtype="f16")
    w = synth.make_weights(cfg, 11)
    a = synth.make_prompts(dict(cfg, batch=2, prompt=24), 2)
    other = synth.make_prompts(dict(cfg, batch=2, prompt=30), 4)
    u = synth.make_uniforms(5, 2, 12)

    def run(interrupt):
        g = HipGpt(cfg, w, max_batch=2, max_seq_len=96)
        g.set_repeat_penalty(2.0)
        g.prefill(a)
        ids1, _ = g.generate(6, mode=TOPP, top_p=0.9, temperature=1.0, uniforms=u[:6])
        if interrupt:
            snap = g.save_rows()
            g.reset()
            g.prefill(other)
            g.generate(3, mode=TOPP, top_p=0.9, temperature=1.0, uniforms=u[:3])
            g.restore_rows(snap)
            snap.close()
        ids2, _ = g.generate(6, mode=TOPP, top_p=0.9, temperature=1.0, uniforms=u[6:])
        g.close()
        return ids1, ids2

    r0, r1 = run(False), run(True)
    assert np.array_equal(r0[0], r1[0]) and np.array_equal(r0[1], r1[1])


def test_refusals_and_the_text_keyed_store():
    from seq2seqsharp_amd._lib import TSHipError
    from seq2seqsharp_amd.gpt import HipGpt, KvStore
    cfg = synth.tiny_config()
    w = synth.make_weights(cfg, 1)
    g = HipGpt(cfg, w, max_batch=2, max_seq_len=64)
    with pytest.raises(TSHipError, match="no sequences"):
        g.save_rows()
    g.prefill(synth.make_prompts(dict(cfg, batch=2, prompt=50), 1))
    snap = g.save_rows()
    small = HipGpt(cfg, w, max_batch=2, max_seq_len=32)               # cache too short for the saved length
    with pytest.raises(TSHipError, match="does not fit"):
        small.restore_rows(snap)
    small.close()
    cfg2 = synth.tiny_config(n_kv_heads=4)
    wide = HipGpt(cfg2, synth.make_weights(cfg2, 1), max_batch=2, max_seq_len=64)
    with pytest.raises(TSHipError, match="another shape"):
        wide.restore_rows(snap)
    wide.close()
    # the store: keyed by text, sliding expiry
    now = [0.0]
    store = KvStore(ttl_seconds=600.0, clock=lambda: now[0])
    store.put("hello world", snap)
    now[0] = 500.0
    assert store.get("hello world") is snap and store.get("something else") is None
    now[0] = 1000.0                                                    # 500 s after the last use: still there
    assert len(store) == 1
    now[0] = 1700.0                                                    # 700 s after the last use: gone, and freed
    assert store.get("hello world") is None and snap.h is None
    g.close()
