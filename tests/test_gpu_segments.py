"""Segment embeddings on the fused GPTDecoder path (TensorUtils.CreateTokensEmbeddings, Seq2SeqSharp/Utils/TensorUtils.cs:60-72,
147-152): against the CPU oracle, whose segment logic tests/test_oracle_layers_numpy.py pins."""
import numpy as np
import pytest

from seq2seqsharp_amd import synth

pytestmark = pytest.mark.gpu

CASES = {
    "f32_rms": dict(),
    "f32_ln_mha": dict(norm_type=synth.LAYERNORM, attn_type=synth.MHA, n_kv_heads=4, act=synth.RELU),
    "f16_rms": dict(dtype="f16"),                                                   # deferred-norm decode step, fused sampling + embedding
    "f16_ln": dict(dtype="f16", norm_type=synth.LAYERNORM, act=synth.RELU),
    "f16_moe": dict(dtype="f16", n_layers=3, n_experts=4, experts_per_token=2, norm_type=synth.LAYERNORM, act=synth.RELU),
}


@pytest.mark.parametrize("name", sorted(CASES))
def test_segment_embeddings_against_oracle(oracle, name):
    from seq2seqsharp_amd.gpt import HipGpt
    cfg = synth.tiny_config(max_segments=4, sep_token_id=3, **CASES[name])
    w = synth.make_weights(cfg, 41, random_bias=True)
    w = {k: np.asarray(v, np.float32) for k, v in w.items()}
    w["SegmentEmbedding"] = (w["SegmentEmbedding"] * 20).astype(np.float32)          # as large as the scaled token embeddings
    seqs = synth.make_prompts(dict(cfg, prompt=12), 42)
    seqs[0, 1] = 3; seqs[0, 7] = 3; seqs[1, 0] = 3; seqs[1, 4] = 3; seqs[1, 9] = 3     # up to three separators: segments 0..3
    f16 = cfg["dtype"] == "f16"

    def close(a, b):
        return np.abs(a - b).max() <= 3e-2 if f16 else np.abs(a - b).max() <= 1e-4 * np.abs(b).max()

    orc = oracle.OracleGpt(cfg, w)
    gpu = HipGpt(cfg, w, max_batch=2, max_seq_len=40)
    p, lg = orc.step(seqs, use_cache=True)
    gpu.prefill(seqs)
    assert close(gpu.logits(), lg)
    # without the table the logits are far away: the comparison can fail
    cfg0 = dict(cfg, max_segments=0)
    p0, lg0 = oracle.OracleGpt(cfg0, {k: v for k, v in w.items() if k != "SegmentEmbedding"}).step(seqs, use_cache=True)
    assert np.abs(lg0 - lg).max() > 0.1
    cur = seqs
    for tok in (3, 11, 3):                              # cached steps: segment 0 whatever the token and the history
        nxt = np.full((2,), tok, np.int32)
        cur = np.concatenate([cur, nxt[:, None]], 1)
        p, lg = orc.step(cur, use_cache=True)
        gpu.decode(nxt)
        assert close(gpu.logits(), lg)
    # the captured generate loop gives the step-wise tokens
    ids, _ = gpu.generate(4)
    gpu.reset()
    gpu.prefill(seqs)
    for tok in (3, 11, 3):
        gpu.decode(np.full((2,), tok, np.int32))
    for s in range(4):
        nxt = gpu.sample()
        assert np.array_equal(nxt, ids[s])
        gpu.decode(nxt)
    gpu.close()


def test_more_separators_than_segments_is_refused():
    from seq2seqsharp_amd._lib import TSHipError
    from seq2seqsharp_amd.gpt import HipGpt
    cfg = synth.tiny_config(max_segments=2, sep_token_id=3)
    w = synth.make_weights(cfg, 1)
    gpu = HipGpt(cfg, w, max_batch=2, max_seq_len=32)
    seqs = synth.make_prompts(cfg, 2)
    seqs[0, 1] = 3; seqs[0, 2] = 3; seqs[0, 3] = 3      # the fourth token would need segment 2
    with pytest.raises(TSHipError, match="more separator tokens"):
        gpu.prefill(seqs)
    seqs[0, 3] = 9; seqs[0, 2] = 9
    gpu.reset()
    gpu.prefill(seqs)                                   # one separator: segments 0 and 1
    gpu.close()
