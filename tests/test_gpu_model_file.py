"""A model file written in the reference's format drives the fused path: same tokens and logits as the weights given directly."""
import numpy as np
import pytest

from seq2seqsharp_amd import model_file, synth

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("storage", ["f32", "f16"])
def test_model_file_to_decode(oracle, storage, tmp_path):
    from seq2seqsharp_amd.gpt import HipGpt
    cfg = synth.tiny_config(dtype="f16" if storage == "f16" else "f32")
    w = synth.make_weights(cfg, 12, random_bias=True)
    path = str(tmp_path / "gpt.model")
    model_file.save_gpt(cfg, w, path, storage=storage)
    ids = synth.make_prompts(cfg, 2)
    m, vocab = HipGpt.from_model_file(path, max_batch=cfg["batch"], max_seq_len=32)
    direct = HipGpt(cfg, w, max_batch=cfg["batch"], max_seq_len=32)
    assert m.cfg["dtype"] == cfg["dtype"] and len(vocab["index_to_word"]) == cfg["vocab"]
    m.prefill(ids)
    direct.prefill(ids)
    lg = m.logits()
    assert np.array_equal(lg, direct.logits())
    assert np.array_equal(m.generate(6)[0], direct.generate(6)[0])
    w_eff = {k: np.asarray(v, np.float32).astype(np.float16).astype(np.float32) for k, v in w.items()} if storage == "f16" else w
    _, want = oracle.OracleGpt(cfg, w_eff).step(ids, use_cache=True)
    assert np.abs(lg - want).max() <= (2e-2 if storage == "f16" else 1e-4) * max(1.0, np.abs(want).max())
    m.close()
    direct.close()
