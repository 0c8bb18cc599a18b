"""Writes tests/golden/tiny_models.{json,npz}: greedy decodes of tiny seeded GPTDecoder models on the CPU oracle.

The reference itself cannot run here (C#, no .NET runtime), so these vectors come from the oracle after it has been
pinned by tests/test_oracle_fixtures.py and tests/test_oracle_model.py; they guard the oracle against drift and give
the GPU tests a fixed target.   Run:  python tests/golden/make_golden.py
"""
import json
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import ts_oracle as O          # noqa: E402
from seq2seqsharp_amd import synth        # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))
CASES = [
    ("gqa_rms_gate_f32", synth.tiny_config(), 0),
    ("mha_ln_relu_f32", synth.tiny_config(attn_type=synth.MHA, n_kv_heads=4, norm_type=synth.LAYERNORM, act=synth.RELU), 1),
    ("gqa_rms_silu_f32", synth.tiny_config(act=synth.SILU), 2),
    ("gqa_rms_gate_f16w", synth.tiny_config(dtype="f16"), 3),
    ("moe_ln_relu_f32", synth.tiny_config(n_layers=4, n_experts=4, experts_per_token=2, norm_type=synth.LAYERNORM, act=synth.RELU), 4),
]


def main():
    O.build()
    meta, arrays = {"cases": []}, {}
    for name, cfg, seed in CASES:
        w = synth.make_weights(cfg, seed, random_bias=True)
        orc = O.OracleGpt(cfg, w)
        seqs = synth.make_prompts(cfg, seed + 100)
        cur, logits = seqs.copy(), []
        steps = 8
        for _ in range(steps + 1):
            p, lg = orc.step(cur, use_cache=True)
            logits.append(lg)
            cur = np.concatenate([cur, O.argmax(p).astype(np.int32)[:, None]], 1)
        arrays[name + "_prompt"] = seqs
        arrays[name + "_tokens"] = cur
        arrays[name + "_logits"] = np.stack(logits)
        meta["cases"].append({"name": name, "cfg": cfg, "weight_seed": seed, "steps": steps})
    np.savez_compressed(os.path.join(HERE, "tiny_models.npz"), **arrays)
    json.dump(meta, open(os.path.join(HERE, "tiny_models.json"), "w"), indent=1)
    print("wrote", len(CASES), "cases")


if __name__ == "__main__":
    main()
