"""CPU-side checks of the boundary: the C-ABI library loads, exports every symbol include/tship.h declares, reports
errors through the reference's convention (0 + per-thread message), and the product package has no route to the
oracle or to any CPU fallback."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "tship.h")).read()
    return sorted(set(re.findall(r"TSHIP_API\s+[\w\s\*]+?\b(TSHip_\w+)\s*\(", text)))


def test_header_declares_the_expected_surface():
    names = _declared()
    assert len(names) >= 45
    for must in ["TSHip_GetLastError", "TSHip_Malloc", "TSHip_Addmm", "TSHip_AddmmBatch", "TSHip_IndexSelect", "TSHip_RoPE",
                 "TSHip_RMSNorm", "TSHip_LayerNorm", "TSHip_Softmax", "TSHip_Argmax", "TSHip_TopK", "TSHip_TopPSample",
                 "TSHip_GptCreate", "TSHip_GptPrefill", "TSHip_GptDecode", "TSHip_GptGenerate"]:
        assert must in names


def test_library_exports_every_declared_symbol():
    from seq2seqsharp_amd._lib import lib
    L = lib()
    missing = [n for n in _declared() if not hasattr(L, n)]
    assert not missing, missing


def test_error_convention_without_a_device():
    from seq2seqsharp_amd._lib import lib
    L = lib()
    n = C.c_int(-1)
    L.TSHip_GetDeviceCount.argtypes = [C.POINTER(C.c_int)]
    assert L.TSHip_GetDeviceCount(C.byref(n)) == 1 and n.value >= 0
    assert L.TSHip_GetDeviceCount(None) == 0                      # null argument -> 0 + message, no crash
    assert b"null" in L.TSHip_GetLastError()
    if n.value == 0:
        L.TSHip_Init.argtypes = [C.c_int]
        assert L.TSHip_Init(0) == 0
        assert len(L.TSHip_GetLastError()) > 0
        # the fused path fails loudly instead of falling back to anything
        from seq2seqsharp_amd import synth
        from seq2seqsharp_amd._lib import TSHipError
        from seq2seqsharp_amd.gpt import HipGpt
        with pytest.raises(TSHipError):
            HipGpt(synth.tiny_config(), synth.make_weights(synth.tiny_config(), 0))


def test_product_never_touches_the_oracle():
    pkg = os.path.join(ROOT, "seq2seqsharp_amd")
    for dirpath, _, files in os.walk(pkg):
        if os.path.basename(dirpath) == "build":
            continue
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cpp")):
                text = open(os.path.join(dirpath, f), errors="ignore").read()
                assert "ts_oracle" not in text and "import oracle" not in text and "from oracle" not in text, f


def test_synthetic_configs_match_the_contract():
    from seq2seqsharp_amd import synth
    c2 = synth.CONFIGS["cfg2_1b_gqa_f16"]
    assert (c2["n_layers"], c2["hidden"], c2["n_heads"], c2["n_kv_heads"], c2["ffn_dim"], c2["vocab"], c2["batch"], c2["prompt"]) == \
        (16, 2048, 32, 8, 5632, 32000, 32, 1024)
    assert c2["rope_base"] == 500000.0            # the reference's literal (TensorApplyCPU.cs:1161)
    # weights streamed per decode step: everything but the embedding table -> 787.0 M parameters
    streamed = synth.n_params(c2) - c2["vocab"] * c2["hidden"] - sum(
        int(__import__("numpy").prod(s)) for n, s, k in synth.weight_shapes(c2) if k != "normal")
    assert abs(streamed - 787.0e6) < 0.5e6
