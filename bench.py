#!/usr/bin/env python3
"""Benchmark of the GPTDecoder decode loop on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config cfg2_1b_gqa_f16] [--no-cpu-baseline]

A "step" is one decode step of the whole batch (one new token per sequence) on synthetic data:
seeded N(0, 0.02) weights of the named architecture and uniform-random prompts, KV cache filled by a real
prefill of the prompts.  Prints ONE JSON line: decode tokens/s (whole batch), the roofline of the
dominant kernel (the one with the largest share of the step; every streaming kernel is listed in roofline_all)
measured live with device events, and the CPU baseline (the oracle's restatement of the reference's CPU backend, single thread,
timed on a bounded sample on this host).
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, vendor figure
MFMA_FP16_PEAK_TFLOPS = 2500.0  # MI355X dense fp16 matrix, vendor figure


def algorithmic_prefill_flops(cfg, B, Tp):
    h, H, G, F, V, L = cfg["hidden"], cfg["n_heads"], cfg["n_kv_heads"], cfg["ffn_dim"], cfg["vocab"], cfg["n_layers"]
    d = h // H
    nW = 3 if cfg["act"] in (3, 4) else 2
    # MoE layers (every layer after the second when the model has experts, GPTDecoder.cs:83-91): a token runs through
    # experts_per_token experts of two matrices h x 4h and 4h x h each, plus the router (MoEFeedForward.cs:76-181)
    E, k = cfg.get("n_experts", 1), cfg.get("experts_per_token", 1)
    n_moe = max(L - 2, 0) if E > 1 else 0
    ffn = (L - n_moe) * nW * h * F + n_moe * (k * 2 * h * 4 * h + h * E)
    per_tok = L * (h * H * d + 2 * h * G * d + H * d * h) + ffn
    return 2.0 * B * Tp * per_tok + 2.0 * B * h * V + L * B * H * d * float(Tp) * Tp * 2.0


def _log(msg):
    print("[bench] " + msg, file=sys.stderr, flush=True)


def _cpu_model():
    try:
        for line in open("/proc/cpuinfo"):
            if line.lower().startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def _oracle_flags():
    """The compiler line of the oracle's build recipe (oracle/Makefile), as text."""
    cxx, flags = "g++", ""
    try:
        for line in open(os.path.join(ROOT, "oracle", "Makefile")):
            if line.startswith("CXXFLAGS"):
                flags = line.split("=", 1)[1].strip()
            elif line.startswith("CXX "):
                cxx = line.split("=", 1)[1].strip()
    except OSError:
        pass
    return (cxx + " " + flags + " -fopenmp").strip()


def cpu_baseline(cfg, gpu, weights, next_ids, budget_note, n_steps=4):
    """n_steps decode steps of the CPU oracle (kind "port": a restatement of the reference's CPU path), single
    thread, at the benchmark's shape, on the KV cache the GPU prefill produced; the mean is reported.  Also returns
    the logits of the first of those steps, for a full-size parity number against the GPU's."""
    from oracle import ts_oracle as O
    O.set_threads(1)
    B = gpu.batch
    H, G = cfg["n_heads"], cfg["n_kv_heads"]
    d = cfg["hidden"] // H
    T = gpu.seq_len()
    orc = O.OracleGpt(cfg, weights)
    for l in range(cfg["n_layers"]):
        k = gpu.get_kv(l, 0)                      # [B, G, T, d]
        v = gpu.get_kv(l, 1)
        # the reference caches K/V expanded to all query heads, K transposed (GroupQueryAttention.cs:156-188)
        ke = np.repeat(k, H // G, axis=1).transpose(0, 1, 3, 2).reshape(B * H, d, T)
        ve = np.repeat(v, H // G, axis=1).reshape(B * H, T, d)
        orc.set_cache(l, 0, ke, B * H, T, d)
        orc.set_cache(l, 1, ve, B * H, T, d)
    seqs = np.ascontiguousarray(next_ids.reshape(B, 1), dtype=np.int32)
    times, first_logits = [], None
    for i in range(max(1, n_steps)):
        t0 = time.perf_counter()
        probs, lg = orc.step(seqs, use_cache=True)       # (a cached step looks at the last token of every sequence only)
        times.append(time.perf_counter() - t0)
        _log("CPU oracle step %d of %d: %.1f s" % (i + 1, n_steps, times[-1]))
        if first_logits is None:
            first_logits = lg
        seqs = np.concatenate([seqs, O.argmax(probs).astype(np.int32).reshape(B, 1)], 1)
    dt = float(np.mean(times))
    return {"value": B / dt, "unit": "tokens/s", "cores": 1, "threads": 1, "kind": "port",
            "cpu_model": _cpu_model(), "nproc": os.cpu_count(), "compiler": _oracle_flags(),
            "seconds_per_step": [round(t, 2) for t in times],
            "sample": "%d decode steps of the whole batch from KV length %d (%s), mean %.1f s per step; the full run of %d steps "
                      "would take about %.0f s at that rate (extrapolated)" % (len(times), T, budget_note, dt, cfg.get("steps", 0), dt * cfg.get("steps", 0))}, first_logits


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--config", default="cfg2_1b_gqa_f16")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-steps", type=int, default=4, help="decode steps of the CPU oracle to time (their mean is the reported baseline)")
    ap.add_argument("--no-topp", action="store_true")
    ap.add_argument("--prompt", type=int, default=0, help="override the prompt length")
    ap.add_argument("--prefill-runs", type=int, default=3, help="timed prefill calls (the fastest is reported; many of them keep the chip under load long enough to sample its clock)")
    ap.add_argument("--no-copy-calibration", action="store_true",
                    help="skip the 256 MiB plain copy that gives rocprofv3 counter runs a kernel of known traffic")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build drives one GPU per process and measures one GPU; --gpus %d is not supported "
              "(each GPU would hold a full replica and its own batch rows, with no per-step exchange)" % args.gpus, file=sys.stderr)
        sys.exit(2)

    from seq2seqsharp_amd import synth
    from seq2seqsharp_amd.gpt import GREEDY, TOPP, HipGpt

    cfg = dict(synth.CONFIGS[args.config])
    if args.prompt:
        cfg["prompt"] = args.prompt
    B, Tp, K, W = cfg["batch"], cfg["prompt"], args.steps, args.warmup
    t0 = time.perf_counter()
    _log("generating weights for %s" % args.config)
    weights = synth.make_weights(cfg, seed=0)
    _log("uploading weights")
    gpu = HipGpt(cfg, weights, max_batch=B, max_seq_len=Tp + 2 * (W + K) + 8)
    t_load = time.perf_counter() - t0
    prompts = synth.make_prompts(cfg, seed=1)

    # prefill (timed separately)
    _log("prefill of %d x %d tokens" % (B, Tp))
    if not args.no_topp:
        gpu.set_repeat_penalty(2.0)        # DecodingOptions.RepeatPenalty's default; only the top-p leg below applies it
    gpu.prefill(prompts)                   # untimed: loads every kernel and sizes the prefill workspace
    prefill_runs = []
    for _ in range(max(1, args.prefill_runs)):       # host wall clock of the whole call (token upload and final sync included)
        gpu.reset()
        t0 = time.perf_counter()
        gpu.prefill(prompts)
        prefill_runs.append(time.perf_counter() - t0)
    t_prefill = min(prefill_runs)
    prefill_tok_s = B * Tp / t_prefill
    prefill_tflops = algorithmic_prefill_flops(cfg, B, Tp) / t_prefill / 1e12

    # decode: W warm-up steps, then exactly K timed steps (device events on the library stream, bracketed by syncs)
    _log("decode: %d warm-up + %d timed steps" % (W, K))
    gpu.generate(max(W, 1))
    T_start = gpu.seq_len()
    wall0 = time.perf_counter()
    ids, ms = gpu.generate(K)
    wall = time.perf_counter() - wall0
    T_end = gpu.seq_len()
    ms_per_step = ms / K
    tok_s = B * K / (ms / 1e3)
    wbytes, _ = gpu.step_bytes(B)
    d = cfg["hidden"] // cfg["n_heads"]
    es = 2 if cfg["dtype"] == "f16" else 4
    kv_per_pos = es * cfg["n_layers"] * B * cfg["n_kv_heads"] * d * 2
    step_bytes = wbytes + kv_per_pos * (T_start + T_end + 1) / 2.0
    step_gbs = step_bytes / (ms_per_step / 1e3) / 1e9

    # per-kernel device times of single decode steps (device events attached to every dispatch on the library stream) ->
    # roofline of every streaming kernel; the dominant kernel is the one with the largest share of the step
    nxt = gpu.sample()
    acc = {}
    n_prof = 5
    symbols = {}
    for _ in range(n_prof):
        prof = gpu.profile_decode(nxt)
        syms = gpu.profile_symbols()
        for (name, t), sym in zip(prof, syms):
            acc.setdefault(name, []).append(t)
            symbols[name] = sym
    kernel_ms = {k: round(float(np.sum(v)) / n_prof, 4) for k, v in acc.items()}
    step_sum = sum(kernel_ms.values())
    t_attn = T_end + 1 + (n_prof - 1) / 2.0                  # mean KV length of the profiled steps
    h, F, V, Hq, Hkv = cfg["hidden"], cfg["ffn_dim"], cfg["vocab"], cfg["n_heads"], cfg["n_kv_heads"]
    nW13 = 2 if cfg["act"] in (3, 4) else 1
    E = cfg.get("n_experts", 1)
    # algorithmic bytes of one launch: the weights (or the cache) it must read once
    launch_bytes = {
        "gemm_qkv": float(h) * (Hq + 2 * Hkv) * d * es,
        "attn_decode": float(es) * B * Hkv * d * 2 * t_attn,
        "gemm_wo": float(h) * h * es,
        "gemm_ffn13": float(h) * F * nW13 * es,
        "gemm_ffn2": float(F) * h * es,
        "gemm_head": float(h) * V * es,
        "moe_gemm1": float(min(E, B * cfg.get("experts_per_token", 1))) * h * 4 * h * es,
        "moe_gemm2": float(min(E, B * cfg.get("experts_per_token", 1))) * 4 * h * h * es,
    }
    roofline_all = {}
    for name, ts in acc.items():
        if name not in launch_bytes:
            continue
        ms_avg = float(np.mean(ts))
        gbs = launch_bytes[name] / (ms_avg / 1e3) / 1e9
        roofline_all[name] = {"kernel": symbols.get(name, ""), "bytes_per_launch": launch_bytes[name], "avg_launch_us": round(ms_avg * 1e3, 2),
                              "launches_per_step": len(ts) // n_prof, "achieved_GBps": round(gbs, 1), "frac": round(gbs / HBM_PEAK_GBS, 4),
                              "share_of_step": round(kernel_ms[name] / step_sum, 3)}
    dom = max(roofline_all, key=lambda k: roofline_all[k]["share_of_step"])
    dom_r = roofline_all[dom]

    # a plain copy of known size: the reference point for scaling FETCH_SIZE / WRITE_SIZE in counter runs
    if not args.no_copy_calibration:
        from seq2seqsharp_amd import ops
        from seq2seqsharp_amd.tensor import HipTensor
        src = ops.fill(HipTensor([64 * 1024 * 1024]), 1.0)        # 256 MiB of float32
        dst = HipTensor([64 * 1024 * 1024])
        ops.copy(dst, src)
        ops.copy(dst, src)
        src.dispose()
        dst.dispose()

    # HBM traffic per launch of the dominant kernel comes from hardware counters, which a separate rocprofv3 --pmc run of this
    # script collects; the figure printed here is the one from the committed summary of that run (named beside it), never
    # a value measured in this process
    traffic, traffic_source, traffic_kv_len, traffic_ratio, traffic_alg = None, None, None, None, None
    tpath = os.path.join(ROOT, "profiles", "decode_%s_%s_traffic.json" % (args.config, dom))
    if os.path.exists(tpath):
        tj = json.load(open(tpath))
        traffic = tj.get("traffic_bytes_per_launch")
        traffic_kv_len = tj.get("kv_len")                    # attention: the KV length of the counter run (its bytes grow with it)
        traffic_alg = tj.get("algorithmic_bytes_per_launch")  # algorithmic bytes at that same KV length
        traffic_ratio = tj.get("traffic_over_algorithmic")    # the comparable figure: both byte counts at the counter run's KV length
        traffic_source = "profiles/" + os.path.basename(tpath)

    out = {
        "metric": "decode tokens/s on 1 GPU (1B GQA fp16, batch 32)" if args.config == "cfg2_1b_gqa_f16" else "decode tokens/s on 1 GPU",
        "value": round(tok_s, 1), "unit": "tokens/s", "n_gpus": 1, "steps": K, "warmup": W,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": cfg["dtype"], "data": "synthetic",
        "config": {"workload": args.config, "batch": B, "prompt_len": Tp, "kv_len_start": T_start, "kv_len_end": T_end,
                   "sampling": "greedy", "rope_base": cfg["rope_base"]},
        "roofline": {"bound": "hbm", "achieved": dom_r["achieved_GBps"], "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": dom_r["frac"],
                     "traffic": traffic, "traffic_over_algorithmic": traffic_ratio, "traffic_algorithmic_bytes_same_run": traffic_alg,
                     "traffic_source": traffic_source, "traffic_kv_len": traffic_kv_len, "kernel": dom_r["kernel"], "launch": dom,
                     "bytes_per_launch": dom_r["bytes_per_launch"], "avg_launch_ms": round(dom_r["avg_launch_us"] / 1e3, 5),
                     "timing": "device events attached to each dispatch of 5 profiled steps (a rocprofv3 kernel trace of the graph replays reads about 5 % longer)",
                     "kv_len": t_attn if dom == "attn_decode" else None, "share_of_step": dom_r["share_of_step"]},
        "roofline_all": roofline_all,
        "whole_step": {"algorithmic_bytes": round(step_bytes), "achieved_GBps": round(step_gbs, 1),
                       "frac_of_hbm_peak": round(step_gbs / HBM_PEAK_GBS, 4), "host_wall_ms_per_step": round(wall / K * 1e3, 4)},
        "prefill": {"tokens_per_s": round(prefill_tok_s, 1), "seconds": round(t_prefill, 4), "runs": [round(t, 4) for t in prefill_runs[:8]], "median_seconds": round(sorted(prefill_runs)[len(prefill_runs) // 2], 4),
                    "algorithmic_TFLOPs": round(prefill_tflops, 2),
                    "frac_of_fp16_mfma_peak": round(prefill_tflops / MFMA_FP16_PEAK_TFLOPS, 4) if cfg["dtype"] == "f16" else None},
        "kernel_ms_per_step": kernel_ms,
        "load_seconds": round(t_load, 1),
    }
    if not args.no_topp:
        _log("top-p decode")
        u = synth.make_uniforms(7, B, K)
        _, ms_p = gpu.generate(K, mode=TOPP, top_p=0.9, temperature=1.0, uniforms=u)
        out["topp"] = {"top_p": 0.9, "repeat_penalty": 2.0, "tokens_per_s": round(B * K / (ms_p / 1e3), 1), "ms_per_step": round(ms_p / K, 4)}
    if not args.no_cpu_baseline:
        _log("CPU baseline (%d decode steps of the oracle, single thread)" % args.cpu_steps)
        nxt = gpu.sample()
        base, lg = cpu_baseline(cfg, gpu, weights, nxt, "cache from the GPU prefill", n_steps=args.cpu_steps)
        gpu.decode(nxt)
        out["cpu_baseline"] = base
        gl = gpu.logits()
        g1, c1 = gl.argmax(1), lg.argmax(1)
        rows = np.nonzero(g1 != c1)[0]
        ar = np.arange(gl.shape[0])
        tie = (lg[ar, c1] - lg[ar, g1]) <= 2.0 * np.abs(gl - lg).max(1)      # the CPU's own gap is within the row's logit error
        out["parity_full_size"] = {"max_abs_logit_diff_vs_cpu": float(np.abs(gl - lg).max()),
                                   "top1_agree": float((g1 == c1).mean()), "top1_agree_ties_counted": float(((g1 == c1) | tie).mean()),
                                   "rows": int(gl.shape[0]),
                                   # where the choices differ: how far apart the CPU's own logits of the two tokens are
                                   # (a gap below the logit difference above is a tie at this precision)
                                   "cpu_logit_gap_where_top1_differs": [float(lg[r, c1[r]] - lg[r, g1[r]]) for r in rows]}
    else:
        out["cpu_baseline"] = None
    print(json.dumps(out))


if __name__ == "__main__":
    main()
