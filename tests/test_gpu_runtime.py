"""Runtime half of the boundary on the GPU: the memory pool behind TSHip_Malloc / TSHip_Free and calls from several
threads (the reference issues ops from Parallel.For workers, BaseSeq2SeqFramework.cs:912-941)."""
import ctypes as C
import threading

import numpy as np
import pytest

from seq2seqsharp_amd import synth

pytestmark = pytest.mark.gpu


def _rt():
    from seq2seqsharp_amd._lib import lib
    L = lib()
    L.TSHip_Init.argtypes = [C.c_int]
    L.TSHip_Malloc.argtypes = [C.POINTER(C.c_void_p), C.c_size_t]
    L.TSHip_Free.argtypes = [C.c_void_p]
    L.TSHip_PoolTrim.argtypes = []
    L.TSHip_GetPoolStats.argtypes = [C.POINTER(C.c_size_t), C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)]
    L.TSHip_GetLastError.restype = C.c_char_p
    assert L.TSHip_Init(0) == 1
    return L


def _stats(L):
    a, b, c = C.c_size_t(0), C.c_size_t(0), C.c_size_t(0)
    assert L.TSHip_GetPoolStats(C.byref(a), C.byref(b), C.byref(c)) == 1
    return a.value, b.value, c.value


def test_pool_reuses_blocks_without_driver_calls():
    L = _rt()
    rng = np.random.default_rng(0)
    allocs0, live0, _ = _stats(L)
    sizes = [int(s) for s in rng.choice([64, 1000, 4096, 70000, 1 << 20, 3 << 20], 10000)]
    held = []
    for i, sz in enumerate(sizes):                          # a working set of up to 40 live tensors, like a layer's temporaries
        p = C.c_void_p()
        assert L.TSHip_Malloc(C.byref(p), sz) == 1 and p.value
        held.append(p)
        if len(held) > 40:
            assert L.TSHip_Free(held.pop(int(rng.integers(0, len(held))))) == 1
    for p in held:
        assert L.TSHip_Free(p) == 1
    allocs1, live1, cached1 = _stats(L)
    assert allocs1 - allocs0 < 100, "10000 allocations must not reach the driver more than a few dozen times"
    assert live1 == live0 and cached1 > 0
    # the same size comes back as the same block
    p, q = C.c_void_p(), C.c_void_p()
    L.TSHip_Malloc(C.byref(p), 5000)
    first = p.value
    L.TSHip_Free(p)
    L.TSHip_Malloc(C.byref(q), 4999)
    assert q.value == first
    L.TSHip_Free(q)
    # what the pool did not hand out is refused, as is a second free
    assert L.TSHip_Free(C.c_void_p(0x1000)) == 0 and b"TSHip_Malloc" in L.TSHip_GetLastError()
    assert L.TSHip_Free(q) == 0
    assert L.TSHip_PoolTrim() == 1 and _stats(L)[2] == 0


def test_pooled_blocks_carry_tensor_data_in_stream_order():
    """A block freed and handed out again while the GPU may still work: results stay those of the ordered stream."""
    from seq2seqsharp_amd import ops
    from seq2seqsharp_amd.tensor import HipTensor as HT
    rng = np.random.default_rng(1)
    a = rng.standard_normal((64, 300)).astype(np.float32)
    want = a.copy()
    t = HT.from_numpy(a)
    for i in range(200):                                    # temporaries come and go; each result is read only at the end
        u = ops.add(None, t, 1.0)                           # "addv" into a fresh tensor
        t.dispose()                                         # back to the pool while the kernel may still be running
        t = u
        want = want + np.float32(1.0)
    assert np.array_equal(t.numpy(), want)


def test_last_error_is_per_thread_and_calls_serialise():
    L = _rt()
    errs = {}

    def worker(name, bad_call, expect):
        for _ in range(200):
            assert bad_call() == 0
            msg = L.TSHip_GetLastError()
            if expect not in msg:
                errs[name] = msg
                return

    t1 = threading.Thread(target=worker, args=("free", lambda: L.TSHip_Free(C.c_void_p(0x2000)), b"TSHip_Free"))
    t2 = threading.Thread(target=worker, args=("malloc", lambda: L.TSHip_Malloc(None, 16), b"TSHip_Malloc: ptr is null"))
    t1.start(); t2.start(); t1.join(); t2.join()
    assert not errs, errs


def test_two_models_on_two_threads():
    """Two TSHipGpt objects driven from two threads at once (graph capture, replays and eager steps interleave on the one
    stream): each produces exactly the tokens it produces alone."""
    from seq2seqsharp_amd import gpt as G
    cfgs = [synth.tiny_config(dtype="f16", batch=3, prompt=9), synth.tiny_config(dtype="f32", batch=2, prompt=6, attn_type=synth.MHA, n_kv_heads=4)]
    models, prompts, alone = [], [], []
    for i, cfg in enumerate(cfgs):
        w = synth.make_weights(cfg, 20 + i, random_bias=True)
        m = G.HipGpt(cfg, w, max_batch=cfg["batch"], max_seq_len=80)
        p = synth.make_prompts(cfg, 30 + i)
        m.prefill(p)
        ids, _ = m.generate(24)
        alone.append(ids)
        models.append(m); prompts.append(p)
    out = [None, None]
    fails = []

    def run(i):
        try:
            for rep in range(5):
                models[i].reset()
                models[i].prefill(prompts[i])
                a, _ = models[i].generate(10)
                t = models[i].sample()
                models[i].decode(t)
                b, _ = models[i].generate(13)
                got = np.concatenate([a, t[None], b])
                if not np.array_equal(got, alone[i]):
                    fails.append((i, rep))
            out[i] = got
        except Exception as e:      # noqa: BLE001
            fails.append((i, repr(e)))

    ts = [threading.Thread(target=run, args=(i,)) for i in range(2)]
    for t in ts:
        t.start()
    for t in ts:
        t.join()
    assert not fails, fails
    for m in models:
        m.close()


def test_profile_reports_the_launched_symbols():
    """TSHip_GptProfileDecode / TSHip_GptProfileSymbols: one entry per launch of a decode step, the symbol being the kernel
    the runtime resolved for the launched function (what a profiler's kernel trace prints)."""
    from seq2seqsharp_amd import synth
    from seq2seqsharp_amd.gpt import HipGpt
    cfg = synth.tiny_config(dtype="f16")
    gpu = HipGpt(cfg, synth.make_weights(cfg, 1), max_batch=cfg["batch"], max_seq_len=32)
    gpu.prefill(synth.make_prompts(cfg, 2))
    prof = gpu.profile_decode(gpu.sample())
    syms = gpu.profile_symbols()
    assert len(prof) == len(syms) > 0
    names = [n for n, _ in prof]
    assert "attn_decode" in names and all(t >= 0 for _, t in prof)
    assert "attn" in syms[names.index("attn_decode")] and all("tship::" in s or "kernel" in s for s in syms)
    gpu.close()

