"""Host-side mirror of the reference's GPT decode loop over the fused C-ABI path.

`HipGpt` plays the role of Seq2SeqSharp's GPT.RunForwardOnSingleDevice + Decoder.GPTDecode
(Seq2SeqSharp/Applications/GPT.cs:212-335, Applications/Decoder.cs:648-794): prompts in, token ids out,
KV cache kept on the device.  Every method is a thin call into libtship.so; nothing is computed here.
"""
import ctypes as C

import numpy as np

from ._lib import TSHipGptConfig, check, lib

GREEDY, TOPP = 0, 1
F32, F16 = 0, 1

_proto_done = False


def _protos():
    global _proto_done
    if _proto_done:
        return
    L = lib()
    vp = C.c_void_p
    L.TSHip_Init.argtypes = [C.c_int]
    L.TSHip_GptCreate.argtypes = [C.POINTER(TSHipGptConfig), C.POINTER(vp)]
    L.TSHip_GptDestroy.argtypes = [vp]
    L.TSHip_GptSetWeight.argtypes = [vp, C.c_char_p, vp, C.c_int, C.POINTER(C.c_int64)]
    L.TSHip_GptFinalize.argtypes = [vp]
    L.TSHip_GptReset.argtypes = [vp]
    L.TSHip_GptPrefill.argtypes = [vp, vp, C.c_int, C.c_int]
    L.TSHip_GptPrefillPadded.argtypes = [vp, vp, vp, C.c_int, C.c_int]
    L.TSHip_GptDecode.argtypes = [vp, vp, C.c_int]
    L.TSHip_GptSample.argtypes = [vp, C.c_int, C.c_float, C.c_float, vp, vp]
    L.TSHip_GptSetRepeatPenalty.argtypes = [vp, C.c_float]
    L.TSHip_GptSetBlockedTokens.argtypes = [vp, vp, C.c_int]
    L.TSHip_GptGenerateUntil.argtypes = [vp, C.c_int, C.c_int, C.c_int, C.c_float, C.c_float, vp, vp, C.POINTER(C.c_int), C.POINTER(C.c_float)]
    L.TSHip_GptGenerate.argtypes = [vp, C.c_int, C.c_int, C.c_float, C.c_float, vp, vp, C.POINTER(C.c_float)]
    L.TSHip_GptBeamPick.argtypes = [vp, C.c_int, C.c_int, C.c_float, C.c_float, vp, vp, vp]
    L.TSHip_GptReorderRows.argtypes = [vp, vp, C.c_int]
    L.TSHip_BeamTopN.argtypes = [vp, C.c_int, C.c_int, vp, C.POINTER(C.c_int)]
    L.TSHip_GptGetLogits.argtypes = [vp, vp]
    L.TSHip_GptGetHidden.argtypes = [vp, vp]
    L.TSHip_GptGetSeqLen.argtypes = [vp, C.POINTER(C.c_int)]
    L.TSHip_GptGetKV.argtypes = [vp, C.c_int, C.c_int, vp]
    L.TSHip_GptSetKV.argtypes = [vp, C.c_int, C.c_int, vp, C.c_int, C.c_int]
    L.TSHip_GptSetSeqLen.argtypes = [vp, C.c_int, C.c_int]
    L.TSHip_GptSaveRows.argtypes = [vp, C.POINTER(vp)]
    L.TSHip_GptRestoreRows.argtypes = [vp, vp]
    L.TSHip_GptSnapshotInfo.argtypes = [vp, C.POINTER(C.c_int), C.POINTER(C.c_int), C.POINTER(C.c_int64)]
    L.TSHip_GptFreeSnapshot.argtypes = [vp]
    L.TSHip_GptGetMoeRouting.argtypes = [vp, C.c_int, vp, vp, vp]
    L.TSHip_GptProfileDecode.argtypes = [vp, vp, C.c_int, vp, vp, C.c_int, C.POINTER(C.c_int)]
    L.TSHip_GptProfileSymbols.argtypes = [vp, vp, C.c_int, C.c_int, C.POINTER(C.c_int)]
    L.TSHip_GptStepBytes.argtypes = [vp, C.c_int, C.POINTER(C.c_double), C.POINTER(C.c_double)]
    L.TSHip_Synchronize.argtypes = []
    _proto_done = True


def _ptr(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


class KvSnapshot:
    """Handle of a TSHipGptSnapshot (device memory, freed by close())."""

    def __init__(self, h):
        self.h = h

    def info(self):
        b, n, nb = C.c_int(0), C.c_int(0), C.c_int64(0)
        check(lib().TSHip_GptSnapshotInfo(self.h, C.byref(b), C.byref(n), C.byref(nb)))
        return b.value, n.value, nb.value

    def close(self):
        if getattr(self, "h", None):
            lib().TSHip_GptFreeSnapshot(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class KvStore:
    """The reference's text-keyed cache of parked conversations (GPT.cs:153-173: MemoryCache, sliding expiry of ten
    minutes), holding device snapshots instead of host tensors.  `clock` is injectable for tests."""

    def __init__(self, ttl_seconds=600.0, clock=None):
        import time
        self.ttl, self.clock, self.items = float(ttl_seconds), clock or time.monotonic, {}

    def _expire(self):
        now = self.clock()
        for key in [k for k, (_, t) in self.items.items() if now - t > self.ttl]:
            self.items.pop(key)[0].close()

    def put(self, key, snap):
        self._expire()
        old = self.items.pop(key, None)
        if old:
            old[0].close()
        self.items[key] = (snap, self.clock())

    def get(self, key):
        """The snapshot parked under `key` (its expiry slides), or None."""
        self._expire()
        hit = self.items.get(key)
        if hit is None:
            return None
        self.items[key] = (hit[0], self.clock())
        return hit[0]

    def remove(self, key):
        hit = self.items.pop(key, None)
        if hit:
            hit[0].close()

    def __len__(self):
        self._expire()
        return len(self.items)


class HipGpt:
    """One GPTDecoder replica on one GPU with a preallocated KV cache."""

    def __init__(self, cfg, weights, max_batch=None, max_seq_len=None, device=0):
        """cfg: dict (see seq2seqsharp_amd.synth); weights: dict or iterable of (name, float32 array)
        under the reference's saved parameter names."""
        _protos()
        L = lib()
        check(L.TSHip_Init(device))
        self.cfg = dict(cfg)
        self.max_batch = int(max_batch or cfg.get("batch", 1))
        self.max_seq_len = int(max_seq_len or (cfg.get("prompt", 16) + cfg.get("steps", 16) + 1))
        c = TSHipGptConfig(cfg["n_layers"], cfg["hidden"], cfg["n_heads"], cfg["n_kv_heads"], cfg["ffn_dim"], cfg["vocab"],
                           cfg["attn_type"], cfg["norm_type"], cfg["act"], cfg.get("n_experts", 1),
                           cfg.get("experts_per_token", 1), cfg.get("norm_eps", 1e-6), cfg.get("rope_base", 500000.0),
                           cfg.get("use_rope", 1), F16 if cfg.get("dtype", "f32") == "f16" else F32,
                           self.max_batch, self.max_seq_len, cfg.get("max_segments", 0), cfg.get("sep_token_id", 3))
        h = C.c_void_p()
        check(L.TSHip_GptCreate(C.byref(c), C.byref(h)))
        self.h = h
        items = weights.items() if hasattr(weights, "items") else weights
        for name, w in items:
            w = np.ascontiguousarray(w, dtype=np.float32)
            sizes = (C.c_int64 * w.ndim)(*w.shape)
            check(L.TSHip_GptSetWeight(self.h, name.encode(), _ptr(w), w.ndim, sizes))
        check(L.TSHip_GptFinalize(self.h))
        self.batch = 0

    @classmethod
    def from_model_file(cls, path, max_batch, max_seq_len, dtype=None, device=0):
        """A replica from a model file the reference saved (see seq2seqsharp_amd.model_file); returns (model, target vocabulary).
        dtype None keeps the file's storage type: Float16 files run in fp16, as the reference demands AMP for them
        (Models/Model.cs:267-270)."""
        from . import model_file
        cfg, weights, vocab = model_file.load_gpt(path, dtype)
        return cls(cfg, weights, max_batch=max_batch, max_seq_len=max_seq_len, device=device), vocab

    def close(self):
        if getattr(self, "h", None):
            lib().TSHip_GptDestroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def reset(self):
        check(lib().TSHip_GptReset(self.h))
        self.batch = 0

    def prefill(self, ids, lens=None):
        """ids [batch, len]; lens: original lengths of sequences that were padded to `len` with the END tag
        (BuildInTokens.PadSentences): the reference's masking for padded batches then applies."""
        ids = np.ascontiguousarray(ids, dtype=np.int32)
        B, T = ids.shape
        if lens is None:
            check(lib().TSHip_GptPrefill(self.h, _ptr(ids), B, T))
        else:
            lens = np.ascontiguousarray(lens, dtype=np.int32).reshape(-1)
            assert lens.size == B
            check(lib().TSHip_GptPrefillPadded(self.h, _ptr(ids), _ptr(lens), B, T))
        self.batch = B

    @staticmethod
    def pad_sentences(seqs, pad_id=0):
        """BuildInTokens.PadSentences (Corpus/BuildInTokens.cs:68-101): lists of token ids -> (ids [batch, longest] padded
        with `pad_id`, the END tag in the reference; original lengths)."""
        lens = np.array([len(s) for s in seqs], np.int32)
        out = np.full((len(seqs), int(lens.max())), pad_id, np.int32)
        for i, s in enumerate(seqs):
            out[i, :len(s)] = s
        return out, lens

    def decode(self, ids):
        ids = np.ascontiguousarray(ids, dtype=np.int32).reshape(-1)
        check(lib().TSHip_GptDecode(self.h, _ptr(ids), ids.size))
        self.batch = ids.size

    def set_blocked_tokens(self, ids):
        """DecodingOptions.BlockedTokens: tokens that are never chosen (Decoder.cs:745-753); an empty list clears them."""
        ids = np.ascontiguousarray(ids, dtype=np.int32).reshape(-1)
        check(lib().TSHip_GptSetBlockedTokens(self.h, _ptr(ids) if ids.size else None, int(ids.size)))

    def set_repeat_penalty(self, repeat_penalty):
        """DecodingOptions.RepeatPenalty for top-p sampling (the reference's default is 2.0); set before the prompt is fed."""
        check(lib().TSHip_GptSetRepeatPenalty(self.h, float(repeat_penalty)))

    def sample(self, mode=GREEDY, top_p=0.0, temperature=1.0, uniforms=None):
        out = np.empty((self.batch,), np.int32)
        u = None if uniforms is None else np.ascontiguousarray(uniforms, dtype=np.float32)
        check(lib().TSHip_GptSample(self.h, mode, top_p, temperature, _ptr(u), _ptr(out)))
        return out

    def generate(self, n_steps, mode=GREEDY, top_p=0.0, temperature=1.0, uniforms=None):
        """Returns (ids [n_steps, batch], device milliseconds of the loop)."""
        out = np.empty((n_steps, self.batch), np.int32)
        u = None if uniforms is None else np.ascontiguousarray(uniforms, dtype=np.float32)
        ms = C.c_float(0.0)
        check(lib().TSHip_GptGenerate(self.h, n_steps, mode, top_p, temperature, _ptr(u), _ptr(out), C.byref(ms)))
        return out, ms.value

    def generate_until(self, max_steps, eos_id, mode=GREEDY, top_p=0.0, temperature=1.0, uniforms=None):
        """The loop of GPT.RunForwardOnSingleDevice with its stop rule: ends after the first step at which every sequence's
        new token is `eos_id` (Decoder.AreAllSentsCompleted).  Returns (ids [steps_done, batch], device milliseconds)."""
        out = np.empty((max_steps, self.batch), np.int32)
        u = None if uniforms is None else np.ascontiguousarray(uniforms, dtype=np.float32)
        ms = C.c_float(0.0)
        done = C.c_int(0)
        check(lib().TSHip_GptGenerateUntil(self.h, max_steps, eos_id, mode, top_p, temperature, _ptr(u), _ptr(out), C.byref(done), C.byref(ms)))
        return out[:done.value], ms.value

    def beam_pick(self, n_picks, mode=GREEDY, top_p=0.0, temperature=1.0, uniforms=None):
        """n_picks picks per cached row from the current logits, the reference's way (pick, zero the picked probability,
        pick again: Decoder.cs:756-792).  Returns (ids [n_picks, batch], log of the picked probabilities [n_picks, batch])."""
        ids = np.empty((n_picks, self.batch), np.int32)
        logp = np.empty((n_picks, self.batch), np.float32)
        u = None if uniforms is None else np.ascontiguousarray(uniforms, dtype=np.float32)
        check(lib().TSHip_GptBeamPick(self.h, n_picks, mode, top_p, temperature, _ptr(u), _ptr(ids), _ptr(logp)))
        return ids, logp

    def reorder_rows(self, src_rows):
        """Row i of the new batch continues old row src_rows[i] (KV cache and token history are gathered)."""
        src = np.ascontiguousarray(src_rows, dtype=np.int32).reshape(-1)
        check(lib().TSHip_GptReorderRows(self.h, _ptr(src), int(src.size)))
        self.batch = int(src.size)

    def beam_search(self, prompts, beam_size, max_len, eos_id=0, mode=GREEDY, top_p=0.0, temperature=1.0, uniforms=None, lens=None):
        """The loop of GPT.RunForwardOnSingleDevice for BeamSearchSize > 1 (Applications/GPT.cs:264-302): every step makes
        beam_size picks from every hypothesis, scores them (previous score - log p; a hypothesis starts at 1.0,
        Utils/BeamSearch.cs:29), keeps the beam_size best per sequence (BeamSearch.GetTopNBSS) and stops when every
        hypothesis ends in the END tag or at max_len tokens.  prompts [batch, len].  uniforms [steps, beam_size picks,
        beam_size * batch rows] for top-p.  Returns (hypotheses [batch][beam] as token lists, scores [batch][beam]),
        beams in the reference's order."""
        prompts = np.ascontiguousarray(prompts, dtype=np.int32)
        B, T0 = prompts.shape
        assert beam_size >= 1 and B * beam_size <= self.max_batch, "max_batch must hold batch x beam_size rows"
        self.reset()
        self.prefill(prompts, lens=lens)
        # rows are hypotheses in beam-major order: row j * B + b = hypothesis j of sequence b
        hyp = [[list(map(int, prompts[b])) for b in range(B)]]
        score = [[np.float32(1.0) for _ in range(B)]]
        step = 0
        for _ in range(T0, max_len):
            nb = len(hyp)
            u = None if uniforms is None else np.ascontiguousarray(uniforms[step][:, :nb * B])
            ids, logp = self.beam_pick(beam_size, mode, top_p, temperature, u)
            new_hyp = [[None] * B for _ in range(beam_size)]
            new_score = [[None] * B for _ in range(beam_size)]
            src = np.zeros((beam_size, B), np.int32)
            tok = np.zeros((beam_size, B), np.int32)
            for b in range(B):
                cand = []                                   # (score, parent beam, token) in the reference's order: beams outer, picks inner
                for j in range(nb):
                    for i in range(beam_size):
                        r = j * B + b
                        cand.append((np.float32(score[j][b] + np.float32(-1.0) * logp[i, r]), j, int(ids[i, r])))
                if beam_size > 1:
                    sc = np.array([c[0] for c in cand], np.float32)
                    kept = np.empty((beam_size,), np.int32)
                    nk = C.c_int(0)
                    check(lib().TSHip_BeamTopN(_ptr(sc), len(cand), beam_size, _ptr(kept), C.byref(nk)))
                    order = [int(k) for k in kept[:nk.value]]
                else:
                    order = [0]
                for jn, k in enumerate(order):
                    s_, j, t = cand[k]
                    new_hyp[jn][b] = hyp[j][b] + [t]
                    new_score[jn][b] = s_
                    src[jn, b] = j * B + b
                    tok[jn, b] = t
            hyp, score = new_hyp, new_score
            step += 1
            done = all(h[-1] == eos_id for beam in hyp for h in beam)
            if done or len(hyp[0][0]) >= max_len:
                break
            self.reorder_rows(src.reshape(-1))
            self.decode(tok.reshape(-1))
        out_h = [[hyp[j][b] for j in range(len(hyp))] for b in range(B)]
        out_s = [[float(score[j][b]) for j in range(len(hyp))] for b in range(B)]
        return out_h, out_s

    def logits(self):
        out = np.empty((self.batch, self.cfg["vocab"]), np.float32)
        check(lib().TSHip_GptGetLogits(self.h, _ptr(out)))
        return out

    def hidden(self):
        out = np.empty((self.batch, self.cfg["hidden"]), np.float32)
        check(lib().TSHip_GptGetHidden(self.h, _ptr(out)))
        return out

    def seq_len(self):
        n = C.c_int(0)
        check(lib().TSHip_GptGetSeqLen(self.h, C.byref(n)))
        return n.value

    def get_kv(self, layer, which):
        """[batch, n_kv_heads, len, head_dim] float32; which = 0 keys (after RoPE), 1 values."""
        T = self.seq_len()
        d = self.cfg["hidden"] // self.cfg["n_heads"]
        out = np.empty((self.batch, self.cfg["n_kv_heads"], T, d), np.float32)
        check(lib().TSHip_GptGetKV(self.h, layer, which, _ptr(out)))
        return out

    def set_kv(self, layer, which, data):
        data = np.ascontiguousarray(data, dtype=np.float32)
        B, G, T, d = data.shape
        check(lib().TSHip_GptSetKV(self.h, layer, which, _ptr(data), B, T))

    def set_seq_len(self, batch, length):
        check(lib().TSHip_GptSetSeqLen(self.h, batch, length))
        self.batch = batch

    def save_rows(self):
        """TSHip_GptSaveRows: the current sequences' cache rows, last logits and token history, copied device to device."""
        h = C.c_void_p()
        check(lib().TSHip_GptSaveRows(self.h, C.byref(h)))
        return KvSnapshot(h)

    def restore_rows(self, snap):
        """TSHip_GptRestoreRows: make a saved set the current sequences again; decoding continues bit for bit."""
        check(lib().TSHip_GptRestoreRows(self.h, snap.h))
        self.batch = snap.info()[0]

    def moe_routing(self, layer):
        k, E = self.cfg["experts_per_token"], self.cfg["n_experts"]
        ti = np.empty((self.batch, k), np.float32)
        tv = np.empty((self.batch, k), np.float32)
        pr = np.empty((self.batch, E), np.float32)
        check(lib().TSHip_GptGetMoeRouting(self.h, layer, _ptr(ti), _ptr(tv), _ptr(pr)))
        return ti, tv, pr

    def profile_decode(self, ids, n_max=4096):
        """One decode step with device events around every kernel: list of (kernel name, milliseconds)."""
        ids = np.ascontiguousarray(ids, dtype=np.int32).reshape(-1)
        names = C.create_string_buffer(48 * n_max)
        ms = np.zeros((n_max,), np.float32)
        n = C.c_int(0)
        check(lib().TSHip_GptProfileDecode(self.h, _ptr(ids), ids.size, C.cast(names, C.c_void_p), _ptr(ms), n_max, C.byref(n)))
        self.batch = ids.size
        out = []
        for i in range(min(n.value, n_max)):
            out.append((names.raw[i * 48:(i + 1) * 48].split(b"\0", 1)[0].decode(), float(ms[i])))
        return out

    def profile_symbols(self, n_max=4096, stride=256):
        """Launched kernel symbols of the step profile_decode timed last, in launch order."""
        buf = C.create_string_buffer(stride * n_max)
        n = C.c_int(0)
        check(lib().TSHip_GptProfileSymbols(self.h, C.cast(buf, C.c_void_p), stride, n_max, C.byref(n)))
        return [buf.raw[i * stride:(i + 1) * stride].split(b"\0", 1)[0].decode() for i in range(min(n.value, n_max))]

    def step_bytes(self, batch=None):
        """Algorithmic bytes of one decode step at the current length: (weight bytes, KV bytes)."""
        w, k = C.c_double(0), C.c_double(0)
        check(lib().TSHip_GptStepBytes(self.h, batch or self.batch, C.byref(w), C.byref(k)))
        return w.value, k.value

