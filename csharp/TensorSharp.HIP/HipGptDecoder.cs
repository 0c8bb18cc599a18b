// Managed wrapper of the fused GPTDecoder path (TSHip_Gpt*): what GPT.RunForwardOnSingleDevice hands a whole decoding job
// to when ProcessorType is HIP, instead of replaying Decoder.GPTDecode op by op (Applications/GPT.cs:212-335,
// Applications/Decoder.cs:648-794).  Weights go in under their saved names (Model.GetWeights names,
// Models/Model.cs:178-380); token ids come back.
using System;
using System.Collections.Generic;
using System.Linq;

namespace TensorSharp.HIP
{
    public enum HipSampling { Greedy = 0, TopP = 1 }

    public sealed class HipGptDecoder : IDisposable
    {
        private IntPtr handle;
        private readonly TSHipGptConfig config;
        private int batch;

        public HipGptDecoder(TSHipGptConfig cfg)
        {
            config = cfg;
            HipNative.Check(HipNative.TSHip_GptCreate(cfg, out handle), "GptCreate");
        }

        public TSHipGptConfig Config => config;

        /// <summary>One parameter under its saved name, e.g. "GPTDecoder.SelfAttn_0.Q" or "TgtEmbeddings"; call Finish after the last one.</summary>
        public void SetWeight(string name, float[] data, long[] sizes) =>
            HipNative.Check(HipNative.TSHip_GptSetWeight(handle, name, data, sizes.Length, sizes), "GptSetWeight");

        public void Finish() => HipNative.Check(HipNative.TSHip_GptFinalize(handle), "GptFinalize");

        public void Reset() { HipNative.Check(HipNative.TSHip_GptReset(handle), "GptReset"); batch = 0; }

        /// <summary>DecodingOptions.RepeatPenalty (before the prompt is fed) and DecodingOptions.BlockedTokens.</summary>
        public void SetRepeatPenalty(float penalty) => HipNative.Check(HipNative.TSHip_GptSetRepeatPenalty(handle, penalty), "GptSetRepeatPenalty");
        public void SetBlockedTokens(IReadOnlyList<int> ids) => HipNative.Check(HipNative.TSHip_GptSetBlockedTokens(handle, ids?.ToArray() ?? Array.Empty<int>(), ids?.Count ?? 0), "GptSetBlockedTokens");

        /// <summary>Prompts of one length, or (paddingAllowed) of different lengths padded with `padId` as BuildInTokens.PadSentences pads them.</summary>
        public void Prefill(List<List<int>> prompts, bool paddingAllowed = false, int padId = 0)
        {
            int b = prompts.Count, len = prompts.Max(p => p.Count);
            int[] ids = new int[b * len];
            int[] lens = new int[b];
            for (int i = 0; i < b; i++)
            {
                lens[i] = prompts[i].Count;
                for (int j = 0; j < len; j++) ids[i * len + j] = j < lens[i] ? prompts[i][j] : padId;
            }
            if (paddingAllowed && b > 1) HipNative.Check(HipNative.TSHip_GptPrefillPadded(handle, ids, lens, b, len), "GptPrefillPadded");
            else
            {
                if (lens.Any(l => l != len)) throw new ArgumentException("prompts differ in length; allow padding");
                HipNative.Check(HipNative.TSHip_GptPrefill(handle, ids, b, len), "GptPrefill");
            }
            batch = b;
        }

        public void Decode(int[] tokens)
        {
            HipNative.Check(HipNative.TSHip_GptDecode(handle, tokens, tokens.Length), "GptDecode");
            batch = tokens.Length;
        }

        public int[] Sample(HipSampling mode = HipSampling.Greedy, float topP = 0.0f, float temperature = 1.0f, float[] uniforms = null)
        {
            int[] ids = new int[batch];
            HipNative.Check(HipNative.TSHip_GptSample(handle, (int)mode, topP, temperature, uniforms, ids), "GptSample");
            return ids;
        }

        /// <summary>steps x batch token ids; the loop runs on the device (one captured graph per step).</summary>
        public int[] Generate(int steps, HipSampling mode = HipSampling.Greedy, float topP = 0.0f, float temperature = 1.0f, float[] uniforms = null)
        {
            int[] ids = new int[steps * batch];
            HipNative.Check(HipNative.TSHip_GptGenerate(handle, steps, (int)mode, topP, temperature, uniforms, ids, out _), "GptGenerate");
            return ids;
        }

        /// <summary>The same loop with the reference's stop rule (every sequence's newest token is the END tag, Decoder.cs:207-221).</summary>
        public int[] GenerateUntil(int maxSteps, int eosId, out int stepsDone, HipSampling mode = HipSampling.Greedy, float topP = 0.0f, float temperature = 1.0f, float[] uniforms = null)
        {
            int[] ids = new int[maxSteps * batch];
            HipNative.Check(HipNative.TSHip_GptGenerateUntil(handle, maxSteps, eosId, (int)mode, topP, temperature, uniforms, ids, out stepsDone, out _), "GptGenerateUntil");
            return ids;
        }

        /// <summary>Beam search as GPT.RunForwardOnSingleDevice runs it for BeamSearchSize > 1 (GPT.cs:264-302): hypotheses are rows of the
        /// cached batch; picks and scores come from the device, pruning is BeamSearch.GetTopNBSS.  maxBatch must hold batch x beamSize rows.</summary>
        public List<List<(List<int> ids, float score)>> BeamSearch(List<List<int>> prompts, int beamSize, int maxLen, int eosId = 0)
        {
            Reset();
            Prefill(prompts);
            int B = prompts.Count;
            var hyp = new List<List<(List<int> ids, float score)>> { prompts.Select(p => (new List<int>(p), 1.0f)).ToList() };     // beam-major; Score starts at 1.0f (BeamSearch.cs:29)
            for (int i = prompts[0].Count; i < maxLen; i++)
            {
                int nb = hyp.Count, rows = nb * B;
                int[] ids = new int[beamSize * rows];
                float[] logp = new float[beamSize * rows];
                HipNative.Check(HipNative.TSHip_GptBeamPick(handle, beamSize, (int)HipSampling.Greedy, 0.0f, 1.0f, null, ids, logp), "GptBeamPick");
                var next = Enumerable.Range(0, beamSize).Select(_ => new (List<int>, float)[B]).ToList();
                int[] src = new int[beamSize * B], tok = new int[beamSize * B];
                for (int b = 0; b < B; b++)
                {
                    var cand = new List<(float score, int parent, int token)>();
                    for (int j = 0; j < nb; j++)
                        for (int p = 0; p < beamSize; p++)
                        {
                            int r = j * B + b;
                            cand.Add((hyp[j][b].score + -1.0f * logp[p * rows + r], j, ids[p * rows + r]));
                        }
                    int[] kept = new int[beamSize];
                    HipNative.Check(HipNative.TSHip_BeamTopN(cand.Select(c => c.score).ToArray(), cand.Count, beamSize, kept, out int nKept), "BeamTopN");
                    for (int jn = 0; jn < nKept; jn++)
                    {
                        var c = cand[kept[jn]];
                        var seq = new List<int>(hyp[c.parent][b].ids) { c.token };
                        next[jn][b] = (seq, c.score);
                        src[jn * B + b] = c.parent * B + b;
                        tok[jn * B + b] = c.token;
                    }
                }
                hyp = next.Select(a => a.ToList()).ToList();
                bool done = hyp.All(beam => beam.All(h => h.ids[h.ids.Count - 1] == eosId));
                if (done || i + 1 >= maxLen) break;
                HipNative.Check(HipNative.TSHip_GptReorderRows(handle, src, beamSize * B), "GptReorderRows");
                Decode(tok);
            }
            return Enumerable.Range(0, B).Select(b => hyp.Select(beam => beam[b]).ToList()).ToList();
        }

        // ---- parked conversations: what GPT.cs keeps in its MemoryCache keyed by the generated text (GPT.cs:153-173, 236-247,
        //      312-328), as device snapshots: no host round trip, the cache's own layout ----
        private readonly Dictionary<string, (IntPtr snapshot, DateTime lastUse)> parked = new Dictionary<string, (IntPtr, DateTime)>();
        public TimeSpan ParkedExpiry { get; set; } = TimeSpan.FromMinutes(10);      // the reference's sliding expiration

        private void DropExpired()
        {
            DateTime now = DateTime.UtcNow;
            foreach (string key in parked.Where(kv => now - kv.Value.lastUse > ParkedExpiry).Select(kv => kv.Key).ToList())
            {
                HipNative.TSHip_GptFreeSnapshot(parked[key].snapshot);
                parked.Remove(key);
            }
        }

        /// <summary>Park the current sequences under `key` (the generated text so far, as the reference keys its cache).</summary>
        public void Park(string key)
        {
            DropExpired();
            HipNative.Check(HipNative.TSHip_GptSaveRows(handle, out IntPtr snap), "GptSaveRows");
            if (parked.TryGetValue(key, out var old)) HipNative.TSHip_GptFreeSnapshot(old.snapshot);
            parked[key] = (snap, DateTime.UtcNow);
        }

        /// <summary>Make the sequences parked under `key` current again; false when nothing (or nothing fresh enough) is parked there.</summary>
        public bool Resume(string key)
        {
            DropExpired();
            if (!parked.TryGetValue(key, out var hit)) return false;
            HipNative.Check(HipNative.TSHip_GptRestoreRows(handle, hit.snapshot), "GptRestoreRows");
            HipNative.Check(HipNative.TSHip_GptSnapshotInfo(hit.snapshot, out int rows, out int _, out long _), "GptSnapshotInfo");
            batch = rows;
            parked[key] = (hit.snapshot, DateTime.UtcNow);
            return true;
        }

        public int ParkedCount { get { DropExpired(); return parked.Count; } }

        // ---- inspection (parity tests, benchmarks) ----
        public float[] Logits() { float[] o = new float[batch * config.Vocab]; HipNative.Check(HipNative.TSHip_GptGetLogits(handle, o), "GptGetLogits"); return o; }
        public float[] Hidden() { float[] o = new float[batch * config.Hidden]; HipNative.Check(HipNative.TSHip_GptGetHidden(handle, o), "GptGetHidden"); return o; }
        public int SequenceLength() { HipNative.Check(HipNative.TSHip_GptGetSeqLen(handle, out int n), "GptGetSeqLen"); return n; }
        public float[] GetKV(int layer, bool values)
        {
            int d = config.Hidden / config.NHeads;
            float[] o = new float[(long)batch * config.NKvHeads * SequenceLength() * d];
            HipNative.Check(HipNative.TSHip_GptGetKV(handle, layer, values ? 1 : 0, o), "GptGetKV");
            return o;
        }
        public void SetKV(int layer, bool values, float[] data, int rows, int len) => HipNative.Check(HipNative.TSHip_GptSetKV(handle, layer, values ? 1 : 0, data, rows, len), "GptSetKV");
        public void SetSequenceLength(int rows, int len) { HipNative.Check(HipNative.TSHip_GptSetSeqLen(handle, rows, len), "GptSetSeqLen"); batch = rows; }
        public (float[] topIdx, float[] topVal, float[] probs) MoeRouting(int layer)
        {
            float[] ti = new float[batch * config.ExpertsPerToken], tv = new float[batch * config.ExpertsPerToken], pr = new float[batch * config.NExperts];
            HipNative.Check(HipNative.TSHip_GptGetMoeRouting(handle, layer, ti, tv, pr), "GptGetMoeRouting");
            return (ti, tv, pr);
        }
        public List<(string kernel, float ms)> ProfileDecode(int[] tokens, int maxKernels = 4096)
        {
            byte[] names = new byte[48 * maxKernels];
            float[] ms = new float[maxKernels];
            HipNative.Check(HipNative.TSHip_GptProfileDecode(handle, tokens, tokens.Length, names, ms, maxKernels, out int n), "GptProfileDecode");
            var r = new List<(string, float)>();
            for (int i = 0; i < Math.Min(n, maxKernels); i++)
            {
                int end = Array.IndexOf(names, (byte)0, i * 48, 48);
                r.Add((System.Text.Encoding.ASCII.GetString(names, i * 48, (end < 0 ? (i + 1) * 48 : end) - i * 48), ms[i]));
            }
            batch = tokens.Length;
            return r;
        }
        public (double weightBytes, double kvBytes) StepBytes()
        {
            HipNative.Check(HipNative.TSHip_GptStepBytes(handle, batch, out double w, out double k), "GptStepBytes");
            return (w, k);
        }

        public void Dispose()
        {
            foreach (var kv in parked) HipNative.TSHip_GptFreeSnapshot(kv.Value.snapshot);
            parked.Clear();
            if (handle != IntPtr.Zero) { HipNative.TSHip_GptDestroy(handle); handle = IntPtr.Zero; }
        }
    }
}
