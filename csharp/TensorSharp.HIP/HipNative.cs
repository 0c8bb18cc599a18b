// P/Invoke surface of libtship.so: one [DllImport] per function declared in include/tship.h, same conventions as
// TensorSharp.GGML/GgmlNative.cs:161-533 (cdecl, int 1/0, per-thread last error).  Tensor views travel by reference
// (`in TSHipTensor` marshals as `const TSHipTensor*`).
using System;
using System.IO;
using System.Reflection;
using System.Runtime.InteropServices;

namespace TensorSharp.HIP
{
    [StructLayout(LayoutKind.Sequential)]
    internal unsafe struct TSHipTensor            // include/tship.h: TSHipTensor
    {
        public IntPtr Data;                       // storage pointer + StorageOffset * element size (a device address)
        public int DType;                         // DType.Float32 = 0, DType.Float16 = 1 (TensorSharp/DType.cs:6-13)
        public int NDim;
        public fixed long Sizes[6];
        public fixed long Strides[6];             // in elements; 0 for expanded dimensions

        public static TSHipTensor From(Tensor t)
        {
            if (t.DimensionCount < 1 || t.DimensionCount > 6) throw new NotSupportedException("The HIP backend supports tensors of 1 to 6 dimensions.");
            if (t.ElementType != TensorSharp.DType.Float32 && t.ElementType != TensorSharp.DType.Float16) throw new NotSupportedException("The HIP backend supports Float32 and Float16 tensors.");
            var v = new TSHipTensor { DType = t.ElementType == TensorSharp.DType.Float16 ? 1 : 0, NDim = t.DimensionCount };
            v.Data = ((HipStorage)t.Storage).DevicePtrAtElement(t.StorageOffset);
            for (int i = 0; i < t.DimensionCount; i++) { v.Sizes[i] = t.Sizes[i]; v.Strides[i] = t.Strides[i]; }
            return v;
        }
    }

    [StructLayout(LayoutKind.Sequential)]
    public struct TSHipGptConfig                  // include/tship.h: TSHipGptConfig
    {
        public int NLayers, Hidden, NHeads, NKvHeads, FfnDim, Vocab;
        public int AttnType;                      // 0 MultiHeadAttention, 1 GroupQueryAttention
        public int NormType;                      // 0 RMSNorm, 1 LayerNorm
        public int Act;                           // 0 ReLU, 1 SiLU, 2 LeakyReLU, 3 SwiGLU (the reference's gate), 4 gated with SiLU
        public int NExperts, ExpertsPerToken;
        public float NormEps, RopeBase;
        public int UseRope;
        public int DType;
        public int MaxBatch, MaxSeqLen;
        public int MaxSegments;                   // IModel.MaxSegmentNum when EnableSegmentEmbeddings, else 0 (table "SegmentEmbedding")
        public int SepTokenId;                    // the vocabulary's index of BuildInTokens.SEP ("[SEP]")
    }

    internal static class HipNative
    {
        private const string Dll = "tship";
        private const CallingConvention CC = CallingConvention.Cdecl;

        static HipNative()
        {
            // probe the application directory and the assembly directory, as GgmlNative.ImportResolver does (GgmlNative.cs:481-524)
            NativeLibrary.SetDllImportResolver(typeof(HipNative).Assembly, (name, asm, path) =>
            {
                if (name != Dll) return IntPtr.Zero;
                foreach (string dir in new[] { AppContext.BaseDirectory, Path.GetDirectoryName(asm.Location) ?? "." })
                {
                    string candidate = Path.Combine(dir, "libtship.so");
                    if (File.Exists(candidate) && NativeLibrary.TryLoad(candidate, out IntPtr h)) return h;
                }
                return IntPtr.Zero;
            });
        }

        // ---- runtime ----
        [DllImport(Dll, CallingConvention = CC)] private static extern IntPtr TSHip_GetLastError();
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_GetDeviceCount(out int count);
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_Init(int deviceId);
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_Malloc(out IntPtr ptr, UIntPtr bytes);
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_Free(IntPtr ptr);
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_PoolTrim();
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_GetPoolStats(out UIntPtr deviceAllocations, out UIntPtr bytesInUse, out UIntPtr bytesCached);
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_MemcpyH2D(IntPtr dst, IntPtr src, UIntPtr bytes);
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_MemcpyD2H(IntPtr dst, IntPtr src, UIntPtr bytes);
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_MemcpyD2D(IntPtr dst, IntPtr src, UIntPtr bytes);
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_Memset(IntPtr dst, int value, UIntPtr bytes);
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_Synchronize();
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_GetMemInfo(out UIntPtr free, out UIntPtr total);

        // ---- per-op surface ----
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_Copy(in TSHipTensor result, in TSHipTensor src);
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_Fill(in TSHipTensor result, float value);
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_Addmm(in TSHipTensor result, float beta, in TSHipTensor src, float alpha, in TSHipTensor m1, in TSHipTensor m2);
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_AddmmBatch(in TSHipTensor result, float beta, in TSHipTensor src, float alpha, in TSHipTensor m1, in TSHipTensor m2);
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_IndexSelect(in TSHipTensor result, in TSHipTensor src, in TSHipTensor indice, int isAdd);
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_IndexSelectGrad(in TSHipTensor grad, in TSHipTensor adj, in TSHipTensor indice);
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_RoPE(in TSHipTensor result, in TSHipTensor src, int seqLen, int rowOffset);
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_RoPEEx(in TSHipTensor result, in TSHipTensor src, int seqLen, int rowOffset, float ropeBase);
        [DllImport(Dll, CallingConvention = CC)] internal static extern unsafe int TSHip_RMSNorm(in TSHipTensor result, in TSHipTensor src, in TSHipTensor gamma, TSHipTensor* betaOrNull, float eps);
        [DllImport(Dll, CallingConvention = CC)] internal static extern unsafe int TSHip_LayerNorm(in TSHipTensor result, in TSHipTensor src, in TSHipTensor gamma, TSHipTensor* betaOrNull, float eps);
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_Softmax(in TSHipTensor result, in TSHipTensor src);
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_Argmax(in TSHipTensor result, in TSHipTensor src, int dim);
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_TopK(in TSHipTensor outVal, in TSHipTensor outIdx, in TSHipTensor src, int k);
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_BinaryTensor(int op, in TSHipTensor result, in TSHipTensor lhs, in TSHipTensor rhs);
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_BinaryScalar(int op, in TSHipTensor result, in TSHipTensor src, float scalar);
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_Unary(int op, in TSHipTensor result, in TSHipTensor src);
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_BuildTriMask(in TSHipTensor result, float value, float maskedValue);
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_BuildSelfTriMask(in TSHipTensor result, in TSHipTensor originalLengths, int paddedSeqLen, float value, float maskedValue);
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_Gather(in TSHipTensor result, in TSHipTensor src, int dim, in TSHipTensor indices);
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_ScatterFill(in TSHipTensor result, float value, int dim, in TSHipTensor indices);
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_IsCorrupted(in TSHipTensor src, out int corrupted);
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_TopPSample(in TSHipTensor result, in TSHipTensor probs, in TSHipTensor uniforms, float topP);
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_TopPSampleNoAlloc(in TSHipTensor result, in TSHipTensor probs, in TSHipTensor uniforms, float topP);
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_TopPSampleEx(in TSHipTensor result, in TSHipTensor probs, in TSHipTensor uniforms, float topP,
            float repeatPenalty, int[] seqs, int[] seqLens, int seqLd);

        // ---- fused GPTDecoder path ----
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_GptCreate(in TSHipGptConfig cfg, out IntPtr model);
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_GptDestroy(IntPtr model);
        [DllImport(Dll, CallingConvention = CC, CharSet = CharSet.Ansi)] internal static extern int TSHip_GptSetWeight(IntPtr model, string name, float[] hostData, int ndim, long[] sizes);
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_GptFinalize(IntPtr model);
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_GptReset(IntPtr model);
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_GptPrefill(IntPtr model, int[] hostIds, int batch, int promptLen);
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_GptPrefillPadded(IntPtr model, int[] hostIds, int[] hostLens, int batch, int paddedLen);
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_GptDecode(IntPtr model, int[] hostIds, int batch);
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_GptSetRepeatPenalty(IntPtr model, float repeatPenalty);
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_GptSetBlockedTokens(IntPtr model, int[] ids, int n);
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_GptSample(IntPtr model, int mode, float topP, float temperature, float[] hostUniforms, int[] hostIdsOut);
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_GptGenerate(IntPtr model, int nSteps, int mode, float topP, float temperature, float[] hostUniforms, int[] hostIdsOut, out float elapsedMs);
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_GptGenerateUntil(IntPtr model, int maxSteps, int eosId, int mode, float topP, float temperature, float[] hostUniforms, int[] hostIdsOut, out int stepsDone, out float elapsedMs);
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_GptBeamPick(IntPtr model, int nPicks, int mode, float topP, float temperature, float[] hostUniforms, int[] hostIdsOut, float[] hostLogpOut);
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_GptReorderRows(IntPtr model, int[] hostSrcRows, int newBatch);
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_BeamTopN(float[] scores, int n, int topN, int[] kept, out int nKept);
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_GptGetLogits(IntPtr model, float[] hostOut);
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_GptGetHidden(IntPtr model, float[] hostOut);
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_GptGetSeqLen(IntPtr model, out int len);
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_GptGetKV(IntPtr model, int layer, int which, float[] hostOut);
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_GptSetKV(IntPtr model, int layer, int which, float[] hostIn, int batch, int len);
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_GptSetSeqLen(IntPtr model, int batch, int len);
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_GptSaveRows(IntPtr model, out IntPtr snapshot);
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_GptRestoreRows(IntPtr model, IntPtr snapshot);
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_GptSnapshotInfo(IntPtr snapshot, out int batch, out int len, out long deviceBytes);
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_GptFreeSnapshot(IntPtr snapshot);
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_GptGetMoeRouting(IntPtr model, int layer, float[] topIdx, float[] topVal, float[] probs);
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_GptProfileDecode(IntPtr model, int[] hostIds, int batch, byte[] names, float[] ms, int nMax, out int n);
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_GptProfileSymbols(IntPtr model, byte[] symbols, int stride, int nMax, out int n);
        [DllImport(Dll, CallingConvention = CC)] internal static extern int TSHip_GptStepBytes(IntPtr model, int batch, out double weightBytes, out double kvBytes);

        // ---- measurement aid ----

        internal static string LastError() => Marshal.PtrToStringAnsi(TSHip_GetLastError()) ?? string.Empty;

        internal static void Check(int rc, string op)      // GgmlNative.CheckResult, GgmlNative.cs:471-479
        {
            if (rc != 0) return;
            string msg = LastError();
            if (msg.StartsWith("out of device memory", StringComparison.Ordinal)) throw new OutOfMemoryException(msg);   // GPT.cs:269-288 catches this
            throw new InvalidOperationException($"Native HIP {op} failed. {msg}");
        }

        internal static void EnsureAvailable(int deviceId)  // cf. GgmlNative.EnsureAvailable, GgmlNative.cs:340-356
        {
            try { Check(TSHip_Init(deviceId), "init"); }
            catch (DllNotFoundException e) { throw new InvalidOperationException("libtship.so was not found beside the application. Build it with `python -m seq2seqsharp_amd.build` (hipcc, gfx950).", e); }
            catch (EntryPointNotFoundException e) { throw new InvalidOperationException("libtship.so is older than this assembly (missing export). Rebuild it.", e); }
        }
    }
}
