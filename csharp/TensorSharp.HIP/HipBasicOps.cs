// OpRegistry handlers of the HIP backend: same op names and parameter lists as the CPU backend
// (TensorSharp/Cpu/CpuBasicOps.cs, CpuIndexingOps.cs, CpuFillCopyOps.cs) and the CUDA backend, each a thin call into
// libtship.so.  Views with arbitrary strides (Expand = stride 0, Transpose, Narrow) go to the native side as they are.
// Handler selection: argument count equal and every Tensor argument on HipStorage (OpRegistryAttributes.cs:60-87).
using System;
using TensorSharp.Core;
using TensorSharp.Cpu;

namespace TensorSharp.HIP
{
    [OpsClass]
    public class HipBasicOps
    {
        // include/tship.h: TSHIP_ADD .. TSHIP_DIV, TSHIP_RELU .. TSHIP_ABS
        private const int Add_ = 0, Sub_ = 1, Mul_ = 2, Div_ = 3;
        private const int Relu_ = 0, SiLU_ = 1, LeakyReLU_ = 2, Exp_ = 3, Log_ = 4, Neg_ = 5, Sigmoid_ = 6, Tanh_ = 7, Sqrt_ = 8, Abs_ = 9;

        public HipBasicOps()
        {
        }

        private static TSHipTensor V(Tensor t) => TSHipTensor.From(t);

        // ---- copy: device to device, host to device, device to host (CudaBasicOps.cs:80-140) ----
        [RegisterOpArgCount("copy")]
        public void CopyHip([OpArgStorageType(typeof(HipStorage))] Tensor result, [OpArgStorageType(typeof(HipStorage))] Tensor src)
        {
            if (result.ElementCount() != src.ElementCount()) throw new InvalidOperationException("Tensors must have equal numbers of elements");
            if (src.DimensionCount == 0) return;
            HipNative.Check(HipNative.TSHip_Copy(V(result), V(src)), "copy");
        }

        [RegisterOpArgCount("copy")]
        public void CopyCpuToHip([OpArgStorageType(typeof(HipStorage))] Tensor result, [OpArgStorageType(typeof(CpuStorage))] Tensor src)
        {
            if (result.ElementCount() != src.ElementCount()) throw new InvalidOperationException("Tensors must have equal numbers of elements");
            if (src.DimensionCount == 0) return;
            Tensor hostSrc = src.IsContiguous() ? src : Ops.NewContiguous(src);
            try
            {
                if (result.IsContiguous() && result.ElementType == hostSrc.ElementType)
                {
                    result.Storage.CopyToStorage(result.StorageOffset, CpuNativeHelpers.GetBufferStart(hostSrc), hostSrc.ElementCount() * hostSrc.ElementType.Size());
                }
                else
                {
                    // stage on the device, then a strided / converting device copy
                    using Tensor staged = new Tensor(result.Allocator, hostSrc.ElementType, hostSrc.Sizes);
                    staged.Storage.CopyToStorage(0, CpuNativeHelpers.GetBufferStart(hostSrc), hostSrc.ElementCount() * hostSrc.ElementType.Size());
                    HipNative.Check(HipNative.TSHip_Copy(V(result), V(staged)), "copy");
                }
            }
            finally { if (!ReferenceEquals(hostSrc, src)) hostSrc.Dispose(); }
        }

        [RegisterOpArgCount("copy")]
        public void CopyHipToCpu([OpArgStorageType(typeof(CpuStorage))] Tensor result, [OpArgStorageType(typeof(HipStorage))] Tensor src)
        {
            if (result.ElementCount() != src.ElementCount()) throw new InvalidOperationException("Tensors must have equal numbers of elements");
            if (src.DimensionCount == 0) return;
            Tensor devSrc = src;
            if (!src.IsContiguous() || src.ElementType != result.ElementType)
            {
                devSrc = new Tensor(src.Allocator, result.ElementType, src.Sizes);
                HipNative.Check(HipNative.TSHip_Copy(V(devSrc), V(src)), "copy");
            }
            try
            {
                if (result.IsContiguous())
                {
                    devSrc.Storage.CopyFromStorage(CpuNativeHelpers.GetBufferStart(result), devSrc.StorageOffset, devSrc.ElementCount() * devSrc.ElementType.Size());
                }
                else
                {
                    using Tensor hostTmp = new Tensor(result.Allocator, result.ElementType, result.Sizes);
                    devSrc.Storage.CopyFromStorage(CpuNativeHelpers.GetBufferStart(hostTmp), devSrc.StorageOffset, devSrc.ElementCount() * devSrc.ElementType.Size());
                    Ops.Copy(result, hostTmp);
                }
            }
            finally { if (!ReferenceEquals(devSrc, src)) devSrc.Dispose(); }
        }

        [RegisterOpStorageType("fill", typeof(HipStorage))]
        public void Fill(Tensor result, float value)
        {
            HipNative.Check(HipNative.TSHip_Fill(V(result), value), "fill");
        }

        // ---- matrix products (CpuBasicOps.cs:49-184) ----
        [RegisterOpStorageType("addmm", typeof(HipStorage))]
        public static Tensor Addmm(Tensor result, float beta, Tensor src, float alpha, Tensor m1, Tensor m2)
        {
            if (src.ElementType != m1.ElementType || src.ElementType != m2.ElementType || (result != null && result.ElementType != src.ElementType))
                throw new InvalidOperationException("All tensors must have the same element type");
            if (result != null && !(result.Storage is HipStorage)) throw new ArgumentException("result must be a HIP tensor", nameof(result));
            if (src.DimensionCount != 2) throw new ArgumentException("src must be a matrix", nameof(src));
            if (m1.DimensionCount != 2) throw new ArgumentException("m1 must be a matrix", nameof(m1));
            if (m2.DimensionCount != 2) throw new ArgumentException("m2 must be a matrix", nameof(m2));
            if (src.Sizes[0] != m1.Sizes[0] || src.Sizes[1] != m2.Sizes[1] || m1.Sizes[1] != m2.Sizes[0]) throw new InvalidOperationException("Size mismatch");
            Tensor writeTarget = TensorResultBuilder.GetWriteTarget(result, src, false, src.Sizes);
            HipNative.Check(HipNative.TSHip_Addmm(V(writeTarget), beta, V(src), alpha, V(m1), V(m2)), "addmm");
            return writeTarget;
        }

        [RegisterOpStorageType("addmmbatch", typeof(HipStorage))]
        public static Tensor AddmmBatch(Tensor result, float beta, Tensor src, float alpha, Tensor m1, Tensor m2)
        {
            if (src.ElementType != m1.ElementType || src.ElementType != m2.ElementType || (result != null && result.ElementType != src.ElementType))
                throw new InvalidOperationException("All tensors must have the same element type");
            if (src.DimensionCount != 3) throw new ArgumentException("src must be a matrix", nameof(src));
            if (m1.DimensionCount != 3) throw new ArgumentException("m1 must be a matrix", nameof(m1));
            if (m2.DimensionCount != 3) throw new ArgumentException("m2 must be a matrix", nameof(m2));
            if (src.Sizes[1] != m1.Sizes[1] || src.Sizes[2] != m2.Sizes[2] || m1.Sizes[2] != m2.Sizes[1]) throw new InvalidOperationException("Size mismatch");
            Tensor writeTarget = TensorResultBuilder.GetWriteTarget(result, src, false, src.Sizes);
            HipNative.Check(HipNative.TSHip_AddmmBatch(V(writeTarget), beta, V(src), alpha, V(m1), V(m2)), "addmmbatch");
            return writeTarget;
        }

        // ---- indexing ----
        [RegisterOpStorageType("indexselect", typeof(HipStorage))]
        public Tensor IndexSelect(Tensor result, Tensor src, Tensor indice, bool isAdd)
        {
            Tensor writeTarget = TensorResultBuilder.GetWriteTarget(result, src, true, new long[] { indice.Sizes[0], src.Sizes[1] });
            HipNative.Check(HipNative.TSHip_IndexSelect(V(writeTarget), V(src), V(indice), isAdd ? 1 : 0), "indexselect");
            return writeTarget;
        }

        [RegisterOpStorageType("indexselectgrad", typeof(HipStorage))]
        public Tensor IndexSelectGrad(Tensor grad, Tensor adj, Tensor indice)
        {
            if (grad == null) throw new ArgumentNullException(nameof(grad));
            HipNative.Check(HipNative.TSHip_IndexSelectGrad(V(grad), V(adj), V(indice)), "indexselectgrad");
            return grad;
        }

        [RegisterOpStorageType("gather", typeof(HipStorage))]
        public Tensor Gather(Tensor result, Tensor src, int dim, Tensor indices)
        {
            if (result != null && result.DimensionCount != src.DimensionCount) throw new InvalidOperationException("result and src must have same number of dimensions");
            if (indices.DimensionCount != src.DimensionCount) throw new InvalidOperationException("src and indices must have same number of dimensions");
            if (result != null && !result.IsSameSizeAs(indices)) throw new InvalidOperationException("result and indices must be the same size");
            Tensor writeTarget = TensorResultBuilder.GetWriteTarget(result, indices.Allocator, src.ElementType, false, indices.Sizes);
            HipNative.Check(HipNative.TSHip_Gather(V(writeTarget), V(src), dim, V(indices)), "gather");
            return writeTarget;
        }

        [RegisterOpStorageType("scatter_fill", typeof(HipStorage))]
        public Tensor ScatterFill(Tensor result, float value, int dim, Tensor indices)
        {
            if (result == null) throw new ArgumentNullException(nameof(result));
            HipNative.Check(HipNative.TSHip_ScatterFill(V(result), value, dim, V(indices)), "scatter_fill");
            return result;
        }

        // ---- position embedding, norms, softmax ----
        [RegisterOpStorageType("rope", typeof(HipStorage))]
        public Tensor RoPE(Tensor result, Tensor src, int seqLen, int rowOffset)
        {
            Tensor writeTarget = TensorResultBuilder.GetWriteTarget(result, src, true, src.Sizes);
            HipNative.Check(HipNative.TSHip_RoPE(V(writeTarget), V(src), seqLen, rowOffset), "rope");
            return writeTarget;
        }

        [RegisterOpStorageType("rmsnorm", typeof(HipStorage))]
        public unsafe Tensor RMSNorm(Tensor result, Tensor src, Tensor gamma_, Tensor beta_, float eps)
        {
            Tensor writeTarget = TensorResultBuilder.GetWriteTarget(result, src, true, src.Sizes);
            TSHipTensor beta = beta_ != null ? V(beta_) : default;
            HipNative.Check(HipNative.TSHip_RMSNorm(V(writeTarget), V(src), V(gamma_), beta_ != null ? &beta : null, eps), "rmsnorm");
            return writeTarget;
        }

        [RegisterOpStorageType("layernorm", typeof(HipStorage))]
        public unsafe Tensor LayerNorm(Tensor result, Tensor src, Tensor gamma_, Tensor beta_, float eps)
        {
            Tensor writeTarget = TensorResultBuilder.GetWriteTarget(result, src, true, src.Sizes);
            TSHipTensor beta = beta_ != null ? V(beta_) : default;
            HipNative.Check(HipNative.TSHip_LayerNorm(V(writeTarget), V(src), V(gamma_), beta_ != null ? &beta : null, eps), "layernorm");
            return writeTarget;
        }

        [RegisterOpStorageType("softmax", typeof(HipStorage))]
        public Tensor Softmax(Tensor result, Tensor src)
        {
            Tensor writeTarget = TensorResultBuilder.GetWriteTarget(result, src, true, src.Sizes);
            HipNative.Check(HipNative.TSHip_Softmax(V(writeTarget), V(src)), "softmax");
            return writeTarget;
        }

        // ---- reductions that pick ----
        [RegisterOpStorageType("argmax", typeof(HipStorage))]
        public Tensor Argmax(Tensor result, Tensor src, int dimension)
        {
            if (dimension < 0 || dimension >= src.Sizes.Length) throw new ArgumentOutOfRangeException(nameof(dimension));
            long[] desiredSize = (long[])src.Sizes.Clone();
            desiredSize[dimension] = 1;
            Tensor writeTarget = TensorResultBuilder.GetWriteTarget(result, src, false, desiredSize);
            HipNative.Check(HipNative.TSHip_Argmax(V(writeTarget), V(src), dimension), "argmax");
            return writeTarget;
        }

        [RegisterOpStorageType("topK", typeof(HipStorage))]
        public void TopK(Tensor outVal, Tensor outIdx, Tensor src, int k)
        {
            HipNative.Check(HipNative.TSHip_TopK(V(outVal), V(outIdx), V(src), k), "topK");
        }

        // ---- element-wise families ----
        private static Tensor Binary(int op, string name, Tensor result, Tensor lhs, Tensor rhs)
        {
            Tensor writeTarget = TensorResultBuilder.GetWriteTarget(result, lhs, false, lhs.Sizes);
            HipNative.Check(HipNative.TSHip_BinaryTensor(op, V(writeTarget), V(lhs), V(rhs)), name);
            return writeTarget;
        }

        private static Tensor Scalar(int op, string name, Tensor result, Tensor lhs, float rhs)
        {
            Tensor writeTarget = TensorResultBuilder.GetWriteTarget(result, lhs, false, lhs.Sizes);
            HipNative.Check(HipNative.TSHip_BinaryScalar(op, V(writeTarget), V(lhs), rhs), name);
            return writeTarget;
        }

        private static Tensor Unary(int op, string name, Tensor result, Tensor src)
        {
            Tensor writeTarget = TensorResultBuilder.GetWriteTarget(result, src, false, src.Sizes);
            HipNative.Check(HipNative.TSHip_Unary(op, V(writeTarget), V(src)), name);
            return writeTarget;
        }

        [RegisterOpStorageType("addt", typeof(HipStorage))] public Tensor Add(Tensor result, Tensor lhs, Tensor rhs) => Binary(Add_, "addt", result, lhs, rhs);
        [RegisterOpStorageType("subt", typeof(HipStorage))] public Tensor Sub(Tensor result, Tensor lhs, Tensor rhs) => Binary(Sub_, "subt", result, lhs, rhs);
        [RegisterOpStorageType("mult", typeof(HipStorage))] public Tensor Mul(Tensor result, Tensor lhs, Tensor rhs) => Binary(Mul_, "mult", result, lhs, rhs);
        [RegisterOpStorageType("divt", typeof(HipStorage))] public Tensor Div(Tensor result, Tensor lhs, Tensor rhs) => Binary(Div_, "divt", result, lhs, rhs);
        [RegisterOpStorageType("addv", typeof(HipStorage))] public Tensor Add(Tensor result, Tensor lhs, float rhs) => Scalar(Add_, "addv", result, lhs, rhs);
        [RegisterOpStorageType("subv", typeof(HipStorage))] public Tensor Sub(Tensor result, Tensor lhs, float rhs) => Scalar(Sub_, "subv", result, lhs, rhs);
        [RegisterOpStorageType("mulv", typeof(HipStorage))] public Tensor Mul(Tensor result, Tensor lhs, float rhs) => Scalar(Mul_, "mulv", result, lhs, rhs);
        [RegisterOpStorageType("divv", typeof(HipStorage))] public Tensor Div(Tensor result, Tensor lhs, float rhs) => Scalar(Div_, "divv", result, lhs, rhs);

        [RegisterOpStorageType("relu", typeof(HipStorage))] public Tensor Relu(Tensor result, Tensor src) => Unary(Relu_, "relu", result, src);
        [RegisterOpStorageType("SiLU", typeof(HipStorage))] public Tensor SiLU(Tensor result, Tensor srcW) => Unary(SiLU_, "SiLU", result, srcW);
        [RegisterOpStorageType("LeakyReLU", typeof(HipStorage))] public Tensor LeakyReLU(Tensor result, Tensor srcW) => Unary(LeakyReLU_, "LeakyReLU", result, srcW);
        [RegisterOpStorageType("exp", typeof(HipStorage))] public Tensor Exp(Tensor result, Tensor src) => Unary(Exp_, "exp", result, src);
        [RegisterOpStorageType("log", typeof(HipStorage))] public Tensor Log(Tensor result, Tensor src) => Unary(Log_, "log", result, src);
        [RegisterOpStorageType("neg", typeof(HipStorage))] public Tensor Neg(Tensor result, Tensor src) => Unary(Neg_, "neg", result, src);
        [RegisterOpStorageType("sigmoid", typeof(HipStorage))] public Tensor Sigmoid(Tensor result, Tensor src) => Unary(Sigmoid_, "sigmoid", result, src);
        [RegisterOpStorageType("tanh", typeof(HipStorage))] public Tensor Tanh(Tensor result, Tensor src) => Unary(Tanh_, "tanh", result, src);
        [RegisterOpStorageType("sqrt", typeof(HipStorage))] public Tensor Sqrt(Tensor result, Tensor src) => Unary(Sqrt_, "sqrt", result, src);
        [RegisterOpStorageType("abs", typeof(HipStorage))] public Tensor Abs(Tensor result, Tensor src) => Unary(Abs_, "abs", result, src);

        // ---- precision changes (a copy between tensors of different element types converts, round to nearest even) ----
        [RegisterOpStorageType("float2half", typeof(HipStorage))]
        public Tensor Float2Half(Tensor result, Tensor src)
        {
            Tensor writeTarget = TensorResultBuilder.GetWriteTarget(result, src.Allocator, DType.Float16, false, src.Sizes);
            HipNative.Check(HipNative.TSHip_Copy(V(writeTarget), V(src)), "float2half");
            return writeTarget;
        }

        [RegisterOpStorageType("half2float", typeof(HipStorage))]
        public Tensor Half2Float(Tensor result, Tensor src)
        {
            Tensor writeTarget = TensorResultBuilder.GetWriteTarget(result, src.Allocator, DType.Float32, false, src.Sizes);
            HipNative.Check(HipNative.TSHip_Copy(V(writeTarget), V(src)), "half2float");
            return writeTarget;
        }

        // ---- masks, checks ----
        [RegisterOpStorageType("buildtrimask", typeof(HipStorage))]
        public Tensor BuildTriMask(Tensor result, float value, float maskedValue)
        {
            HipNative.Check(HipNative.TSHip_BuildTriMask(V(result), value, maskedValue), "buildtrimask");
            return result;
        }

        [RegisterOpStorageType("buildselftrimask", typeof(HipStorage))]
        public Tensor BuildSelfTriMask(Tensor result, Tensor originalLengths, int paddedSeqLen, float value, float maskedValue)
        {
            HipNative.Check(HipNative.TSHip_BuildSelfTriMask(V(result), V(originalLengths), paddedSeqLen, value, maskedValue), "buildselftrimask");
            return result;
        }

        [RegisterOpStorageType("iscorrupted", typeof(HipStorage))]
        public bool IsCorrupted(Tensor src)
        {
            HipNative.Check(HipNative.TSHip_IsCorrupted(V(src), out int corrupted), "iscorrupted");
            return corrupted != 0;
        }

        // ---- top-p sampling on the device (the managed ComputeGraphTensor.TopPSample, ComputeGraphTensor.cs:2305-2403, downloads
        //      the probabilities and walks them on the host; a graph that knows this backend calls these instead) ----
        public static Tensor TopPSample(Tensor probs, Tensor uniforms, float topP, float repeatPenalty = 0.0f, int[] seqs = null, int[] seqLens = null, int seqLd = 0)
        {
            Tensor result = new Tensor(probs.Allocator, DType.Float32, probs.Sizes[0], 1);
            if (seqs == null) HipNative.Check(HipNative.TSHip_TopPSample(V(result), V(probs), V(uniforms), topP), "TopPSample");
            else HipNative.Check(HipNative.TSHip_TopPSampleEx(V(result), V(probs), V(uniforms), topP, repeatPenalty, seqs, seqLens, seqLd), "TopPSample");
            return result;
        }

        /// <summary>The same pick into a caller-supplied result, with no allocation and no synchronisation (inputs up to about 300000 probabilities).</summary>
        public static void TopPSampleNoAlloc(Tensor result, Tensor probs, Tensor uniforms, float topP) =>
            HipNative.Check(HipNative.TSHip_TopPSampleNoAlloc(V(result), V(probs), V(uniforms), topP), "TopPSampleNoAlloc");

        /// <summary>RoPE with another base than the reference's literal 500000 (no OpRegistry name: the reference has no such parameter).</summary>
        public static Tensor RoPEWithBase(Tensor result, Tensor src, int seqLen, int rowOffset, float ropeBase)
        {
            Tensor writeTarget = TensorResultBuilder.GetWriteTarget(result, src, true, src.Sizes);
            HipNative.Check(HipNative.TSHip_RoPEEx(V(writeTarget), V(src), seqLen, rowOffset, ropeBase), "rope");
            return writeTarget;
        }

        /// <summary>Raw device helpers for callers that manage buffers themselves.</summary>
        public static void Memset(IntPtr devicePtr, int value, long bytes) => HipNative.Check(HipNative.TSHip_Memset(devicePtr, value, (UIntPtr)(ulong)bytes), "memset");
        public static void MemcpyDeviceToDevice(IntPtr dst, IntPtr src, long bytes) => HipNative.Check(HipNative.TSHip_MemcpyD2D(dst, src, (UIntPtr)(ulong)bytes), "memcpy");
        public static void Synchronize() => HipNative.Check(HipNative.TSHip_Synchronize(), "synchronize");
        public static void TrimPool() => HipNative.Check(HipNative.TSHip_PoolTrim(), "pool trim");
        public static int DeviceCount() { HipNative.Check(HipNative.TSHip_GetDeviceCount(out int n), "device count"); return n; }
    }
}
