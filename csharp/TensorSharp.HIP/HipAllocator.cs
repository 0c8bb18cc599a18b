// IAllocator of the HIP backend (TensorSharp/IAllocator.cs:13-20), modelled on TensorSharp.GGML/GgmlAllocator.cs.
using System;

namespace TensorSharp.HIP
{
    [Serializable]
    public class HipAllocator : IAllocator
    {
        private readonly HipContext context;
        private readonly int deviceId;

        public HipAllocator(HipContext context, int deviceId)
        {
            this.context = context ?? throw new ArgumentNullException(nameof(context));
            this.deviceId = deviceId;
        }

        // BlasEnum has no HIP member; it is only consulted by the CPU GEMM dispatch (MatrixMultiplication.cs:618), which never
        // sees a HipStorage tensor.
        public BlasEnum BlasEnum => BlasEnum.CUDA;

        public int DeviceId => deviceId;

        public HipContext Context => context;

        public Storage Allocate(DType elementType, long elementCount)
        {
            if (elementType != DType.Float32 && elementType != DType.Float16)
                throw new NotSupportedException("The HIP backend holds Float32 and Float16 tensors (indices travel as Float32, as everywhere in Seq2SeqSharp).");
            return new HipStorage(this, context, elementType, elementCount);
        }

        public float GetAllocatedMemoryRatio()
        {
            HipNative.Check(HipNative.TSHip_GetMemInfo(out UIntPtr free, out UIntPtr total), "meminfo");
            double t = total.ToUInt64();
            return t > 0 ? (float)(1.0 - free.ToUInt64() / t) : 0.0f;
        }
    }
}
