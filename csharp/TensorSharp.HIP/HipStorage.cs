// Device storage: the ten abstract members of TensorSharp/Storage.cs:32-47 as synchronous device <-> host copies, like
// TensorSharp.CUDA/CudaStorage.cs:35-173 (a GgmlStorage lives in host memory and dereferences its pointer instead).
using System;
using System.Runtime.InteropServices;
using ManagedCuda.BasicTypes;

namespace TensorSharp.HIP
{
    [Serializable]
    public class HipStorage : Storage
    {
        private IntPtr buffer;        // device address from TSHip_Malloc

        public HipStorage(HipAllocator allocator, HipContext context, DType elementType, long elementCount)
            : base(allocator, elementType, elementCount)
        {
            Context = context ?? throw new ArgumentNullException(nameof(context));
            HipNative.Check(HipNative.TSHip_Malloc(out buffer, (UIntPtr)(ulong)Math.Max(ByteLength, 4)), "malloc");
        }

        public HipContext Context { get; }

        public int DeviceId => ((HipAllocator)Allocator).DeviceId;

        protected override void Destroy()
        {
            if (buffer != IntPtr.Zero)
            {
                HipNative.TSHip_Free(buffer);      // back to the native pool; no device synchronisation
                buffer = IntPtr.Zero;
            }
        }

        public override string LocationDescription() => $"HIP:{DeviceId}";

        public IntPtr DevicePtrAtElement(long index) => new IntPtr(buffer.ToInt64() + index * ElementType.Size());

        private unsafe void Download(long index, void* dst, long bytes) =>
            HipNative.Check(HipNative.TSHip_MemcpyD2H(new IntPtr(dst), DevicePtrAtElement(index), (UIntPtr)(ulong)bytes), "memcpy device to host");

        private unsafe void Upload(long index, void* src, long bytes) =>
            HipNative.Check(HipNative.TSHip_MemcpyH2D(DevicePtrAtElement(index), new IntPtr(src), (UIntPtr)(ulong)bytes), "memcpy host to device");

        private static float HalfToFloat(ushort h) => (float)BitConverter.UInt16BitsToHalf(h);
        private static ushort FloatToHalf(float f) => BitConverter.HalfToUInt16Bits((Half)f);      // round to nearest even, as BasicTypesStructAsTypes.cs:800-840

        public override unsafe float GetElementAsFloat(long index)
        {
            if (ElementType == DType.Float32) { float v; Download(index, &v, 4); return v; }
            if (ElementType == DType.Float16) { ushort h; Download(index, &h, 2); return HalfToFloat(h); }
            throw new NotSupportedException("Element type " + ElementType + " not supported");
        }

        public override unsafe float[] GetElementsAsFloat(long index, int length)
        {
            float[] array = new float[length];
            if (length == 0) return array;
            if (ElementType == DType.Float32)
            {
                fixed (float* p = array) Download(index, p, 4L * length);
                return array;
            }
            if (ElementType == DType.Float16)
            {
                ushort[] tmp = new ushort[length];
                fixed (ushort* p = tmp) Download(index, p, 2L * length);
                for (int i = 0; i < length; i++) array[i] = HalfToFloat(tmp[i]);
                return array;
            }
            throw new NotSupportedException("Element type " + ElementType + " not supported");
        }

        public override unsafe void SetElementAsFloat(long index, float value)
        {
            if (ElementType == DType.Float32) { Upload(index, &value, 4); return; }
            if (ElementType == DType.Float16) { ushort h = FloatToHalf(value); Upload(index, &h, 2); return; }
            throw new NotSupportedException("Element type " + ElementType + " not supported");
        }

        public override unsafe void SetElementsAsFloat(long index, float[] value)
        {
            if (value.Length == 0) return;
            if (ElementType == DType.Float32)
            {
                fixed (float* p = value) Upload(index, p, 4L * value.Length);
                return;
            }
            if (ElementType == DType.Float16)
            {
                ushort[] tmp = new ushort[value.Length];
                for (int i = 0; i < value.Length; i++) tmp[i] = FloatToHalf(value[i]);
                fixed (ushort* p = tmp) Upload(index, p, 2L * tmp.Length);
                return;
            }
            throw new NotSupportedException("Element type " + ElementType + " not supported");
        }

        public override unsafe void SetElementsAsHalf(long index, half[] value)      // fp16 weight upload, WeightTensor.cs:504-515
        {
            if (ElementType != DType.Float16) throw new NotSupportedException("SetElementsAsHalf needs a Float16 storage");
            if (value.Length == 0) return;
            fixed (half* p = value) Upload(index, p, 2L * value.Length);
        }

        public override int[] GetElementsAsInt(long index, int length)
        {
            float[] f = GetElementsAsFloat(index, length);      // indices are stored as floats on this backend
            int[] r = new int[length];
            for (int i = 0; i < length; i++) r[i] = (int)f[i];
            return r;
        }

        public override void SetElementsAsInt(long index, int[] value)
        {
            float[] f = new float[value.Length];
            for (int i = 0; i < value.Length; i++) f[i] = value[i];
            SetElementsAsFloat(index, f);
        }

        public override void CopyToStorage(long storageIndex, IntPtr src, long byteCount) =>
            HipNative.Check(HipNative.TSHip_MemcpyH2D(DevicePtrAtElement(storageIndex), src, (UIntPtr)(ulong)byteCount), "memcpy host to device");

        public override void CopyFromStorage(IntPtr dst, long storageIndex, long byteCount) =>
            HipNative.Check(HipNative.TSHip_MemcpyD2H(dst, DevicePtrAtElement(storageIndex), (UIntPtr)(ulong)byteCount), "memcpy device to host");
    }
}
