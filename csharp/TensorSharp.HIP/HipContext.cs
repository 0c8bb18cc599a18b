// Backend context: checks that the native library and a gfx950 device are there, registers this assembly's op handlers.
// Mirrors TensorSharp.GGML/GgmlContext.cs:10-28; the memory pool lives in the native library (TSHip_Malloc / TSHip_Free).
using System;
using System.Reflection;

namespace TensorSharp.HIP
{
    public sealed class HipContext
    {
        public HipContext(int[] deviceIds)
        {
            if (deviceIds == null || deviceIds.Length == 0) throw new ArgumentException("At least one device id is required for the HIP backend.", nameof(deviceIds));
            if (deviceIds.Length != 1) throw new NotSupportedException("The HIP backend drives one device per process.");
            DeviceId = deviceIds[0];
            HipNative.EnsureAvailable(DeviceId);
            OpRegistry.RegisterAssembly(Assembly.GetExecutingAssembly());
        }

        public int DeviceId { get; }

        /// <summary>Bytes the native pool has handed out and bytes it keeps cached for reuse.</summary>
        public (long inUse, long cached) PoolBytes()
        {
            HipNative.Check(HipNative.TSHip_GetPoolStats(out _, out UIntPtr inUse, out UIntPtr cached), "pool stats");
            return ((long)inUse.ToUInt64(), (long)cached.ToUInt64());
        }
    }
}
