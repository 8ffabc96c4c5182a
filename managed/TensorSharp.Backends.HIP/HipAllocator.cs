// Allocator of host-resident tensors for the HIP backend (the role GgmlAllocator plays for the GGML backends,
// TensorSharp.Backends.GGML/GgmlAllocator.cs:14-46).  Activations live in page-aligned host memory; the library moves
// them to the device per call and keeps quantized weights resident there (TSHip_PreloadQuantizedWeight), so nothing
// allocated here counts against device memory.
using System;
using System.Threading;

namespace TensorSharp.HIP
{
    [Serializable]
    public class HipAllocator : IAllocator
    {
        private long liveBytes;       // host bytes currently held by storages of this allocator

        public HipAllocator(HipContext context, int deviceId)
        {
            Context = context ?? throw new ArgumentNullException(nameof(context));
            DeviceId = deviceId;
        }

        public HipContext Context { get; }

        public int DeviceId { get; }

        /// <summary>Dense fp32 operators without a HIP export run on the CPU implementations registered for host storage.</summary>
        public BlasEnum BlasEnum => BlasEnum.GGML_CPU;

        public long LiveHostBytes => Interlocked.Read(ref liveBytes);

        public Storage Allocate(DType elementType, long elementCount)
        {
            if (elementType == DType.Float16)
                throw new NotSupportedException("The HIP backend computes in Float32 tensors only. Disable AMP to use this backend.");
            var storage = new HipStorage(this, Context, elementType, elementCount);
            Interlocked.Add(ref liveBytes, storage.ByteLength);
            return storage;
        }

        internal void Released(long bytes) => Interlocked.Add(ref liveBytes, -bytes);

        /// <summary>Host memory is not a budgeted pool: the trainer-side heuristics that read this see an empty device.</summary>
        public float GetAllocatedMemoryRatio() => 0.0f;
    }
}
