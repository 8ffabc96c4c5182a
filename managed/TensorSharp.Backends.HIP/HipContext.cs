// One HIP device for the quantized matmul path (the role of TensorSharp.Backends.GGML/GgmlContext.cs:15-42): a single
// device id, availability checked when the context is built, operators of this assembly registered with the registry.
using System;
using System.Reflection;

namespace TensorSharp.HIP
{
    public sealed class HipContext
    {
        /// <summary>Device pickers ask this first; it loads the library and probes the device without initialising it.</summary>
        public static bool CanInitialize() => HipNative.CanInitialize();

        public HipContext(int[] deviceIds)
        {
            if (deviceIds == null || deviceIds.Length != 1)
            {
                if (deviceIds == null || deviceIds.Length == 0)
                    throw new ArgumentException("At least one device id is required for the HIP backend.", nameof(deviceIds));
                throw new NotSupportedException("The HIP backend drives one device per process; run one process per GPU.");
            }

            DeviceId = deviceIds[0];
            HipNative.EnsureAvailable();                                    // throws with the library's own message
            OpRegistry.RegisterAssembly(Assembly.GetExecutingAssembly());
        }

        public HipBackendType BackendType => HipBackendType.Hip;

        public int DeviceId { get; }
    }
}
