// Host buffer behind a tensor of the HIP backend.  Counterpart of TensorSharp.Backends.GGML/GgmlStorage.cs:14-202: the
// same Storage contract (element accessors for Float32 / Float64 / Int32 / UInt8, raw copies in and out, PtrAtElement
// for the operator layer), over memory from TSHip_AlignedAlloc so that the library can pin or map whole pages.
using System;

namespace TensorSharp.HIP
{
    [Serializable]
    public class HipStorage : Storage
    {
        private IntPtr buffer;

        public HipStorage(HipAllocator allocator, HipContext context, DType elementType, long elementCount)
            : base(allocator, elementType, elementCount)
        {
            Context = context ?? throw new ArgumentNullException(nameof(context));
            buffer = HipNative.TSHip_AlignedAlloc((UIntPtr)(ulong)Math.Max(ByteLength, 1));
            if (buffer == IntPtr.Zero)
                throw new OutOfMemoryException($"Unable to allocate {ByteLength} bytes of host memory for a HIP tensor.");
        }

        public HipContext Context { get; }

        public int DeviceId => ((HipAllocator)Allocator).DeviceId;

        protected override void Destroy()
        {
            if (buffer == IntPtr.Zero)
                return;
            // a KV cache or weight the library mirrored on the device under this address must not outlive the host block
            HipNative.TSHip_InvalidateHostBuffer(buffer);
            HipNative.TSHip_AlignedFree(buffer);
            buffer = IntPtr.Zero;
            ((HipAllocator)Allocator).Released(ByteLength);
        }

        public override string LocationDescription() => $"HIP:{DeviceId}";

        public IntPtr PtrAtElement(long index) => new IntPtr(buffer.ToInt64() + index * ElementType.Size());

        private NotSupportedException Unsupported() => new NotSupportedException("Element type " + ElementType + " not supported");

        private unsafe float Read(long i)
        {
            void* p = buffer.ToPointer();
            switch (ElementType)
            {
                case DType.Float32: return ((float*)p)[i];
                case DType.Float64: return (float)((double*)p)[i];
                case DType.Int32: return ((int*)p)[i];
                case DType.UInt8: return ((byte*)p)[i];
                default: throw Unsupported();
            }
        }

        private unsafe void Write(long i, float v)
        {
            void* p = buffer.ToPointer();
            switch (ElementType)
            {
                case DType.Float32: ((float*)p)[i] = v; break;
                case DType.Float64: ((double*)p)[i] = v; break;
                case DType.Int32: ((int*)p)[i] = (int)v; break;
                case DType.UInt8: ((byte*)p)[i] = (byte)v; break;
                default: throw Unsupported();
            }
        }

        public override float GetElementAsFloat(long index) => Read(index);

        public override void SetElementAsFloat(long index, float value) => Write(index, value);

        public override unsafe float[] GetElementsAsFloat(long index, int length)
        {
            if (ElementType != DType.Float32)
                throw Unsupported();
            var result = new float[length];
            new ReadOnlySpan<float>((float*)buffer.ToPointer() + index, length).CopyTo(result);
            return result;
        }

        public override unsafe void SetElementsAsFloat(long index, float[] value)
        {
            if (ElementType != DType.Float32)
                throw Unsupported();
            value.AsSpan().CopyTo(new Span<float>((float*)buffer.ToPointer() + index, value.Length));
        }

        public override unsafe int[] GetElementsAsInt(long index, int length)
        {
            if (ElementType != DType.Int32)
                throw Unsupported();
            var result = new int[length];
            new ReadOnlySpan<int>((int*)buffer.ToPointer() + index, length).CopyTo(result);
            return result;
        }

        public override unsafe void SetElementsAsInt(long index, int[] value)
        {
            if (ElementType != DType.Int32)
                throw Unsupported();
            value.AsSpan().CopyTo(new Span<int>((int*)buffer.ToPointer() + index, value.Length));
        }

        public override void SetElementsAsHalf(long index, half[] value)
            => throw new NotSupportedException("The HIP backend computes in Float32 tensors only. Disable AMP to use this backend.");

        public override unsafe void CopyToStorage(long storageIndex, IntPtr src, long byteCount)
            => Buffer.MemoryCopy(src.ToPointer(), PtrAtElement(storageIndex).ToPointer(), byteCount, byteCount);

        public override unsafe void CopyFromStorage(IntPtr dst, long storageIndex, long byteCount)
            => Buffer.MemoryCopy(PtrAtElement(storageIndex).ToPointer(), dst.ToPointer(), byteCount, byteCount);
    }
}
