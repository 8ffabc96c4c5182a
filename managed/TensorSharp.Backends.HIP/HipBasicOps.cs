// Operator facade of the HIP backend for the quantized matmul path: tensor checks, view construction, native call.
// Counterpart of the quantized entry points of TensorSharp.Backends.GGML/GgmlBasicOps.cs (AddmmQuant :313-329,
// FusedRmsNormMatMulQuant / FusedMatMulQuantAdd / FusedFFNSwiGLUQuant :335-414, FusedOutProjNormRouter :416-447,
// FusedOutProjFFN :449-480, GetRowsQuant :565-579, MoEExperts* :586-700, AddmmQuantBatch :689-704,
// PreloadQuantizedWeight :706-709) with the same argument meaning and exception types, so that ModelBase.LinearForward
// and the model classes switch backends by switching the class they call.
using System;

namespace TensorSharp.HIP
{
    public static class HipBasicOps
    {
        // ---- tensor -> view ----------------------------------------------------------------------------------------
        // Tensors of this backend (HipStorage) and of the CPU backend (CpuStorage) both expose host memory.
        private static bool HostBacked(Tensor t) => t != null && (t.Storage is HipStorage || t.Storage is CpuStorage);

        private static IntPtr Start(Tensor t)
        {
            switch (t.Storage)
            {
                case HipStorage hs: return hs.PtrAtElement(t.StorageOffset);
                case CpuStorage cs: return cs.PtrAtElement(t.StorageOffset);
                default: throw new ArgumentException("Tensor storage must expose a host buffer.", nameof(t));
            }
        }

        /// <summary>Byte span from the first to the last addressed element, or -1 on overflow / empty dimensions.</summary>
        private static long SpanBytes(Tensor t)
        {
            try
            {
                long last = 0;
                for (int d = 0; d < t.DimensionCount; ++d)
                {
                    if (t.Sizes[d] <= 0) return -1;
                    last = checked(last + checked((t.Sizes[d] - 1) * t.Strides[d]));
                }
                return checked((last + 1) * t.ElementType.Size());
            }
            catch (OverflowException)
            {
                return -1;
            }
        }

        private static bool FitsInt(long v, out int r)
        {
            r = (int)v;
            return v >= int.MinValue && v <= int.MaxValue;
        }

        /// <summary>Any fp32 2-D view with strides that fit an int (the library packs non-standard inputs itself).</summary>
        private static bool Raw(Tensor t, out HipTensorView2D view)
        {
            view = default;
            long span;
            if (t.DimensionCount != 2 || t.ElementType != DType.Float32 || !HostBacked(t) || (span = SpanBytes(t)) < 0
                || !FitsInt(t.Sizes[0], out int d0) || !FitsInt(t.Sizes[1], out int d1)
                || !FitsInt(t.Strides[0], out int s0) || !FitsInt(t.Strides[1], out int s1))
                return false;
            view = new HipTensorView2D(Start(t), d0, d1, s0, s1, span);
            return true;
        }

        /// <summary>Innermost stride 1 and no overlap between rows: what the library writes results into.</summary>
        private static bool RowContiguous(Tensor t)
        {
            int n = t.DimensionCount;
            if (t.ElementType != DType.Float32 || n < 1 || n > 4 || t.Strides[n - 1] != 1)
                return false;
            long need = 1;
            for (int d = n - 1; d >= 0; --d)
            {
                if (t.Sizes[d] <= 0) return false;
                if (t.Sizes[d] == 1) continue;
                if (t.Strides[d] < need) return false;
                try { need = checked(t.Strides[d] * t.Sizes[d]); }
                catch (OverflowException) { return false; }
            }
            return true;
        }

        private static bool Standard(Tensor t, out HipTensorView2D view)
        {
            view = default;
            return RowContiguous(t) && Raw(t, out view);
        }

        private static bool Standard3(Tensor t, out HipTensorView3D view)
        {
            view = default;
            long span;
            if (t.DimensionCount != 3 || !RowContiguous(t) || !HostBacked(t) || (span = SpanBytes(t)) < 0
                || !FitsInt(t.Sizes[0], out int d0) || !FitsInt(t.Sizes[1], out int d1) || !FitsInt(t.Sizes[2], out int d2)
                || !FitsInt(t.Strides[0], out int s0) || !FitsInt(t.Strides[1], out int s1) || !FitsInt(t.Strides[2], out int s2))
                return false;
            view = new HipTensorView3D(Start(t), d0, d1, d2, s0, s1, s2, span);
            return true;
        }

        /// <summary>(in/out tensor as standard view, input as raw view) or the exceptions of the GGML facade.</summary>
        private static void Pair(string op, Tensor inout, Tensor input, out HipTensorView2D ioView, out HipTensorView2D inView)
        {
            if (inout.DimensionCount != 2 || input.DimensionCount != 2)
                throw new ArgumentException($"{op} requires 2D tensors.");
            if (inout.ElementType != DType.Float32 || input.ElementType != DType.Float32)
                throw new ArgumentException($"{op} requires Float32 tensors.");
            if (!HostBacked(inout) || !HostBacked(input))
                throw new ArgumentException($"{op} requires tensors backed by native CPU-accessible storage.");
            if (!Standard(inout, out ioView) | !Raw(input, out inView))
                throw new NotSupportedException($"HIP {op} requires tensors with supported row-contiguous layouts.");
        }

        private static IntPtr VectorStart(string op, Tensor v)
        {
            if (!HostBacked(v) || v.ElementType != DType.Float32)
                throw new ArgumentException($"{op} requires native-backed Float32 norm weights.");
            return Start(v);
        }

        // ---- matmul --------------------------------------------------------------------------------------------------
        /// <summary>result = m1 * W^T; W is ne1 rows of raw GGUF blocks with ne0 weights each.</summary>
        public static void AddmmQuant(Tensor result, Tensor m1, IntPtr weightData, int ggmlType, long ne0, long ne1, long rawBytes)
        {
            Pair("AddmmQuant", result, m1, out var r, out var x);
            HipNative.AddmmQuant(r, x, weightData, ggmlType, ne0, ne1, rawBytes);
        }

        /// <summary>Row b of m1 times the sub-weight at weightOffsets[b] of one stacked blob.</summary>
        public static void AddmmQuantBatch(Tensor result, Tensor m1, IntPtr weightData, int ggmlType, long ne0, long rawBytes,
            int batchCount, long[] weightOffsets, long[] weightNe1Arr)
        {
            Pair("AddmmQuantBatch", result, m1, out var r, out var x);
            HipNative.AddmmQuantBatch(r, x, weightData, ggmlType, ne0, rawBytes, batchCount, weightOffsets, weightNe1Arr);
        }

        public static void PreloadQuantizedWeight(IntPtr cacheKey, IntPtr hostData, int ggmlType, long ne0, long ne1, long rawBytes)
            => HipNative.PreloadQuantizedWeight(cacheKey, hostData, ggmlType, ne0, ne1, rawBytes);

        public static IntPtr AlignedAlloc(long size) => HipNative.TSHip_AlignedAlloc((UIntPtr)(ulong)size);

        public static void AlignedFree(IntPtr ptr) => HipNative.TSHip_AlignedFree(ptr);

        public static void InvalidateHostBuffer(IntPtr ptr) => HipNative.TSHip_InvalidateHostBuffer(ptr);

        public static void ClearHostBufferCache() => HipNative.TSHip_ClearHostBufferCache();

        /// <summary>Copies the device mirror of a host buffer (a KV cache the layer decode updates) back; no-op when none exists.</summary>
        public static void SyncHostBuffer(IntPtr ptr, long bytes) => HipNative.SyncHostBuffer(ptr, bytes);

        public static long GetRowSizeBytes(int ggmlType, long ne0)
        {
            long rb = (long)(ulong)HipNative.TSHip_RowSize(ggmlType, ne0);
            if (rb <= 0)
                throw new NotSupportedException($"GGML tensor type {ggmlType} is not supported, or ne[0]={ne0} is not aligned to the type block size.");
            return rb;
        }

        public static unsafe void DequantizeToFloat32(int ggmlType, IntPtr src, float[] dst, long numElements)
        {
            if (dst == null || numElements < 0 || numElements > dst.LongLength)
                throw new ArgumentOutOfRangeException(nameof(numElements));
            fixed (float* p = dst)
                HipNative.DequantizeToF32(ggmlType, src, numElements, (IntPtr)p);
        }

        // ---- fused wrappers --------------------------------------------------------------------------------------------
        public static void FusedRmsNormMatMulQuant(Tensor result, Tensor input, Tensor normWeight, float eps,
            IntPtr weightData, int ggmlType, long ne0, long ne1, long rawBytes)
        {
            Pair("FusedRmsNormMatMulQuant", result, input, out var r, out var x);
            HipNative.FusedRmsNormMatMulQuant(r, x, VectorStart("FusedRmsNormMatMulQuant", normWeight), (int)normWeight.ElementCount(), eps,
                weightData, ggmlType, ne0, ne1, rawBytes);
        }

        public static void FusedMatMulQuantAdd(Tensor residual, Tensor input, IntPtr weightData, int ggmlType, long ne0, long ne1, long rawBytes)
        {
            Pair("FusedMatMulQuantAdd", residual, input, out var r, out var x);
            HipNative.FusedMatMulQuantAdd(r, x, weightData, ggmlType, ne0, ne1, rawBytes);
        }

        public static void FusedFFNSwiGLUQuant(Tensor residual, Tensor input, Tensor normWeight, float eps,
            IntPtr gateUpData, int gateUpType, long gateUpNe0, long gateUpNe1, long gateUpRawBytes,
            IntPtr downData, int downType, long downNe0, long downNe1, long downRawBytes, int halfDim)
        {
            Pair("FusedFFNSwiGLUQuant", residual, input, out var r, out var x);
            HipNative.FusedFFNSwiGLUQuant(r, x, VectorStart("FusedFFNSwiGLUQuant", normWeight), (int)normWeight.ElementCount(), eps,
                gateUpData, gateUpType, gateUpNe0, gateUpNe1, gateUpRawBytes, downData, downType, downNe0, downNe1, downRawBytes, halfDim);
        }

        public static void FusedOutProjFFN(Tensor residual, Tensor input,
            IntPtr outProjData, int outProjType, long outNe0, long outNe1, long outRawBytes, Tensor ffnNormWeight, float eps,
            IntPtr guData, int guType, long guNe0, long guNe1, long guRawBytes,
            IntPtr dnData, int dnType, long dnNe0, long dnNe1, long dnRawBytes, int halfDim)
        {
            Pair("FusedOutProjFFN", residual, input, out var r, out var x);
            HipNative.FusedOutProjFFN(r, x, outProjData, outProjType, outNe0, outNe1, outRawBytes,
                VectorStart("FusedOutProjFFN", ffnNormWeight), (int)ffnNormWeight.ElementCount(), eps,
                guData, guType, guNe0, guNe1, guRawBytes, dnData, dnType, dnNe0, dnNe1, dnRawBytes, halfDim);
        }

        public static void FusedOutProjNormRouter(Tensor residual, Tensor input,
            IntPtr outProjData, int outProjType, long outNe0, long outNe1, long outRawBytes, Tensor normWeight, float eps, Tensor normedOutput,
            IntPtr routerData, int routerType, long routerNe0, long routerNe1, long routerRawBytes, Tensor routerOutput)
        {
            Pair("FusedOutProjNormRouter", residual, input, out var r, out var x);
            if (!HostBacked(normedOutput) || !HostBacked(routerOutput))
                throw new ArgumentException("FusedOutProjNormRouter requires native-backed tensors.");
            if (!Standard(normedOutput, out var n) | !Standard(routerOutput, out var l))
                throw new NotSupportedException("FusedOutProjNormRouter requires standard row-contiguous output tensors.");
            HipNative.FusedOutProjNormRouter(r, x, outProjData, outProjType, outNe0, outNe1, outRawBytes,
                VectorStart("FusedOutProjNormRouter", normWeight), (int)normWeight.ElementCount(), eps, n,
                routerData, routerType, routerNe0, routerNe1, routerRawBytes, l);
        }

        // ---- embedding gather and mul_mat_id ----------------------------------------------------------------------------
        private static HipContiguousTensor Indices(string op, Tensor indices)
        {
            if (!HostBacked(indices) || !indices.IsContiguous())
                throw new NotSupportedException($"HIP {op} requires contiguous native-backed indices.");
            int code = indices.ElementType == DType.Int32 ? 3 : indices.ElementType == DType.Float32 ? 0 : -1;
            if (code < 0)
                throw new ArgumentException($"{op} indices must be Int32 or Float32.");
            return new HipContiguousTensor(Start(indices), indices.ElementCount(), code);
        }

        /// <summary>result[i] = dequantized row indices[i] of the [ne1 x ne0] quantized table.</summary>
        public static void GetRowsQuant(Tensor result, IntPtr weightData, int ggmlType, long ne0, long ne1, long rawBytes, Tensor indices)
        {
            if (result.DimensionCount != 2 || result.ElementType != DType.Float32 || !HostBacked(result))
                throw new ArgumentException("GetRowsQuant requires a native-backed 2D Float32 result tensor.");
            if (!Standard(result, out var r))
                throw new NotSupportedException("HIP GetRowsQuant requires a standard-layout result.");
            HipNative.GetRowsQuant(r, weightData, ggmlType, ne0, ne1, rawBytes, Indices("GetRowsQuant", indices));
        }

        /// <summary>result[t, s, :] = expertWeights[ids[t, s]] * input[t, s mod slots] with F32 experts.</summary>
        public static void MulMatId(Tensor result, Tensor expertWeights, Tensor input, Tensor ids)
        {
            if (ids.DimensionCount != 2)
                throw new ArgumentException("MulMatId requires a 2D id tensor.");
            if (!Standard3(result, out var r) | !Standard3(expertWeights, out var w) | !Standard3(input, out var x))
                throw new NotSupportedException("HIP MulMatId requires native-backed standard-layout 3D Float32 tensors.");
            HipNative.MulMatId(r, w, x, Indices("MulMatId", ids), (int)ids.Sizes[0], (int)ids.Sizes[1]);
        }

        /// <summary>result[t, s, :] = src[t, s, :] + bias[ids[t, s], :]: the per-expert bias of a MulMatId (GgmlBasicOps.AddID).</summary>
        [RegisterOpStorageType("addid", typeof(HipStorage))]
        public static Tensor AddID(Tensor result, Tensor src, Tensor bias, Tensor ids)
        {
            if (src.DimensionCount != 3)
                throw new NotSupportedException("addid expects a 3D source tensor.");
            if (bias.DimensionCount != 2 || ids.DimensionCount != 2)
                throw new NotSupportedException("addid expects 2D bias and id tensors.");
            if (src.Sizes[2] != bias.Sizes[1] || src.Sizes[0] != ids.Sizes[0] || src.Sizes[1] != ids.Sizes[1])
                throw new InvalidOperationException("addid expects src shape [tokens, expert_used, rows], bias shape [experts, rows], and ids shape [tokens, expert_used].");
            Tensor writeTarget = TensorResultBuilder.GetWriteTarget(result, src, false, src.Sizes);
            if (!Standard3(writeTarget, out var r) | !Standard3(src, out var s) | !Standard(bias, out var b))
                throw new NotSupportedException("HIP addid requires Float32 standard-layout source/result tensors and a standard-layout 2D bias matrix.");
            HipNative.AddId(r, s, b, Indices("AddID", ids), (int)ids.Sizes[0], (int)ids.Sizes[1]);
            return writeTarget;
        }

        // ---- weighted expert sets -----------------------------------------------------------------------------------------
        public static void MoEExpertsForward(Tensor result, Tensor input, int numExperts, IntPtr[] upDataPtrs, IntPtr[] downDataPtrs,
            int upGgmlType, long upNe0, long upNe1, long upRawBytesEach,
            int downGgmlType, long downNe0, long downNe1, long downRawBytesEach, float[] routeWeights)
        {
            Pair("MoEExpertsForward", result, input, out var r, out var x);
            HipNative.MoEExpertsForward(r, x, numExperts, upDataPtrs, downDataPtrs, upGgmlType, upNe0, upNe1, upRawBytesEach,
                downGgmlType, downNe0, downNe1, downRawBytesEach, routeWeights);
        }

        public static void MoEExpertsSwiGLUForward(Tensor result, Tensor input, int numExperts,
            IntPtr[] gateDataPtrs, IntPtr[] upDataPtrs, IntPtr[] downDataPtrs,
            int gateGgmlType, long gateNe0, long gateNe1, long gateRawBytesEach,
            int upGgmlType, long upNe0, long upNe1, long upRawBytesEach,
            int downGgmlType, long downNe0, long downNe1, long downRawBytesEach, float[] routeWeights)
        {
            Pair("MoEExpertsSwiGLUForward", result, input, out var r, out var x);
            HipNative.MoEExpertsSwiGLUForward(r, x, numExperts, gateDataPtrs, upDataPtrs, downDataPtrs,
                gateGgmlType, gateNe0, gateNe1, gateRawBytesEach, upGgmlType, upNe0, upNe1, upRawBytesEach,
                downGgmlType, downNe0, downNe1, downRawBytesEach, routeWeights);
        }

        public static void MoEExpertsSwiGLUResidual(Tensor residual, Tensor input, int numExperts,
            IntPtr[] gateDataPtrs, IntPtr[] upDataPtrs, IntPtr[] downDataPtrs,
            int gateGgmlType, long gateNe0, long gateNe1, long gateRawBytesEach,
            int upGgmlType, long upNe0, long upNe1, long upRawBytesEach,
            int downGgmlType, long downNe0, long downNe1, long downRawBytesEach, float[] routeWeights,
            bool useShared, IntPtr sharedGateData, IntPtr sharedUpData, IntPtr sharedDownData,
            int sharedGateGgmlType, long sharedGateNe0, long sharedGateNe1, long sharedGateRawBytes,
            int sharedUpGgmlType, long sharedUpNe0, long sharedUpNe1, long sharedUpRawBytes,
            int sharedDownGgmlType, long sharedDownNe0, long sharedDownNe1, long sharedDownRawBytes, float sharedScalar)
        {
            Pair("MoEExpertsSwiGLUResidual", residual, input, out var r, out var x);
            HipNative.MoEExpertsSwiGLUResidual(r, x, numExperts, gateDataPtrs, upDataPtrs, downDataPtrs,
                gateGgmlType, gateNe0, gateNe1, gateRawBytesEach, upGgmlType, upNe0, upNe1, upRawBytesEach,
                downGgmlType, downNe0, downNe1, downRawBytesEach, routeWeights, useShared, sharedGateData, sharedUpData, sharedDownData,
                sharedGateGgmlType, sharedGateNe0, sharedGateNe1, sharedGateRawBytes, sharedUpGgmlType, sharedUpNe0, sharedUpNe1,
                sharedUpRawBytes, sharedDownGgmlType, sharedDownNe0, sharedDownNe1, sharedDownRawBytes, sharedScalar);
        }

        // ---- whole-layer decode: the arguments are already raw pointers in the callers (Qwen3Model and friends) ------------
        public static void TransformerLayerDecode(IntPtr hidden, int hiddenSize, IntPtr attnNorm,
            IntPtr qkv, int qkvType, long qkvNe0, long qkvNe1, long qkvBytes, IntPtr qNorm, IntPtr kNorm, int headDim,
            IntPtr o, int oType, long oNe0, long oNe1, long oBytes, IntPtr ffnNorm,
            IntPtr gu, int guType, long guNe0, long guNe1, long guBytes, IntPtr down, int downType, long downNe0, long downNe1, long downBytes,
            IntPtr kCache, IntPtr vCache, int numHeads, int numKvHeads, int maxSeqLen, int position, float eps, float ropeBase,
            float ropeFreqScale, int intermediateSize, int ropeMode)
            => HipNative.TransformerLayerDecode(hidden, hiddenSize, attnNorm, qkv, qkvType, qkvNe0, qkvNe1, qkvBytes, qNorm, kNorm, headDim,
                o, oType, oNe0, oNe1, oBytes, ffnNorm, gu, guType, guNe0, guNe1, guBytes, down, downType, downNe0, downNe1, downBytes,
                kCache, vCache, numHeads, numKvHeads, maxSeqLen, position, eps, ropeBase, ropeFreqScale, intermediateSize, ropeMode);
    }
}
