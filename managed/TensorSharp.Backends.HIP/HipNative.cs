// P/Invoke layer of the HIP backend: one declaration per host-pointer export of include/tship_ops.h.
// Counterpart of TensorSharp.Backends.GGML/GgmlNative.cs (struct layouts :27-132, quantized entry points :203-420,
// :518-531, :647-659, result checking :1539-1547, :1622-1627).  Not compiled in this repository (no .NET toolchain in
// the build image); the argument lists are kept in step with the header by tests/test_abi_cpu.py, which parses both.
using System;
using System.Runtime.InteropServices;

namespace TensorSharp.HIP
{
    /// <summary>Backend selector passed to TSHip_IsBackendAvailable; continues GgmlBackendType (Metal 1, Cpu 2, Cuda 3).</summary>
    public enum HipBackendType
    {
        Hip = 4,
    }

    /// <summary>2-D fp32 view; strides in elements, RawBytes is the byte span from Data to the last element.</summary>
    [StructLayout(LayoutKind.Sequential)]
    internal readonly struct HipTensorView2D
    {
        public readonly IntPtr Data;
        public readonly int Dim0, Dim1, Stride0, Stride1;
        public readonly long RawBytes;

        public HipTensorView2D(IntPtr data, int dim0, int dim1, int stride0, int stride1, long rawBytes)
        {
            Data = data; Dim0 = dim0; Dim1 = dim1; Stride0 = stride0; Stride1 = stride1; RawBytes = rawBytes;
        }
    }

    [StructLayout(LayoutKind.Sequential)]
    internal readonly struct HipTensorView3D
    {
        public readonly IntPtr Data;
        public readonly int Dim0, Dim1, Dim2, Stride0, Stride1, Stride2;
        public readonly long RawBytes;

        public HipTensorView3D(IntPtr data, int dim0, int dim1, int dim2, int stride0, int stride1, int stride2, long rawBytes)
        {
            Data = data; Dim0 = dim0; Dim1 = dim1; Dim2 = dim2; Stride0 = stride0; Stride1 = stride1; Stride2 = stride2; RawBytes = rawBytes;
        }
    }

    /// <summary>Contiguous index / value array; ElementType 0 = Float32, 3 = Int32.</summary>
    [StructLayout(LayoutKind.Sequential)]
    internal readonly struct HipContiguousTensor
    {
        public readonly IntPtr Data;
        public readonly long ElementCount;
        public readonly int ElementType;

        public HipContiguousTensor(IntPtr data, long elementCount, int elementType)
        {
            Data = data; ElementCount = elementCount; ElementType = elementType;
        }
    }

    internal static class HipNative
    {
        private const string Dll = "TsHipOps";      // libTsHipOps.so beside the assembly or on LD_LIBRARY_PATH
        private const CallingConvention CC = CallingConvention.Cdecl;

        // ---- utilities -------------------------------------------------------------------------------------
        [DllImport(Dll, CallingConvention = CC)] private static extern IntPtr TSHip_GetLastError();
        [DllImport(Dll, CallingConvention = CC)] private static extern int TSHip_IsBackendAvailable(int backendType);
        [DllImport(Dll, CallingConvention = CC)] private static extern int TSHip_CanInitializeBackend(int backendType);
        [DllImport(Dll, CallingConvention = CC)] internal static extern UIntPtr TSHip_RowSize(int ggmlType, long ne);
        [DllImport(Dll, CallingConvention = CC)] internal static extern IntPtr TSHip_AlignedAlloc(UIntPtr size);
        [DllImport(Dll, CallingConvention = CC)] internal static extern void TSHip_AlignedFree(IntPtr ptr);
        [DllImport(Dll, CallingConvention = CC)] internal static extern void TSHip_InvalidateHostBuffer(IntPtr ptr);
        [DllImport(Dll, CallingConvention = CC)] internal static extern void TSHip_ClearHostBufferCache();
        [DllImport(Dll, CallingConvention = CC)] private static extern int TSHip_SyncHostBuffer(IntPtr ptr, UIntPtr size);
        [DllImport(Dll, CallingConvention = CC)] private static extern int TSHip_DequantizeToF32(int ggmlType, IntPtr src, long numElements, IntPtr dst);

        // ---- quantized matmul --------------------------------------------------------------------------------
        [DllImport(Dll, CallingConvention = CC)]
        private static extern int TSHip_AddmmQuantF32(HipTensorView2D result, HipTensorView2D m1, IntPtr m2Data, int m2GgmlType,
            long m2Ne0, long m2Ne1, long m2RawBytes);

        [DllImport(Dll, CallingConvention = CC)]
        private static extern int TSHip_AddmmQuantBatchF32(HipTensorView2D result, HipTensorView2D m1, IntPtr m2Data, int m2GgmlType,
            long m2Ne0, long m2RawBytes, int batchCount, long[] weightOffsets, long[] weightNe1Arr);

        [DllImport(Dll, CallingConvention = CC)]
        private static extern int TSHip_PreloadQuantizedWeight(IntPtr cacheKey, IntPtr hostData, int ggmlType, long ne0, long ne1, long rawBytes);

        [DllImport(Dll, CallingConvention = CC)]
        private static extern int TSHip_GetRowsQuantF32(HipTensorView2D result, IntPtr srcData, int srcGgmlType, long srcNe0, long srcNe1,
            long srcRawBytes, HipContiguousTensor indices);

        [DllImport(Dll, CallingConvention = CC)]
        private static extern int TSHip_MulMatIdF32(HipTensorView3D result, HipTensorView3D expertWeights, HipTensorView3D input,
            HipContiguousTensor ids, int idsRows, int idsCols);

        [DllImport(Dll, CallingConvention = CC)]
        private static extern int TSHip_AddIdF32(HipTensorView3D result, HipTensorView3D src, HipTensorView2D bias,
            HipContiguousTensor ids, int idsRows, int idsCols);

        // ---- fused wrappers ------------------------------------------------------------------------------------
        [DllImport(Dll, CallingConvention = CC)]
        private static extern int TSHip_FusedRmsNormMatMulQuantF32(HipTensorView2D result, HipTensorView2D input, IntPtr normWeightData,
            int normWeightCount, float eps, IntPtr m2Data, int m2GgmlType, long m2Ne0, long m2Ne1, long m2RawBytes);

        [DllImport(Dll, CallingConvention = CC)]
        private static extern int TSHip_FusedMatMulQuantAddF32(HipTensorView2D residual, HipTensorView2D input, IntPtr m2Data, int m2GgmlType,
            long m2Ne0, long m2Ne1, long m2RawBytes);

        [DllImport(Dll, CallingConvention = CC)]
        private static extern int TSHip_FusedFFNSwiGLUQuantF32(HipTensorView2D residual, HipTensorView2D input, IntPtr normWeightData,
            int normWeightCount, float eps, IntPtr gateUpData, int gateUpGgmlType, long gateUpNe0, long gateUpNe1, long gateUpRawBytes,
            IntPtr downData, int downGgmlType, long downNe0, long downNe1, long downRawBytes, int halfDim);

        [DllImport(Dll, CallingConvention = CC)]
        private static extern int TSHip_FusedOutProjFFNQuantF32(HipTensorView2D residual, HipTensorView2D input,
            IntPtr outProjData, int outProjType, long outNe0, long outNe1, long outRawBytes,
            IntPtr ffnNormData, int ffnNormCount, float eps,
            IntPtr guData, int guType, long guNe0, long guNe1, long guRawBytes,
            IntPtr dnData, int dnType, long dnNe0, long dnNe1, long dnRawBytes, int halfDim);

        [DllImport(Dll, CallingConvention = CC)]
        private static extern int TSHip_FusedOutProjNormRouterQuantF32(HipTensorView2D residual, HipTensorView2D input,
            IntPtr outProjData, int outProjType, long outNe0, long outNe1, long outRawBytes,
            IntPtr normData, int normCount, float eps, HipTensorView2D normedOut,
            IntPtr routerData, int routerType, long routerNe0, long routerNe1, long routerRawBytes, HipTensorView2D routerOut);

        // ---- weighted expert sets ------------------------------------------------------------------------------
        [DllImport(Dll, CallingConvention = CC)]
        private static extern int TSHip_MoEExpertsForwardF32(HipTensorView2D result, HipTensorView2D input, int numExperts,
            IntPtr[] upDataPtrs, IntPtr[] downDataPtrs, int upGgmlType, long upNe0, long upNe1, long upRawBytesEach,
            int downGgmlType, long downNe0, long downNe1, long downRawBytesEach, float[] routeWeights);

        [DllImport(Dll, CallingConvention = CC)]
        private static extern int TSHip_MoEExpertsSwiGLUForwardF32(HipTensorView2D result, HipTensorView2D input, int numExperts,
            IntPtr[] gateDataPtrs, IntPtr[] upDataPtrs, IntPtr[] downDataPtrs,
            int gateGgmlType, long gateNe0, long gateNe1, long gateRawBytesEach,
            int upGgmlType, long upNe0, long upNe1, long upRawBytesEach,
            int downGgmlType, long downNe0, long downNe1, long downRawBytesEach, float[] routeWeights);

        [DllImport(Dll, CallingConvention = CC)]
        private static extern int TSHip_MoEExpertsSwiGLUResidualF32(HipTensorView2D residual, HipTensorView2D input, int numExperts,
            IntPtr[] gateDataPtrs, IntPtr[] upDataPtrs, IntPtr[] downDataPtrs,
            int gateGgmlType, long gateNe0, long gateNe1, long gateRawBytesEach,
            int upGgmlType, long upNe0, long upNe1, long upRawBytesEach,
            int downGgmlType, long downNe0, long downNe1, long downRawBytesEach, float[] routeWeights,
            int useShared, IntPtr sharedGateData, IntPtr sharedUpData, IntPtr sharedDownData,
            int sharedGateGgmlType, long sharedGateNe0, long sharedGateNe1, long sharedGateRawBytes,
            int sharedUpGgmlType, long sharedUpNe0, long sharedUpNe1, long sharedUpRawBytes,
            int sharedDownGgmlType, long sharedDownNe0, long sharedDownNe1, long sharedDownRawBytes, float sharedScalar);

        // ---- whole-layer decode ---------------------------------------------------------------------------------
        [DllImport(Dll, CallingConvention = CC)]
        private static extern int TSHip_TransformerLayerDecode(IntPtr hidden, int hiddenSize, IntPtr attnNorm,
            IntPtr qkvData, int qkvType, long qkvNe0, long qkvNe1, long qkvBytes, IntPtr qNorm, IntPtr kNorm, int headDim,
            IntPtr oData, int oType, long oNe0, long oNe1, long oBytes, IntPtr ffnNorm,
            IntPtr guData, int guType, long guNe0, long guNe1, long guBytes,
            IntPtr downData, int downType, long downNe0, long downNe1, long downBytes,
            IntPtr kCache, IntPtr vCache, int numHeads, int numKvHeads, int maxSeqLen, int position, float eps, float ropeBase,
            float ropeFreqScale, int intermediateSize, int ropeMode);

        [DllImport(Dll, CallingConvention = CC)]
        private static extern int TSHip_TransformerModelDecode(IntPtr hidden, int hiddenSize, int numLayers,
            IntPtr[] attnNorm, IntPtr[] qkv, IntPtr[] qNorm, IntPtr[] kNorm, IntPtr[] o, IntPtr[] ffnNorm, IntPtr[] gu, IntPtr[] down,
            IntPtr[] kCache, IntPtr[] vCache,
            int qkvType, long qkvNe0, long qkvNe1, long qkvBytes, int oType, long oNe0, long oNe1, long oBytes,
            int guType, long guNe0, long guNe1, long guBytes, int downType, long downNe0, long downNe1, long downBytes,
            int headDim, int numHeads, int numKvHeads, int maxSeqLen, int position, float eps, float ropeBase, float ropeFreqScale,
            int intermediateSize, int ropeMode);

        // ---- availability and error reporting --------------------------------------------------------------------
        private static readonly Lazy<bool> available = new Lazy<bool>(() =>
        {
            try
            {
                return TSHip_IsBackendAvailable((int)HipBackendType.Hip) != 0;
            }
            catch (DllNotFoundException)
            {
                return false;
            }
            catch (EntryPointNotFoundException)
            {
                return false;
            }
        });

        /// <summary>Side-effect-free probe (TSHip_CanInitializeBackend) for device pickers.</summary>
        internal static bool CanInitialize()
        {
            try { return TSHip_CanInitializeBackend((int)HipBackendType.Hip) != 0; }
            catch (DllNotFoundException) { return false; }
        }

        internal static void EnsureAvailable()
        {
            if (!available.Value)
                throw new InvalidOperationException("The HIP backend is not available: " + LastError("libTsHipOps.so missing or no gfx950 device"));
        }

        private static string LastError(string fallback)
        {
            IntPtr p = TSHip_GetLastError();
            string msg = p == IntPtr.Zero ? null : Marshal.PtrToStringUTF8(p);
            return string.IsNullOrEmpty(msg) ? fallback : msg;
        }

        /// <summary>The exports return 1 on success and 0 with a thread-local message on failure.</summary>
        private static void Check(int ok, string what)
        {
            if (ok == 0)
                throw new InvalidOperationException($"Native HIP {what} failed: {LastError("unknown native error")}");
        }

        // ---- checked entry points (what HipBasicOps calls) --------------------------------------------------------
        internal static void AddmmQuant(HipTensorView2D result, HipTensorView2D m1, IntPtr w, int type, long ne0, long ne1, long rawBytes)
            => Check(TSHip_AddmmQuantF32(result, m1, w, type, ne0, ne1, rawBytes), "addmm_quant");

        internal static void AddmmQuantBatch(HipTensorView2D result, HipTensorView2D m1, IntPtr w, int type, long ne0, long rawBytes,
            int batchCount, long[] offsets, long[] ne1)
            => Check(TSHip_AddmmQuantBatchF32(result, m1, w, type, ne0, rawBytes, batchCount, offsets, ne1), "addmm_quant_batch");

        internal static void PreloadQuantizedWeight(IntPtr cacheKey, IntPtr hostData, int type, long ne0, long ne1, long rawBytes)
            => Check(TSHip_PreloadQuantizedWeight(cacheKey, hostData, type, ne0, ne1, rawBytes), "preload_quantized_weight");

        internal static void SyncHostBuffer(IntPtr ptr, long bytes) => Check(TSHip_SyncHostBuffer(ptr, (UIntPtr)(ulong)bytes), "sync_host_buffer");

        internal static void GetRowsQuant(HipTensorView2D result, IntPtr src, int type, long ne0, long ne1, long rawBytes, HipContiguousTensor indices)
            => Check(TSHip_GetRowsQuantF32(result, src, type, ne0, ne1, rawBytes, indices), "get_rows_quant");

        internal static void MulMatId(HipTensorView3D result, HipTensorView3D experts, HipTensorView3D input, HipContiguousTensor ids, int rows, int cols)
            => Check(TSHip_MulMatIdF32(result, experts, input, ids, rows, cols), "mulmatid");

        internal static void AddId(HipTensorView3D result, HipTensorView3D src, HipTensorView2D bias, HipContiguousTensor ids, int rows, int cols)
            => Check(TSHip_AddIdF32(result, src, bias, ids, rows, cols), "addid");

        internal static void FusedRmsNormMatMulQuant(HipTensorView2D result, HipTensorView2D input, IntPtr norm, int normCount, float eps,
            IntPtr w, int type, long ne0, long ne1, long rawBytes)
            => Check(TSHip_FusedRmsNormMatMulQuantF32(result, input, norm, normCount, eps, w, type, ne0, ne1, rawBytes), "fused_rms_norm_matmul_quant");

        internal static void FusedMatMulQuantAdd(HipTensorView2D residual, HipTensorView2D input, IntPtr w, int type, long ne0, long ne1, long rawBytes)
            => Check(TSHip_FusedMatMulQuantAddF32(residual, input, w, type, ne0, ne1, rawBytes), "fused_matmul_quant_add");

        internal static void FusedFFNSwiGLUQuant(HipTensorView2D residual, HipTensorView2D input, IntPtr norm, int normCount, float eps,
            IntPtr gu, int guType, long guNe0, long guNe1, long guBytes, IntPtr dn, int dnType, long dnNe0, long dnNe1, long dnBytes, int halfDim)
            => Check(TSHip_FusedFFNSwiGLUQuantF32(residual, input, norm, normCount, eps, gu, guType, guNe0, guNe1, guBytes, dn, dnType, dnNe0,
                dnNe1, dnBytes, halfDim), "fused_ffn_swiglu_quant");

        internal static void FusedOutProjFFN(HipTensorView2D residual, HipTensorView2D input, IntPtr o, int oType, long oNe0, long oNe1, long oBytes,
            IntPtr norm, int normCount, float eps, IntPtr gu, int guType, long guNe0, long guNe1, long guBytes,
            IntPtr dn, int dnType, long dnNe0, long dnNe1, long dnBytes, int halfDim)
            => Check(TSHip_FusedOutProjFFNQuantF32(residual, input, o, oType, oNe0, oNe1, oBytes, norm, normCount, eps, gu, guType, guNe0, guNe1,
                guBytes, dn, dnType, dnNe0, dnNe1, dnBytes, halfDim), "fused_outproj_ffn");

        internal static void FusedOutProjNormRouter(HipTensorView2D residual, HipTensorView2D input, IntPtr o, int oType, long oNe0, long oNe1,
            long oBytes, IntPtr norm, int normCount, float eps, HipTensorView2D normedOut, IntPtr router, int routerType, long rNe0, long rNe1,
            long rBytes, HipTensorView2D routerOut)
            => Check(TSHip_FusedOutProjNormRouterQuantF32(residual, input, o, oType, oNe0, oNe1, oBytes, norm, normCount, eps, normedOut, router,
                routerType, rNe0, rNe1, rBytes, routerOut), "fused_outproj_norm_router");

        internal static void MoEExpertsForward(HipTensorView2D result, HipTensorView2D input, int n, IntPtr[] up, IntPtr[] down,
            int upType, long upNe0, long upNe1, long upBytes, int downType, long downNe0, long downNe1, long downBytes, float[] routeWeights)
            => Check(TSHip_MoEExpertsForwardF32(result, input, n, up, down, upType, upNe0, upNe1, upBytes, downType, downNe0, downNe1, downBytes,
                routeWeights), "moe_experts_forward");

        internal static void MoEExpertsSwiGLUForward(HipTensorView2D result, HipTensorView2D input, int n, IntPtr[] gate, IntPtr[] up, IntPtr[] down,
            int gateType, long gateNe0, long gateNe1, long gateBytes, int upType, long upNe0, long upNe1, long upBytes,
            int downType, long downNe0, long downNe1, long downBytes, float[] routeWeights)
            => Check(TSHip_MoEExpertsSwiGLUForwardF32(result, input, n, gate, up, down, gateType, gateNe0, gateNe1, gateBytes, upType, upNe0, upNe1,
                upBytes, downType, downNe0, downNe1, downBytes, routeWeights), "moe_experts_swiglu_forward");

        internal static void MoEExpertsSwiGLUResidual(HipTensorView2D residual, HipTensorView2D input, int n, IntPtr[] gate, IntPtr[] up, IntPtr[] down,
            int gateType, long gateNe0, long gateNe1, long gateBytes, int upType, long upNe0, long upNe1, long upBytes,
            int downType, long downNe0, long downNe1, long downBytes, float[] routeWeights, bool useShared,
            IntPtr shGate, IntPtr shUp, IntPtr shDown, int shGateType, long shGateNe0, long shGateNe1, long shGateBytes,
            int shUpType, long shUpNe0, long shUpNe1, long shUpBytes, int shDownType, long shDownNe0, long shDownNe1, long shDownBytes,
            float sharedScalar)
            => Check(TSHip_MoEExpertsSwiGLUResidualF32(residual, input, n, gate, up, down, gateType, gateNe0, gateNe1, gateBytes, upType, upNe0,
                upNe1, upBytes, downType, downNe0, downNe1, downBytes, routeWeights, useShared ? 1 : 0, shGate, shUp, shDown, shGateType,
                shGateNe0, shGateNe1, shGateBytes, shUpType, shUpNe0, shUpNe1, shUpBytes, shDownType, shDownNe0, shDownNe1, shDownBytes,
                sharedScalar), "moe_experts_swiglu_residual");

        internal static void TransformerLayerDecode(IntPtr hidden, int hiddenSize, IntPtr attnNorm,
            IntPtr qkv, int qkvType, long qkvNe0, long qkvNe1, long qkvBytes, IntPtr qNorm, IntPtr kNorm, int headDim,
            IntPtr o, int oType, long oNe0, long oNe1, long oBytes, IntPtr ffnNorm,
            IntPtr gu, int guType, long guNe0, long guNe1, long guBytes, IntPtr down, int downType, long downNe0, long downNe1, long downBytes,
            IntPtr kCache, IntPtr vCache, int numHeads, int numKvHeads, int maxSeqLen, int position, float eps, float ropeBase,
            float ropeFreqScale, int intermediateSize, int ropeMode)
            => Check(TSHip_TransformerLayerDecode(hidden, hiddenSize, attnNorm, qkv, qkvType, qkvNe0, qkvNe1, qkvBytes, qNorm, kNorm, headDim,
                o, oType, oNe0, oNe1, oBytes, ffnNorm, gu, guType, guNe0, guNe1, guBytes, down, downType, downNe0, downNe1, downBytes,
                kCache, vCache, numHeads, numKvHeads, maxSeqLen, position, eps, ropeBase, ropeFreqScale, intermediateSize, ropeMode),
                "transformer_layer_decode");

        internal static void TransformerModelDecode(IntPtr hidden, int hiddenSize, int numLayers,
            IntPtr[] attnNorm, IntPtr[] qkv, IntPtr[] qNorm, IntPtr[] kNorm, IntPtr[] o, IntPtr[] ffnNorm, IntPtr[] gu, IntPtr[] down,
            IntPtr[] kCache, IntPtr[] vCache, int qkvType, long qkvNe0, long qkvNe1, long qkvBytes, int oType, long oNe0, long oNe1, long oBytes,
            int guType, long guNe0, long guNe1, long guBytes, int downType, long downNe0, long downNe1, long downBytes,
            int headDim, int numHeads, int numKvHeads, int maxSeqLen, int position, float eps, float ropeBase, float ropeFreqScale,
            int intermediateSize, int ropeMode)
            => Check(TSHip_TransformerModelDecode(hidden, hiddenSize, numLayers, attnNorm, qkv, qNorm, kNorm, o, ffnNorm, gu, down, kCache, vCache,
                qkvType, qkvNe0, qkvNe1, qkvBytes, oType, oNe0, oNe1, oBytes, guType, guNe0, guNe1, guBytes, downType, downNe0, downNe1,
                downBytes, headDim, numHeads, numKvHeads, maxSeqLen, position, eps, ropeBase, ropeFreqScale, intermediateSize, ropeMode),
                "transformer_model_decode");

        /// <summary>TSHip_DequantizeToF32 codes: 0 ok, -1 bad arguments, -2 unsupported type, -3 device failure.</summary>
        internal static void DequantizeToF32(int ggmlType, IntPtr src, long numElements, IntPtr dst)
        {
            int rc = TSHip_DequantizeToF32(ggmlType, src, numElements, dst);
            if (rc == -2)
                throw new NotSupportedException($"The HIP backend cannot dequantize GGUF tensor type {ggmlType}.");
            if (rc != 0)
                throw new InvalidOperationException($"Native HIP dequantization failed (code {rc}): {LastError("no message")}");
        }
    }
}
