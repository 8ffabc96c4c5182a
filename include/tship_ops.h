/*
 * libTsHipOps — C ABI of the MI355X (gfx950) GGUF quantized-matmul backend.
 *
 * Every entry point mirrors, argument for argument, the export of the reference's
 * native bridge (libGgmlOps, `TSGgml_*`) that a `TensorSharp.Backends.HIP` P/Invoke
 * class would bind instead.  Conventions are the bridge's own:
 *   - cdecl, descriptor structs passed BY VALUE, strides in ELEMENTS;
 *   - int return 1 = ok / 0 = failure, message through TSHip_GetLastError()
 *     (thread-local, valid until the next call on that thread) — except
 *     TSHip_DequantizeToF32*, which keeps the bridge's 0 / -1 / -2 codes;
 *   - nothing throws across the boundary; the caller owns every buffer.
 * Matmul weight types: Q4_0 (2), Q4_1 (3), Q5_0 (6), Q5_1 (7), Q8_0 (8), Q4_K (12), Q5_K (13), Q6_K (14), IQ4_NL (20),
 * MXFP4 (39) - the block formats of ManagedQuantizedOps.cs:40-59 without Q8_1.  Dequantize / row gather additionally
 * read F16 (1) and BF16 (30).  (ids: TensorSharp.Runtime/GgufReader.cs:26-37)
 *
 * Two families:
 *   host-pointer entry points   drop-in for the bridge (activations/results in host
 *                               memory, weights device-resident after preload);
 *   *Device entry points        same contracts with every pointer in device memory;
 *                               pure kernel launches on the stream set by TSHip_SetStream.
 * Concurrency: host-pointer entry points serialise on one lock (which also orders them against Invalidate / Clear /
 * Preload, so a device copy is never freed under a running call).  The *Device entry points launch on the calling
 * THREAD's stream (TSHip_SetStream is per thread) and keep their scratch per stream: threads that use different
 * streams run concurrently, threads that share a stream are serialised while they enqueue.
 * Operands beyond 2 GiB (a weight, or the fp16 copy of a call's activations) are cut by rows inside the call.
 */
#ifndef TSHIP_OPS_H
#define TSHIP_OPS_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TSHIP_EXPORT __attribute__((visibility("default")))

/* Backend ids. 1..3 are the bridge's (TensorSharp.Backends.GGML/GgmlNative.cs:20-25); 4 is new. */
enum { TSHIP_BACKEND_METAL = 1, TSHIP_BACKEND_CPU = 2, TSHIP_BACKEND_CUDA = 3, TSHIP_BACKEND_HIP = 4 };

enum {
    TSHIP_TYPE_F32 = 0, TSHIP_TYPE_F16 = 1, TSHIP_TYPE_Q4_0 = 2, TSHIP_TYPE_Q4_1 = 3, TSHIP_TYPE_Q5_0 = 6, TSHIP_TYPE_Q5_1 = 7,
    TSHIP_TYPE_Q8_0 = 8, TSHIP_TYPE_Q4_K = 12, TSHIP_TYPE_Q5_K = 13, TSHIP_TYPE_Q6_K = 14, TSHIP_TYPE_IQ4_NL = 20,
    TSHIP_TYPE_BF16 = 30, TSHIP_TYPE_MXFP4 = 39
};

/* TensorSharp.GGML.Native/ggml_ops_internal.h:69-77 == GgmlNative.cs:27-45 (GgmlTensorView2D). */
typedef struct TSHipTensorView2D {
    void* data;
    int dim0;
    int dim1;
    int stride0;
    int stride1;
    int64_t raw_bytes;
} TSHipTensorView2D;

/* ggml_ops_internal.h TensorView3DDesc == GgmlNative.cs:49-71 (GgmlTensorView3D): strides in elements. */
typedef struct TSHipTensorView3D {
    void* data;
    int dim0;
    int dim1;
    int dim2;
    int stride0;
    int stride1;
    int stride2;
    int64_t raw_bytes;
} TSHipTensorView3D;

/* ggml_ops_internal.h:104-109 == GgmlNative.cs:100-113 (GgmlContiguousTensor). element_type: 0 = F32, 3 = I32. */
typedef struct TSHipContiguousTensor {
    void* data;
    int64_t element_count;
    int element_type;
} TSHipContiguousTensor;

/* ---- utilities -------------------------------------------------------------------- */

/* replaces TSGgml_GetLastError (ggml_ops_core.cpp:1117-1120; GgmlNative.cs:211-212) */
TSHIP_EXPORT const char* TSHip_GetLastError(void);

/* replaces TSGgml_CanInitializeBackend (ggml_ops_core.cpp:1128-1132): 1 iff backendType == HIP and a gfx950
 * device answers; does not initialise anything. */
TSHIP_EXPORT int TSHip_CanInitializeBackend(int backendType);

/* replaces TSGgml_IsBackendAvailable (ggml_ops_core.cpp:1134-1138): initialises the process-wide backend. */
TSHIP_EXPORT int TSHip_IsBackendAvailable(int backendType);

/* replaces TSGgml_RowSize (ggml_ops_core.cpp:1320-1329): bytes of one row, 0 on any error. */
TSHIP_EXPORT size_t TSHip_RowSize(int ggml_type, int64_t ne);

/* replace TSGgml_AlignedAlloc / TSGgml_AlignedFree (ggml_ops_core.cpp:1140-1164): 16384-byte aligned host memory. */
TSHIP_EXPORT void* TSHip_AlignedAlloc(size_t size);
TSHIP_EXPORT void TSHip_AlignedFree(void* ptr);

/* ---- host-pointer entry points (drop-in) ------------------------------------------- */

/* replaces TSGgml_DequantizeToF32 (ggml_ops_core.cpp:1331-1354; GgmlNative.cs:1493-1536).
 * 0 ok, -1 bad arguments, -2 unsupported type.  Bit-exact with ManagedQuantizedOps.cs:411-427/447-479/579-598. */
TSHIP_EXPORT int TSHip_DequantizeToF32(int ggml_type, const void* src, int64_t num_elements, float* dst);

/* replaces TSGgml_AddmmQuantF32 (ggml_ops_matmul.cpp:1308-1337, impl :293-516; GgmlNative.cs:231-240).
 * result[M x N] = m1[M x K] * W[N x K]^T (overwrites).  m2_data is a readable host pointer to the raw GGUF
 * blocks or a key previously passed to TSHip_PreloadQuantizedWeight. */
TSHIP_EXPORT int TSHip_AddmmQuantF32(TSHipTensorView2D result, TSHipTensorView2D m1, void* m2_data,
                                     int m2_ggml_type, int64_t m2_ne0, int64_t m2_ne1, int64_t m2_raw_bytes);

/* replaces TSGgml_AddmmQuantBatchF32 (ggml_ops_matmul.cpp:1370-1401, impl :672-729): row b of m1 times the
 * sub-weight at byte offset weight_offsets[b] with weight_ne1[b] rows -> the first weight_ne1[b] columns of row b of
 * result.  m2_data may be a preload key: sub-weights are then served from the device copy of the whole stack. */
TSHIP_EXPORT int TSHip_AddmmQuantBatchF32(TSHipTensorView2D result, TSHipTensorView2D m1, void* m2_data,
                                          int m2_ggml_type, int64_t m2_ne0, int64_t m2_raw_bytes,
                                          int batch_count, int64_t* weight_offsets, int64_t* weight_ne1_arr);

/* replaces TSGgml_PreloadQuantizedWeight (ggml_ops_core.cpp:1199-1318): upload once, keep the device copy
 * under cache_key; the host bytes may be released afterwards. */
TSHIP_EXPORT int TSHip_PreloadQuantizedWeight(void* cache_key, void* host_data, int ggml_type, int64_t ne0,
                                              int64_t ne1, int64_t raw_bytes);

/* replace TSGgml_InvalidateHostBuffer / TSGgml_ClearHostBufferCache / TSGgml_SyncHostBuffer
 * (ggml_ops_core.cpp:1166-1197).  SyncHostBuffer copies a device copy made from caller memory back to it; as in the
 * bridge (ggml_ops_core.cpp:664-684) it succeeds without doing anything for a null pointer, a zero size, a pointer
 * that was never cached or a preload key, and fails only when `size` exceeds the cached bytes or the copy fails. */
TSHIP_EXPORT void TSHip_InvalidateHostBuffer(void* ptr);
TSHIP_EXPORT void TSHip_ClearHostBufferCache(void);
TSHIP_EXPORT int TSHip_SyncHostBuffer(void* ptr, size_t size);

/* ---- device-pointer entry points ---------------------------------------------------- */

/* No counterpart in the bridge (its tensors are host memory): selects the HIP stream the *Device entry
 * points launch on when called from THIS thread (NULL = default stream, the initial setting of every thread). */
TSHIP_EXPORT int TSHip_SetStream(void* hip_stream);

/* Device form of TSGgml_DequantizeToF32 (same codes). */
TSHIP_EXPORT int TSHip_DequantizeToF32Device(int ggml_type, const void* src, int64_t num_elements, float* dst);

/* Device form of TSGgml_AddmmQuantF32: result.data, m1.data and m2_data are device pointers; both views
 * need stride1 == 1.  Asynchronous on the current stream. */
TSHIP_EXPORT int TSHip_AddmmQuantF32Device(TSHipTensorView2D result, TSHipTensorView2D m1, const void* m2_data,
                                           int m2_ggml_type, int64_t m2_ne0, int64_t m2_ne1,
                                           int64_t m2_raw_bytes);

/* No counterpart in the reference.  TSHip_AddmmQuantF32Device for callers that cannot allocate device memory (code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc): the same kernels and the same
 * results, but the scratch of the prefill path (fp16 activations + row scales, sums of K chunks) lives in a static
 * device array of TSHIP_NO_ALLOC_SCRATCH_BYTES that every GPU the library runs on holds until the process ends; the
 * call makes no hipMalloc / hipFree.  A call whose converted activations (about 2 bytes per activation + 4 per row)
 * exceed the array fails with an error; when only the sums of K chunks do not fit, the launch runs with whole K per
 * tile (results then agree with TSHip_AddmmQuantF32Device to fp32 summation order) or, for the shapes that cannot
 * do without chunks (at most 128 rows with K > 4096 ... 32768 depending on the format), fails with an error.
 * All calls on one GPU share the array: calls that overlap on one GPU (two streams, two threads) race. */
#define TSHIP_NO_ALLOC_SCRATCH_BYTES (64u << 20)
TSHIP_EXPORT int TSHip_AddmmQuantF32DeviceNoAlloc(TSHipTensorView2D result, TSHipTensorView2D m1, const void* m2_data,
                                                  int m2_ggml_type, int64_t m2_ne0, int64_t m2_ne1,
                                                  int64_t m2_raw_bytes);

/* No counterpart in the bridge: the reference issues one AddmmQuant per projection from C#
 * (ModelBase.LinearForward, TensorSharp.Models/ModelBase.cs:875-905).  `count` independent
 * AddmmQuantF32Device problems of one block type; when every problem is a decode GEMV (M == 1) and
 * count <= 8 they are served by ONE kernel launch, otherwise they run back to back.  Results equal those of
 * one TSHip_AddmmQuantF32Device call per problem up to fp32 summation order. */
TSHIP_EXPORT int TSHip_AddmmQuantGroupF32Device(int count, const TSHipTensorView2D* results,
                                                const TSHipTensorView2D* m1s, const void* const* m2_datas,
                                                int m2_ggml_type, const int64_t* m2_ne0s, const int64_t* m2_ne1s,
                                                const int64_t* m2_raw_bytes);

/* ---- fused wrappers around the matmul ------------------------------------------------------ */

/* replaces TSGgml_FusedRmsNormMatMulQuantF32 (ggml_ops_fused.cpp:21-217, :1380-1400; GgmlNative.cs:243-253, :903-912;
 * caller Qwen35Model.cs:1492): result[M x ne1] = (RMSNorm(input, eps) * norm_weight) * W^T, RMSNorm as ggml_rms_norm
 * (sum of squares in double, 1/sqrtf(mean + eps)).  Host pointers, weight cached like TSHip_AddmmQuantF32. */
TSHIP_EXPORT int TSHip_FusedRmsNormMatMulQuantF32(TSHipTensorView2D result, TSHipTensorView2D input, void* norm_weight_data,
                                                  int norm_weight_count, float eps, void* m2_data, int m2_ggml_type,
                                                  int64_t m2_ne0, int64_t m2_ne1, int64_t m2_raw_bytes);

/* replaces TSGgml_FusedMatMulQuantAddF32 (ggml_ops_fused.cpp:219-388, :1410-1430; GgmlNative.cs:256-263, :914-920; caller
 * Qwen35Model.cs:1615): residual[M x ne1] += input * W^T, in place. */
TSHIP_EXPORT int TSHip_FusedMatMulQuantAddF32(TSHipTensorView2D residual, TSHipTensorView2D input, void* m2_data,
                                              int m2_ggml_type, int64_t m2_ne0, int64_t m2_ne1, int64_t m2_raw_bytes);

/* replaces TSGgml_FusedFFNSwiGLUQuantF32 (ggml_ops_fused.cpp:390-640, :1440-1480; GgmlNative.cs:266-283, :922-937; caller
 * Qwen35Model.cs:1663): residual += W_down * ( silu(g) * u ), [g | u] = W_gate_up * (RMSNorm(input, eps) * norm_weight),
 * g the first half_dim outputs, u the next half_dim; silu(g) = g / (1 + expf(-g)). */
TSHIP_EXPORT int TSHip_FusedFFNSwiGLUQuantF32(TSHipTensorView2D residual, TSHipTensorView2D input, void* norm_weight_data,
                                              int norm_weight_count, float eps, void* gate_up_data, int gate_up_ggml_type,
                                              int64_t gate_up_ne0, int64_t gate_up_ne1, int64_t gate_up_raw_bytes,
                                              void* down_data, int down_ggml_type, int64_t down_ne0, int64_t down_ne1,
                                              int64_t down_raw_bytes, int half_dim);

/* device-pointer forms of the three (every pointer in device memory, asynchronous on the selected stream; they use the
 * grow-only device workspace). */
TSHIP_EXPORT int TSHip_FusedRmsNormMatMulQuantF32Device(TSHipTensorView2D result, TSHipTensorView2D input,
                                                        const float* norm_weight, int norm_weight_count, float eps,
                                                        const void* m2_data, int m2_ggml_type, int64_t m2_ne0,
                                                        int64_t m2_ne1, int64_t m2_raw_bytes);
TSHIP_EXPORT int TSHip_FusedMatMulQuantAddF32Device(TSHipTensorView2D residual, TSHipTensorView2D input, const void* m2_data,
                                                    int m2_ggml_type, int64_t m2_ne0, int64_t m2_ne1, int64_t m2_raw_bytes);
TSHIP_EXPORT int TSHip_FusedFFNSwiGLUQuantF32Device(TSHipTensorView2D residual, TSHipTensorView2D input,
                                                    const float* norm_weight, int norm_weight_count, float eps,
                                                    const void* gate_up_data, int gate_up_ggml_type, int64_t gate_up_ne0,
                                                    int64_t gate_up_ne1, int64_t gate_up_raw_bytes, const void* down_data,
                                                    int down_ggml_type, int64_t down_ne0, int64_t down_ne1,
                                                    int64_t down_raw_bytes, int half_dim);

/* replaces TSGgml_FusedOutProjFFNQuantF32 (ggml_ops_fused.cpp:1057-1220; GgmlNative.cs:303-309; GgmlBasicOps.cs:449-480):
 *   residual [M x hidden] += input [M x out_ne0] * W_out^T
 *   residual += W_down * ( silu(g) * u ),  [g | u] = W_gate_up * (RMSNorm(residual, eps) * ffn_norm)
 * in place on residual; host pointers, weights cached like TSHip_AddmmQuantF32. */
TSHIP_EXPORT int TSHip_FusedOutProjFFNQuantF32(TSHipTensorView2D residual, TSHipTensorView2D input, void* out_proj_data,
                                               int out_proj_type, int64_t out_ne0, int64_t out_ne1, int64_t out_raw_bytes,
                                               void* ffn_norm_data, int ffn_norm_count, float eps, void* gu_data, int gu_type,
                                               int64_t gu_ne0, int64_t gu_ne1, int64_t gu_raw_bytes, void* dn_data, int dn_type,
                                               int64_t dn_ne0, int64_t dn_ne1, int64_t dn_raw_bytes, int half_dim);

/* replaces TSGgml_FusedOutProjNormRouterQuantF32 (ggml_ops_fused.cpp:1223-1380; GgmlNative.cs:285-292;
 * GgmlBasicOps.cs:416-447):
 *   residual += input * W_out^T;  normed_out = RMSNorm(residual, eps) * norm;  router_out = normed_out * W_router^T
 * three outputs: residual (in place), normed_out [M x hidden], router_out [M x router_ne1].  The router weight is
 * usually dense: F32, F16 and BF16 weights are accepted beside the block formats. */
TSHIP_EXPORT int TSHip_FusedOutProjNormRouterQuantF32(TSHipTensorView2D residual, TSHipTensorView2D input, void* out_proj_data,
                                                      int out_proj_type, int64_t out_ne0, int64_t out_ne1, int64_t out_raw_bytes,
                                                      void* norm_data, int norm_count, float eps, TSHipTensorView2D normed_out,
                                                      void* router_data, int router_type, int64_t router_ne0,
                                                      int64_t router_ne1, int64_t router_raw_bytes, TSHipTensorView2D router_out);

/* device-pointer forms of the two: asynchronous on the selected stream; normed_out must be contiguous. */
TSHIP_EXPORT int TSHip_FusedOutProjFFNQuantF32Device(TSHipTensorView2D residual, TSHipTensorView2D input, const void* out_proj_data,
                                                     int out_proj_type, int64_t out_ne0, int64_t out_ne1, int64_t out_raw_bytes,
                                                     const float* ffn_norm_weight, int ffn_norm_count, float eps,
                                                     const void* gu_data, int gu_type, int64_t gu_ne0, int64_t gu_ne1,
                                                     int64_t gu_raw_bytes, const void* dn_data, int dn_type, int64_t dn_ne0,
                                                     int64_t dn_ne1, int64_t dn_raw_bytes, int half_dim);
TSHIP_EXPORT int TSHip_FusedOutProjNormRouterQuantF32Device(TSHipTensorView2D residual, TSHipTensorView2D input,
                                                            const void* out_proj_data, int out_proj_type, int64_t out_ne0,
                                                            int64_t out_ne1, int64_t out_raw_bytes, const float* norm_weight,
                                                            int norm_count, float eps, TSHipTensorView2D normed_out,
                                                            const void* router_data, int router_type, int64_t router_ne0,
                                                            int64_t router_ne1, int64_t router_raw_bytes,
                                                            TSHipTensorView2D router_out);

/* ---- weighted expert sets: the bridge's per-token MoE calls ---------------------------------- */

/* replaces TSGgml_MoEExpertsForwardF32 (ggml_ops_fused.cpp:1576-1760; GgmlNative.cs:333-347; GgmlBasicOps.cs:586-613;
 * Nemotron experts): result = sum_e route_weights[e] * W_down[e] * max(W_up[e] * input, 0)^2 over the num_experts
 * (1..16) selected experts, added in index order.  The pointer arrays and route_weights are host arrays; each expert's
 * blocks are cached on the device under their host address like any weight.  One token runs as grouped GEMV
 * launches; more rows of block-format experts run every linear as one tile-table GEMM over the experts' pointers (dense
 * or Q8_1 experts: expert by expert through the matmul path). */
TSHIP_EXPORT int TSHip_MoEExpertsForwardF32(TSHipTensorView2D result, TSHipTensorView2D input, int num_experts,
                                            void** up_data_ptrs, void** down_data_ptrs, int up_ggml_type, int64_t up_ne0,
                                            int64_t up_ne1, int64_t up_raw_bytes_each, int down_ggml_type, int64_t down_ne0,
                                            int64_t down_ne1, int64_t down_raw_bytes_each, float* route_weights);

/* replaces TSGgml_MoEExpertsSwiGLUForwardF32 (ggml_ops_fused.cpp:1766-1940; GgmlNative.cs:350-369;
 * GgmlBasicOps.cs:615-645): result = sum_e route_weights[e] * W_down[e] * ( silu(W_gate[e] x) * (W_up[e] x) ),
 * num_experts 1..32 as in the bridge (ggml_ops_fused.cpp:1795-1799; only the squared-ReLU form above stops at 16). */
TSHIP_EXPORT int TSHip_MoEExpertsSwiGLUForwardF32(TSHipTensorView2D result, TSHipTensorView2D input, int num_experts,
                                                  void** gate_data_ptrs, void** up_data_ptrs, void** down_data_ptrs,
                                                  int gate_ggml_type, int64_t gate_ne0, int64_t gate_ne1,
                                                  int64_t gate_raw_bytes_each, int up_ggml_type, int64_t up_ne0, int64_t up_ne1,
                                                  int64_t up_raw_bytes_each, int down_ggml_type, int64_t down_ne0,
                                                  int64_t down_ne1, int64_t down_raw_bytes_each, float* route_weights);

/* replaces TSGgml_MoEExpertsSwiGLUResidualF32 (ggml_ops_fused.cpp:1953-2160; GgmlNative.cs:372-408;
 * GgmlBasicOps.cs:647-700; Qwen3.5 MoE decode): residual += sum_e route_weights[e] * expert_e(input)
 * [+ shared_scalar * shared_expert(input)], num_experts 1..32.  The shared expert takes part only when use_shared is
 * non-zero and its three pointers are non-null; it may have its own types and intermediate width. */
TSHIP_EXPORT int TSHip_MoEExpertsSwiGLUResidualF32(
    TSHipTensorView2D residual, TSHipTensorView2D input, int num_experts, void** gate_data_ptrs, void** up_data_ptrs,
    void** down_data_ptrs, int gate_ggml_type, int64_t gate_ne0, int64_t gate_ne1, int64_t gate_raw_bytes_each, int up_ggml_type,
    int64_t up_ne0, int64_t up_ne1, int64_t up_raw_bytes_each, int down_ggml_type, int64_t down_ne0, int64_t down_ne1,
    int64_t down_raw_bytes_each, float* route_weights, int use_shared, void* shared_gate_data, void* shared_up_data,
    void* shared_down_data, int shared_gate_ggml_type, int64_t shared_gate_ne0, int64_t shared_gate_ne1,
    int64_t shared_gate_raw_bytes, int shared_up_ggml_type, int64_t shared_up_ne0, int64_t shared_up_ne1,
    int64_t shared_up_raw_bytes, int shared_down_ggml_type, int64_t shared_down_ne0, int64_t shared_down_ne1,
    int64_t shared_down_raw_bytes, float shared_scalar);

/* device-pointer forms of the three: the tensors and every weight pointer are device memory, the pointer arrays and
 * route_weights stay host arrays (read before the call returns); asynchronous on the selected stream. */
TSHIP_EXPORT int TSHip_MoEExpertsForwardF32Device(TSHipTensorView2D result, TSHipTensorView2D input, int num_experts,
                                                  void* const* up_data_ptrs, void* const* down_data_ptrs, int up_ggml_type,
                                                  int64_t up_ne0, int64_t up_ne1, int64_t up_raw_bytes_each, int down_ggml_type,
                                                  int64_t down_ne0, int64_t down_ne1, int64_t down_raw_bytes_each,
                                                  const float* route_weights);
TSHIP_EXPORT int TSHip_MoEExpertsSwiGLUForwardF32Device(TSHipTensorView2D result, TSHipTensorView2D input, int num_experts,
                                                        void* const* gate_data_ptrs, void* const* up_data_ptrs,
                                                        void* const* down_data_ptrs, int gate_ggml_type, int64_t gate_ne0,
                                                        int64_t gate_ne1, int64_t gate_raw_bytes_each, int up_ggml_type,
                                                        int64_t up_ne0, int64_t up_ne1, int64_t up_raw_bytes_each,
                                                        int down_ggml_type, int64_t down_ne0, int64_t down_ne1,
                                                        int64_t down_raw_bytes_each, const float* route_weights);
TSHIP_EXPORT int TSHip_MoEExpertsSwiGLUResidualF32Device(
    TSHipTensorView2D residual, TSHipTensorView2D input, int num_experts, void* const* gate_data_ptrs, void* const* up_data_ptrs,
    void* const* down_data_ptrs, int gate_ggml_type, int64_t gate_ne0, int64_t gate_ne1, int64_t gate_raw_bytes_each,
    int up_ggml_type, int64_t up_ne0, int64_t up_ne1, int64_t up_raw_bytes_each, int down_ggml_type, int64_t down_ne0,
    int64_t down_ne1, int64_t down_raw_bytes_each, const float* route_weights, int use_shared, void* shared_gate_data,
    void* shared_up_data, void* shared_down_data, int shared_gate_ggml_type, int64_t shared_gate_ne0, int64_t shared_gate_ne1,
    int64_t shared_gate_raw_bytes, int shared_up_ggml_type, int64_t shared_up_ne0, int64_t shared_up_ne1,
    int64_t shared_up_raw_bytes, int shared_down_ggml_type, int64_t shared_down_ne0, int64_t shared_down_ne1,
    int64_t shared_down_raw_bytes, float shared_scalar);

/* replaces TSGgml_MulMatIdF32 (ggml_ops_matmul.cpp:958-1121, :1427-1449; GgmlNative.cs:433-439, :1076-1079): ggml_mul_mat_id
 * with F32 expert weights, not a quantized path.  expert_weights [E x rows x K], input [T x slots x K], ids [ids_rows x
 * ids_cols] (I32, or F32 truncated) with ids_rows == T and ids_cols a multiple of slots;
 *   result[t][s][r] = sum_k expert_weights[ids[t][s]][r][k] * input[t][s % slots][k],  result [T x ids_cols x rows].
 * Host pointers, standard views (innermost stride 1, no overlap); like the bridge the weights travel on every call
 * (nothing is cached).  An id outside [0, E) is an error (the bridge's ggml asserts). */
TSHIP_EXPORT int TSHip_MulMatIdF32(TSHipTensorView3D result, TSHipTensorView3D expert_weights, TSHipTensorView3D input,
                                   TSHipContiguousTensor ids, int ids_rows, int ids_cols);

/* device-pointer form: ids is a device array of ids_rows x ids_cols int32; rows of an out-of-range id are zero;
 * any number of (token, slot) pairs (cut into launches of 65535).  Asynchronous on the selected stream. */
TSHIP_EXPORT int TSHip_MulMatIdF32Device(TSHipTensorView3D result, TSHipTensorView3D expert_weights, TSHipTensorView3D input,
                                         const int32_t* ids, int ids_rows, int ids_cols);

/* Diagnostics, no counterpart in the reference: while a device buffer is set, the single-row (GEMV) launches of the plain
 * activation mode run a build of the kernel in which every wavefront writes 64-bit words at byte offset
 * 64 * (workgroup * 8 + wavefront) of the buffer: the 100 MHz constant-clock times of [0] its entry, [1] the arrival of its
 * activations, [2] the barrier behind the staging, [3] the end of its first weight step, [4] its exit, and [5] (XCC id |
 * problem index << 8 | wavefront index << 16).  Launches with more wavefronts than capacity_bytes / 64 run the normal kernel.  Pass a null buffer to switch it off.  For profiling runs only
 * (bench.py --timeline); not thread-safe. */
TSHIP_EXPORT int TSHip_SetGemvTimeline(void* device_buffer, int64_t capacity_bytes);

/* replaces TSGgml_AddIdF32 (ggml_ops_matmul.cpp:1123-1290, :1451-1473; GgmlNative.cs:442-448, :1081-1084; managed
 * GgmlBasicOps.AddID :1092-1108): ggml_add_id, the per-expert bias that goes with a mul_mat_id,
 *   result[t][s][r] = src[t][s][r] + bias[ids[t][s]][r],  src / result [T x ids_cols x rows], bias [E x rows],
 * ids [ids_rows x ids_cols] (I32, or F32 truncated) with ids_rows == T.  Host pointers, standard views.  An id outside
 * [0, E) is an error (the bridge's ggml asserts). */
TSHIP_EXPORT int TSHip_AddIdF32(TSHipTensorView3D result, TSHipTensorView3D src, TSHipTensorView2D bias, TSHipContiguousTensor ids,
                                int ids_rows, int ids_cols);

/* device-pointer form: ids is a device array of ids_rows x ids_cols int32 (a pair with an id outside [0, E) gets no
 * bias); result may be src (in place).  Asynchronous on the selected stream. */
TSHIP_EXPORT int TSHip_AddIdF32Device(TSHipTensorView3D result, TSHipTensorView3D src, TSHipTensorView2D bias, const int32_t* ids,
                                      int ids_rows, int ids_cols);

/* replaces TSGgml_GetRowsQuantF32 (ggml_ops_matmul.cpp:519-668, :1339-1368; GgmlNative.cs:324, :1003-1006; caller
 * ModelBase.cs:826-856 embedding lookup): result[i, 0..ne0) = dequantized row indices[i] of the [ne1 x ne0] source
 * (type F32 copies rows).  Host pointers; the source is cached on the device by pointer / preload key like the
 * matmul weight.  result must be a standard view [num_indices x ne0]; indices I32 (or F32, truncated).  An index
 * outside [0, ne1) is an error (the bridge's ggml_get_rows asserts). */
TSHIP_EXPORT int TSHip_GetRowsQuantF32(TSHipTensorView2D result, void* src_data, int src_ggml_type, int64_t src_ne0,
                                       int64_t src_ne1, int64_t src_raw_bytes, TSHipContiguousTensor indices);

/* device-pointer form of the same: asynchronous on the selected stream; rows of out-of-range indices are zero. */
TSHIP_EXPORT int TSHip_GetRowsQuantF32Device(TSHipTensorView2D result, const void* src_data, int src_ggml_type,
                                             int64_t src_ne0, int64_t src_ne1, int64_t src_raw_bytes,
                                             const int32_t* indices, int64_t num_indices);

/* No bridge export: the reference routes in C# (GptOssModel.MoERoute, TensorSharp.Models/Models/GptOss/GptOssModel.cs:814-865,
 * the part after the router linear).  logits [T x E] -> ids / weights [T x k]: top-k by repeated argmax (first
 * maximum wins ties), softmax over the k selected logits.  1 <= k <= 16. */
TSHIP_EXPORT int TSHip_MoERouteF32Device(TSHipTensorView2D logits, int k, int32_t* ids, float* weights);

/* No bridge export: replaces the per-expert C# loop GptOssModel.MoEForwardSingleToken / MoEForwardBatched / ExpertFFN
 * (GptOssModel.cs:718-812, :867-934) that issues two AddmmQuant calls per expert.
 *   result[t] = sum_s weights[t,s] * ( W_down[e] * swiglu_oai( W_gate_up[e] * hidden[t] + b_gate_up[e] ) + b_down[e] ),
 *   e = ids[t,s]
 * gate_up_w: [E][2F rows][H] raw blocks (gate rows, then up rows), down_w: [E][H rows][F]; biases [E][2F] / [E][H] or
 * NULL.  Few assignments (T*k <= 8) run as grouped decode GEMVs with the expert picked on the device; otherwise the
 * assignments are counting-sorted by expert on the device and each linear is ONE grouped MFMA GEMM launch.
 * Accumulation order over experts: ascending expert id for T > 1, selection order for T == 1 (as the reference). */
TSHIP_EXPORT int TSHip_MoEExpertsGptOssForwardF32Device(TSHipTensorView2D result, TSHipTensorView2D hidden, const int32_t* ids,
                                                  const float* weights, int k, const void* gate_up_w,
                                                  const float* gate_up_bias, const void* down_w, const float* down_bias,
                                                  int ggml_type, int n_experts, int64_t H, int64_t F, float alpha,
                                                  float limit);

/* replaces TSGgml_TransformerLayerDecode (TensorSharp.GGML.Native/ggml_ops_transformer.cpp:318-470, :572-600;
 * GgmlNative.cs:518-531): one token through one transformer layer with every pointer in DEVICE memory.
 *   x   = RMSNorm(hidden) * attn_norm;  [q | k | v] = W_qkv x            (q: num_heads heads, k / v: num_kv_heads)
 *   q, k: per-head RMSNorm * q_norm / k_norm (skipped when the pointer is NULL), RoPE at `position`
 *         (rope_mode 0: adjacent pairs, 2: NeoX halves; n_dims = head_dim)
 *   k, v -> row `position` of the fp32 caches [num_kv_heads][max_seq_len][head_dim]
 *   a   = softmax(q K^T / sqrt(head_dim)) V over rows 0..position, grouped-query heads sharing their KV head
 *   hidden += W_o a;  hidden += W_down( silu(g) * u ), [g | u] = W_gate_up (RMSNorm(hidden) * ffn_norm)
 * hidden [hidden_size] is updated in place.  Same argument list as the bridge export. */
TSHIP_EXPORT int TSHip_TransformerLayerDecodeDevice(float* hidden, int hidden_size, const float* attn_norm, const void* qkv_data,
                                                    int qkv_type, int64_t qkv_ne0, int64_t qkv_ne1, int64_t qkv_bytes,
                                                    const float* q_norm, const float* k_norm, int head_dim, const void* o_data,
                                                    int o_type, int64_t o_ne0, int64_t o_ne1, int64_t o_bytes, const float* ffn_norm,
                                                    const void* gu_data, int gu_type, int64_t gu_ne0, int64_t gu_ne1, int64_t gu_bytes,
                                                    const void* down_data, int down_type, int64_t down_ne0, int64_t down_ne1,
                                                    int64_t down_bytes, float* k_cache, float* v_cache, int num_heads,
                                                    int num_kv_heads, int max_seq_len, int position, float eps, float rope_base,
                                                    float rope_freq_scale, int intermediate_size, int rope_mode);

/* replaces TSGgml_TransformerModelDecode (ggml_ops_transformer.cpp:1040-1230; GgmlNative.cs:647-659): the same for
 * num_layers layers in sequence; the arrays (host memory) hold one device pointer per layer, shapes and types are shared. */
TSHIP_EXPORT int TSHip_TransformerModelDecodeDevice(float* hidden, int hidden_size, int num_layers, const float* const* attn_norm,
                                                    const void* const* qkv, const float* const* q_norm, const float* const* k_norm,
                                                    const void* const* o, const float* const* ffn_norm, const void* const* gu,
                                                    const void* const* down, float* const* k_cache, float* const* v_cache,
                                                    int qkv_type, int64_t qkv_ne0, int64_t qkv_ne1, int64_t qkv_bytes, int o_type,
                                                    int64_t o_ne0, int64_t o_ne1, int64_t o_bytes, int gu_type, int64_t gu_ne0,
                                                    int64_t gu_ne1, int64_t gu_bytes, int down_type, int64_t down_ne0,
                                                    int64_t down_ne1, int64_t down_bytes, int head_dim, int num_heads,
                                                    int num_kv_heads, int max_seq_len, int position, float eps, float rope_base,
                                                    float rope_freq_scale, int intermediate_size, int rope_mode);

/* replaces TSGgml_TransformerLayerDecode with the bridge's own HOST pointers (GgmlNative.cs:518-531; argument list of
 * ggml_ops_transformer.cpp:572-600).  hidden [hidden_size] travels host -> device -> host on every call.  Every other
 * buffer - norm weights, raw weight blocks, the two fp32 KV caches - is kept on the device under the host pointer
 * passed (uploaded the first time that pointer is seen, the protocol of the bridge's cacheable buffers,
 * ggml_ops_transformer.cpp:244-300).  The device copy of a KV cache is the one this call updates:
 * TSHip_SyncHostBuffer(k_cache, bytes) copies it back to host memory, TSHip_InvalidateHostBuffer(ptr) drops a device
 * copy so that the next call uploads the host bytes again (after the caller has edited or truncated the cache).
 * Synchronous; runs on the default stream. */
TSHIP_EXPORT int TSHip_TransformerLayerDecode(void* hidden, int hidden_size, void* attn_norm, void* qkv_data, int qkv_type,
                                              int64_t qkv_ne0, int64_t qkv_ne1, int64_t qkv_bytes, void* q_norm, void* k_norm,
                                              int head_dim, void* o_data, int o_type, int64_t o_ne0, int64_t o_ne1, int64_t o_bytes,
                                              void* ffn_norm, void* gu_data, int gu_type, int64_t gu_ne0, int64_t gu_ne1,
                                              int64_t gu_bytes, void* down_data, int down_type, int64_t down_ne0, int64_t down_ne1,
                                              int64_t down_bytes, void* k_cache, void* v_cache, int num_heads, int num_kv_heads,
                                              int max_seq_len, int position, float eps, float rope_base, float rope_freq_scale,
                                              int intermediate_size, int rope_mode);

/* replaces TSGgml_TransformerModelDecode with HOST pointers (GgmlNative.cs:647-659; ggml_ops_transformer.cpp:1040-1230):
 * num_layers layers in sequence with ONE round trip of hidden; the arrays hold one host pointer per layer, cached on
 * the device as above. */
TSHIP_EXPORT int TSHip_TransformerModelDecode(void* hidden, int hidden_size, int num_layers, void* const* attn_norm,
                                              void* const* qkv, void* const* q_norm, void* const* k_norm, void* const* o,
                                              void* const* ffn_norm, void* const* gu, void* const* down, void* const* k_cache,
                                              void* const* v_cache, int qkv_type, int64_t qkv_ne0, int64_t qkv_ne1,
                                              int64_t qkv_bytes, int o_type, int64_t o_ne0, int64_t o_ne1, int64_t o_bytes,
                                              int gu_type, int64_t gu_ne0, int64_t gu_ne1, int64_t gu_bytes, int down_type,
                                              int64_t down_ne0, int64_t down_ne1, int64_t down_bytes, int head_dim, int num_heads,
                                              int num_kv_heads, int max_seq_len, int position, float eps, float rope_base,
                                              float rope_freq_scale, int intermediate_size, int rope_mode);

#ifdef __cplusplus
}
#endif
#endif /* TSHIP_OPS_H */
