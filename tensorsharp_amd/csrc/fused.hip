// Small kernels around the quantized matmul for the bridge's fused entry points
// (TensorSharp.GGML.Native/ggml_ops_fused.cpp:21-640): RMSNorm rows and the SiLU-gated product.
#include "tship_internal.h"

namespace tship {
namespace {

// One workgroup of 1024 threads per row.  Follows ggml_compute_forward_rms_norm_f32 (ggml-cpu/ops.cpp:3646-3695):
// squares in fp32, their sum in double, mean and scale = 1/sqrtf(mean + eps) in fp32, then ggml_mul by the weight:
// (x * scale) * w.  (The sum is a tree over the workgroup, the reference adds in index order; in double the
// difference is far below one fp32 ulp of the mean.)  The row is read once: each thread keeps up to kHold float4
// of it in registers; longer rows re-read the rest.
constexpr int kRmsThreads = 1024;
constexpr int kHold = 4;      // 1024 threads x 4 x float4 = 16384 elements held

__global__ void __launch_bounds__(kRmsThreads) rms_norm_rows_kernel(const float* __restrict__ x, int64_t ldx, const float* __restrict__ w,
                                                                    float eps, int K, float* __restrict__ out)
{
    const float* src = x + (int64_t)blockIdx.x * ldx;
    float* dst = out + (int64_t)blockIdx.x * K;
    __shared__ double red[kRmsThreads / 64];
    const int k4 = K >> 2;                       // whole float4 (rows are 16-byte aligned); K % 4 elements handled below
    float4 hold[kHold], wv[kHold];
    double ss = 0.0;
#pragma unroll
    for (int i = 0; i < kHold; ++i) {
        const int q = (int)threadIdx.x + i * kRmsThreads;
        hold[i] = q < k4 ? reinterpret_cast<const float4*>(src)[q] : float4{0.f, 0.f, 0.f, 0.f};
        wv[i] = q < k4 ? reinterpret_cast<const float4*>(w)[q] : float4{0.f, 0.f, 0.f, 0.f};
    }
#pragma unroll
    for (int i = 0; i < kHold; ++i)
        ss += (double)(hold[i].x * hold[i].x) + (double)(hold[i].y * hold[i].y) + (double)(hold[i].z * hold[i].z) +
              (double)(hold[i].w * hold[i].w);
    for (int k = kHold * kRmsThreads * 4 + (int)threadIdx.x; k < K; k += kRmsThreads) ss += (double)(src[k] * src[k]);
    for (int k = (k4 << 2) + (int)threadIdx.x; k < K && k < kHold * kRmsThreads * 4; k += kRmsThreads) ss += (double)(src[k] * src[k]);
    for (int o = 32; o > 0; o >>= 1) ss += __shfl_xor(ss, o);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = ss;
    __syncthreads();
    double tot = 0.0;
#pragma unroll
    for (int i = 0; i < kRmsThreads / 64; ++i) tot += red[i];
    const float mean = (float)(tot / (double)K);
    const float scale = 1.0f / sqrtf(mean + eps);
#pragma unroll
    for (int i = 0; i < kHold; ++i) {
        const int q = (int)threadIdx.x + i * kRmsThreads;
        if (q < k4)
            reinterpret_cast<float4*>(dst)[q] = float4{(hold[i].x * scale) * wv[i].x, (hold[i].y * scale) * wv[i].y,
                                                       (hold[i].z * scale) * wv[i].z, (hold[i].w * scale) * wv[i].w};
    }
    for (int k = kHold * kRmsThreads * 4 + (int)threadIdx.x; k < K; k += kRmsThreads) dst[k] = (src[k] * scale) * w[k];
    for (int k = (k4 << 2) + (int)threadIdx.x; k < K && k < kHold * kRmsThreads * 4; k += kRmsThreads) dst[k] = (src[k] * scale) * w[k];
}

// ggml_silu then ggml_mul (ggml-cpu/vec.h:958-960): silu(g) = g / (1 + expf(-g))
__global__ void __launch_bounds__(256) silu_mul_kernel(const float* __restrict__ gu, int64_t ldgu, int half, float* __restrict__ out)
{
    const int j = blockIdx.x * 256 + threadIdx.x;
    if (j >= half) return;
    const float* row = gu + (int64_t)blockIdx.y * ldgu;
    const float g = row[j], u = row[half + j];
    out[(int64_t)blockIdx.y * half + j] = (g / (1.0f + expf(-g))) * u;
}

}  // namespace

bool launch_rms_norm_rows(const float* x, int64_t ldx, const float* w, float eps, int M, int K, float* out, hipStream_t stream)
{
    if (M <= 0 || K <= 0) return true;
    if ((reinterpret_cast<uintptr_t>(x) & 15) || (reinterpret_cast<uintptr_t>(w) & 15) || (reinterpret_cast<uintptr_t>(out) & 15) ||
        (M > 1 && (ldx & 3)) || (K & 3)) {
        set_last_error("rms_norm: rows and the norm weight must be 16-byte aligned and K a multiple of 4.");
        return false;
    }
    hipLaunchKernelGGL(rms_norm_rows_kernel, dim3(M), dim3(kRmsThreads), 0, stream, x, ldx, w, eps, K, out);
    return hip_ok(hipGetLastError(), "rms_norm launch");
}

bool launch_silu_mul(const float* gu, int64_t ldgu, int M, int half, float* out, hipStream_t stream)
{
    if (M <= 0 || half <= 0) return true;
    if (M > 65535) {
        set_last_error("silu_mul: more than 65535 rows per call.");
        return false;
    }
    hipLaunchKernelGGL(silu_mul_kernel, dim3((half + 255) / 256, M), dim3(256), 0, stream, gu, ldgu, half, out);
    return hip_ok(hipGetLastError(), "silu_mul launch");
}

}  // namespace tship
