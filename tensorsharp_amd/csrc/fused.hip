// Small kernels around the quantized matmul for the bridge's fused entry points
// (TensorSharp.GGML.Native/ggml_ops_fused.cpp:21-640): RMSNorm rows and the SiLU-gated product.
#include "tship_internal.h"

namespace tship {
namespace {

// One workgroup per row.  Follows ggml_compute_forward_rms_norm_f32 (ggml-cpu/ops.cpp:3646-3695): squares in
// fp32, their sum in double, mean and scale = 1/sqrtf(mean + eps) in fp32, then ggml_mul by the weight:
// (x * scale) * w.  (The sum is a tree over the workgroup, the reference adds in index order; in double the
// difference is far below one fp32 ulp of the mean.)
__global__ void __launch_bounds__(256) rms_norm_rows_kernel(const float* __restrict__ x, int64_t ldx, const float* __restrict__ w,
                                                            float eps, int K, float* __restrict__ out)
{
    const float* src = x + (int64_t)blockIdx.x * ldx;
    float* dst = out + (int64_t)blockIdx.x * K;
    __shared__ double red[4];
    double ss = 0.0;
    for (int k = threadIdx.x; k < K; k += 256) ss += (double)(src[k] * src[k]);
    for (int o = 32; o > 0; o >>= 1) ss += __shfl_xor(ss, o);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = ss;
    __syncthreads();
    const float mean = (float)(((red[0] + red[1]) + (red[2] + red[3])) / (double)K);
    const float scale = 1.0f / sqrtf(mean + eps);
    for (int k = threadIdx.x; k < K; k += 256) dst[k] = (src[k] * scale) * w[k];
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
    hipLaunchKernelGGL(rms_norm_rows_kernel, dim3(M), dim3(256), 0, stream, x, ldx, w, eps, K, out);
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
