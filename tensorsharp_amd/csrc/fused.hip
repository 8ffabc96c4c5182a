// Small kernels around the quantized matmul for the bridge's fused entry points
// (TensorSharp.GGML.Native/ggml_ops_fused.cpp:21-640): RMSNorm rows and the SiLU-gated product.
#include "tship_internal.h"

#include <algorithm>

#include <hip/hip_fp16.h>

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

// squared ReLU in place (Nemotron experts: ggml_relu then ggml_sqr, ggml_ops_fused.cpp:1700-1710)
__global__ void __launch_bounds__(256) relu_sqr_kernel(float* __restrict__ x, int64_t n)
{
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const float v = fmaxf(x[i], 0.f);
    x[i] = v * v;
}

// out[m][j] = (base ? base[m][j] : 0) + sum_e w.v[e] * rows[e * set_stride + m * N + j], experts added in index order as the
// bridge's graph chains its ggml_add nodes (ggml_ops_fused.cpp:1716-1722)
__global__ void __launch_bounds__(256) weighted_sum_kernel(const float* __restrict__ rows, int64_t set_stride, WeightedSumCoeffs w, int count,
                                                          int N, const float* base, int64_t ldb, float* out, int64_t ldo)
{
    const int j = blockIdx.x * 256 + threadIdx.x;
    const int m = blockIdx.y;
    if (j >= N) return;
    float acc = 0.f;
    for (int e = 0; e < count; ++e) {
        const float v = rows[(int64_t)e * set_stride + (int64_t)m * N + j] * w.v[e];
        acc = e == 0 ? v : acc + v;
    }
    out[(int64_t)m * ldo + j] = base ? base[(int64_t)m * ldb + j] + acc : acc;
}

// ---- dense (F32 / F16 / BF16) weights -----------------------------------------------------------
// The block formats are the hot path; dense weights appear as small matrices beside them (an F32 router, an F16 head).
// One wavefront per weight row and up to kDenseRows activation rows per workgroup: the weight row is read once per
// kDenseRows activation rows, fp32 accumulation in k order per lane, then a butterfly over the 64 lanes.
constexpr int kDenseRows = 4;

__device__ inline float dense_elem(const float* w, int64_t i) { return w[i]; }
__device__ inline float dense_elem(const __half* w, int64_t i) { return __half2float(w[i]); }
__device__ inline float dense_elem(const uint16_t* w, int64_t i) { return __uint_as_float((uint32_t)w[i] << 16); }   // bf16

template <typename T>
__global__ void __launch_bounds__(256) dense_matmul_kernel(const T* __restrict__ w, const float* __restrict__ x, int64_t ldx,
                                                          float* __restrict__ y, int64_t ldy, int M, int N, int K, int accumulate)
{
    const int lane = threadIdx.x & 63;
    const int n = blockIdx.x * 4 + (threadIdx.x >> 6);
    const int m0 = blockIdx.y * kDenseRows;
    if (n >= N) return;
    const T* wr = w + (int64_t)n * K;
    float acc[kDenseRows] = {};
    for (int k = lane; k < K; k += 64) {
        const float wv = dense_elem(wr, k);
#pragma unroll
        for (int r = 0; r < kDenseRows; ++r)
            if (m0 + r < M) acc[r] = fmaf(wv, x[(int64_t)(m0 + r) * ldx + k], acc[r]);
    }
#pragma unroll
    for (int r = 0; r < kDenseRows; ++r) {
        float v = acc[r];
        for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
        if (lane == 0 && m0 + r < M) {
            float* dst = y + (int64_t)(m0 + r) * ldy + n;
            *dst = accumulate ? *dst + v : v;
        }
    }
}

// ggml_mul_mat_id with F32 experts (include/ggml.h:1409-1413): out[t][s][r] = sum_k W[ids[t][s]][r][k] * x[t][s % slots][k].
// One wavefront per output row r of one (t, s) pair; rows of an id outside [0, E) are zero.
__global__ void __launch_bounds__(256) mul_mat_id_f32_kernel(const float* __restrict__ w, int64_t w_s0, int64_t w_s1, int E, int rows,
                                                            int K, const float* __restrict__ x, int64_t x_s0, int64_t x_s1, int slots,
                                                            const int32_t* __restrict__ ids, int cols, float* __restrict__ out,
                                                            int64_t o_s0, int64_t o_s1)
{
    const int lane = threadIdx.x & 63;
    const int r = blockIdx.x * 4 + (threadIdx.x >> 6);
    const int t = blockIdx.y / cols, s = blockIdx.y % cols;
    if (r >= rows) return;
    const int e = ids[(int64_t)t * cols + s];
    float acc = 0.f;
    if (e >= 0 && e < E) {
        const float* wr = w + (int64_t)e * w_s0 + (int64_t)r * w_s1;
        const float* xr = x + (int64_t)t * x_s0 + (int64_t)(s % slots) * x_s1;
        for (int k = lane; k < K; k += 64) acc = fmaf(wr[k], xr[k], acc);
    }
    for (int o = 32; o > 0; o >>= 1) acc += __shfl_xor(acc, o);
    if (lane == 0) out[(int64_t)t * o_s0 + (int64_t)s * o_s1 + r] = acc;
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

// Tables of a tile-table GEMM launch over experts held by pointer (every expert sees the same M rows): m-tiles of bm rows
// per expert, the experts' byte offsets from the launch's base pointer, and the row map that repeats the M source rows
// once per member of the set.
__global__ void __launch_bounds__(256) expert_tiles_kernel(ExpertTileSpec s, int M, int bm, int* tile_expert, int* tile_row0, int* tile_rows,
                                                          int64_t* off_table, int* row_map, int map_rows)
{
    const int per = (M + bm - 1) / bm;
    const int i0 = blockIdx.x * 256 + threadIdx.x, step = gridDim.x * 256;
    for (int i = i0; i < s.count * per; i += step) {
        const int e = i / per, j = i - e * per;
        tile_expert[i] = e;
        tile_row0[i] = s.slot[e] * M + j * bm;
        tile_rows[i] = min(bm, M - j * bm);
    }
    for (int i = i0; i < s.count; i += step) off_table[i] = s.off[i];
    if (row_map)
        for (int i = i0; i < map_rows; i += step) row_map[i] = i % M;
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

bool launch_relu_sqr(float* x, int64_t n, hipStream_t stream)
{
    if (n <= 0) return true;
    hipLaunchKernelGGL(relu_sqr_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, x, n);
    return hip_ok(hipGetLastError(), "relu_sqr launch");
}

bool launch_expert_tiles(const ExpertTileSpec& spec, int M, int bm, int* tile_expert, int* tile_row0, int* tile_rows, int64_t* off_table,
                         int* row_map, int map_rows, hipStream_t stream)
{
    if (spec.count < 1 || spec.count > kMaxWeightedRows || M < 1 || bm < 1) {
        set_last_error("expert_tiles: bad expert count or tile height.");
        return false;
    }
    const int items = std::max(spec.count * ((M + bm - 1) / bm), row_map ? map_rows : 0);
    hipLaunchKernelGGL(expert_tiles_kernel, dim3((unsigned)std::min(64, (items + 255) / 256)), dim3(256), 0, stream, spec, M, bm, tile_expert,
                       tile_row0, tile_rows, off_table, row_map, map_rows);
    return hip_ok(hipGetLastError(), "expert_tiles launch");
}

bool launch_weighted_sum(const float* rows, int64_t set_stride, const WeightedSumCoeffs& w, int count, int M, int N, const float* base,
                         int64_t ldb, float* out, int64_t ldo, hipStream_t stream)
{
    if (M <= 0 || N <= 0) return true;
    if (count < 1 || count > kMaxWeightedRows || M > 65535) {
        set_last_error("weighted_sum: bad row-set count or more than 65535 rows.");
        return false;
    }
    hipLaunchKernelGGL(weighted_sum_kernel, dim3((N + 255) / 256, M), dim3(256), 0, stream, rows, set_stride, w, count, N, base, ldb, out, ldo);
    return hip_ok(hipGetLastError(), "weighted_sum launch");
}

bool launch_dense_matmul(int type, const void* w, const float* x, int64_t ldx, float* y, int64_t ldy, int M, int N, int K,
                         bool accumulate, hipStream_t stream)
{
    if (M <= 0 || N <= 0 || K <= 0) return true;
    const dim3 grid((N + 3) / 4, (M + kDenseRows - 1) / kDenseRows);
    if (grid.y > 65535) {
        set_last_error("dense matmul: too many activation rows per call.");
        return false;
    }
    const int acc = accumulate ? 1 : 0;
    switch (type) {
    case kTypeF32:
        hipLaunchKernelGGL(dense_matmul_kernel<float>, grid, dim3(256), 0, stream, static_cast<const float*>(w), x, ldx, y, ldy, M, N, K, acc);
        break;
    case kTypeF16:
        hipLaunchKernelGGL(dense_matmul_kernel<__half>, grid, dim3(256), 0, stream, static_cast<const __half*>(w), x, ldx, y, ldy, M, N, K, acc);
        break;
    case kTypeBF16:
        hipLaunchKernelGGL(dense_matmul_kernel<uint16_t>, grid, dim3(256), 0, stream, static_cast<const uint16_t*>(w), x, ldx, y, ldy, M, N, K, acc);
        break;
    default:
        set_last_error("dense matmul: the weight type is not F32, F16 or BF16.");
        return false;
    }
    return hip_ok(hipGetLastError(), "dense matmul launch");
}

// out[t][s][r] = src[t][s][r] + bias[ids[t][s]][r] (ggml_add_id: ggml.h:886-891); a pair with an id outside the table
// gets no bias (the host entry point refuses such ids before anything is launched)
__global__ void __launch_bounds__(256) add_id_f32_kernel(const float* __restrict__ src, int64_t s_s0, int64_t s_s1, const float* __restrict__ bias,
                                                         int64_t b_s0, int E, const int32_t* __restrict__ ids, int cols, int rows,
                                                         float* __restrict__ out, int64_t o_s0, int64_t o_s1, int64_t pairs)
{
    for (int64_t p = blockIdx.y; p < pairs; p += gridDim.y) {
        const int t = (int)(p / cols), sl = (int)(p - (int64_t)t * cols);
        const int e = ids[p];
        const float* sp = src + t * s_s0 + sl * s_s1;
        const float* bp = (e >= 0 && e < E) ? bias + e * b_s0 : nullptr;
        float* op = out + t * o_s0 + sl * o_s1;
        for (int r = blockIdx.x * 256 + threadIdx.x; r < rows; r += gridDim.x * 256) op[r] = sp[r] + (bp ? bp[r] : 0.f);
    }
}

bool launch_add_id_f32(const float* src, int64_t s_s0, int64_t s_s1, const float* bias, int64_t b_s0, int E, const int32_t* ids, int T,
                       int cols, int rows, float* out, int64_t o_s0, int64_t o_s1, hipStream_t stream)
{
    if (T <= 0 || cols <= 0 || rows <= 0) return true;
    const int64_t pairs = (int64_t)T * cols;
    hipLaunchKernelGGL(add_id_f32_kernel, dim3(std::min((rows + 255) / 256, 64), (unsigned)std::min<int64_t>(pairs, 65535)), dim3(256), 0, stream,
                       src, s_s0, s_s1, bias, b_s0, E, ids, cols, rows, out, o_s0, o_s1, pairs);
    return hip_ok(hipGetLastError(), "addid launch");
}

bool launch_mul_mat_id_f32(const float* w, int64_t w_s0, int64_t w_s1, int E, int rows, int K, const float* x, int64_t x_s0, int64_t x_s1,
                           int slots, const int32_t* ids, int T, int cols, float* out, int64_t o_s0, int64_t o_s1, hipStream_t stream)
{
    if (T <= 0 || cols <= 0 || rows <= 0) return true;
    if ((int64_t)T * cols > 65535 || slots <= 0) {
        set_last_error("mulmatid: more than 65535 (token, slot) pairs per call.");
        return false;
    }
    hipLaunchKernelGGL(mul_mat_id_f32_kernel, dim3((rows + 3) / 4, T * cols), dim3(256), 0, stream, w, w_s0, w_s1, E, rows, K, x, x_s0, x_s1,
                       slots, ids, cols, out, o_s0, o_s1);
    return hip_ok(hipGetLastError(), "mulmatid launch");
}

}  // namespace tship
