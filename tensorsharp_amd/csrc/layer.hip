// Single-token attention pieces of the whole-layer decode (TensorSharp.GGML.Native/ggml_ops_transformer.cpp:318-470):
// what sits between the fused QKV projection and the output projection.
//
//   qkv_post_kernel      per head: optional RMSNorm over the head (ggml_rms_norm, then * weight), RoPE at `position`
//                        (ggml_rope_ext with n_dims = head_dim, ext_factor 0, attn_factor 1: ggml-cpu/ops.cpp:5549-5563,
//                        :5636-5652); q heads go to a scratch row, k heads and the untouched v heads into the fp32 KV
//                        cache [kv_head][max_seq_len][head_dim] at row `position`
//   attn_decode_kernel   softmax(q . K^T / sqrt(head_dim)) V over positions 0..position for one query head, grouped-query
//                        heads sharing their KV head (what ggml_flash_attn_ext computes for one query row); the positions
//                        are cut into splits of 256, each split leaves (max, sum, weighted V) behind
//   attn_combine_kernel  merges the splits of a head
//
// HBM-bound on the KV cache: 2 * num_kv_heads * (position + 1) * head_dim * 4 bytes per call.
#include "tship_internal.h"

namespace tship {
namespace {

constexpr int kMaxHeadDim = 256;
constexpr int kSplit = 256;          // positions per workgroup of the attention kernel
constexpr int kAttnWaves = 4;

__device__ __forceinline__ float wave_sum(float v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
    return v;
}
__device__ __forceinline__ double wave_sum(double v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
    return v;
}

// one wavefront per head: blocks [0, H) are query heads, [H, H + KV) key heads, [H + KV, H + 2 KV) value heads
__global__ void __launch_bounds__(64) qkv_post_kernel(const float* __restrict__ qkv, int num_heads, int num_kv_heads, int head_dim,
                                                      const float* __restrict__ q_norm_w, const float* __restrict__ k_norm_w,
                                                      float eps, int position, float theta_scale, float freq_scale, int neox,
                                                      float* __restrict__ q_out, float* __restrict__ k_cache,
                                                      float* __restrict__ v_cache, int max_seq_len)
{
    __shared__ float head[kMaxHeadDim];
    const int b = blockIdx.x, lane = threadIdx.x;
    const float* src = qkv + (int64_t)b * head_dim;          // q heads, then k heads, then v heads, all head_dim wide
    if (b >= num_heads + num_kv_heads) {
        float* dst = v_cache + ((int64_t)(b - num_heads - num_kv_heads) * max_seq_len + position) * head_dim;
        for (int d = lane; d < head_dim; d += 64) dst[d] = src[d];
        return;
    }
    const bool is_q = b < num_heads;
    const float* nw = is_q ? q_norm_w : k_norm_w;
    float scale = 1.f;
    if (nw) {
        // ggml-cpu/ops.cpp:3646-3695: sum of squares in double, scale = 1 / sqrtf(mean + eps)
        double ss = 0.0;
        for (int d = lane; d < head_dim; d += 64) ss += (double)(src[d] * src[d]);
        ss = wave_sum(ss);
        scale = 1.0f / sqrtf((float)(ss / (double)head_dim) + eps);
    }
    for (int d = lane; d < head_dim; d += 64) head[d] = nw ? (src[d] * scale) * nw[d] : src[d];
    __syncthreads();
    float* dst = is_q ? q_out + (int64_t)b * head_dim
                      : k_cache + ((int64_t)(b - num_heads) * max_seq_len + position) * head_dim;
    const int half = head_dim >> 1;
    for (int p = lane; p < half; p += 64) {
        // the reference builds theta by repeated multiplication; the same float products in the same order
        float theta = (float)position;
        for (int i = 0; i < p; ++i) theta *= theta_scale;
        const float ang = freq_scale * theta;
        const float c = cosf(ang), s = sinf(ang);
        const int i0 = neox ? p : 2 * p, i1 = neox ? p + half : 2 * p + 1;
        const float x0 = head[i0], x1 = head[i1];
        dst[i0] = x0 * c - x1 * s;
        dst[i1] = x0 * s + x1 * c;
    }
}

// grid (num_heads, splits): 4 wavefronts, wavefront w takes positions w, w + 4, ... of the split; lane l holds the
// head dimensions l, l + 64, ...
__global__ void __launch_bounds__(kAttnWaves * 64) attn_decode_kernel(const float* __restrict__ q, const float* __restrict__ k_cache,
                                                                       const float* __restrict__ v_cache, int head_dim, int group,
                                                                       int max_seq_len, int total, float scale,
                                                                       float* __restrict__ partial)
{
    constexpr int kPer = kMaxHeadDim / 64;
    __shared__ float sm[kAttnWaves], sl[kAttnWaves], sacc[kAttnWaves][kMaxHeadDim];
    const int h = blockIdx.x, split = blockIdx.y;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int kvh = h / group;
    const float* kb = k_cache + (int64_t)kvh * max_seq_len * head_dim;
    const float* vb = v_cache + (int64_t)kvh * max_seq_len * head_dim;
    float qr[kPer], acc[kPer];
#pragma unroll
    for (int j = 0; j < kPer; ++j) {
        const int d = lane + 64 * j;
        qr[j] = d < head_dim ? q[(int64_t)h * head_dim + d] : 0.f;
        acc[j] = 0.f;
    }
    float m = -INFINITY, l = 0.f;
    const int t_end = min(total, (split + 1) * kSplit);
    for (int t = split * kSplit + wave; t < t_end; t += kAttnWaves) {
        const float* kr = kb + (int64_t)t * head_dim;
        float dot = 0.f;
#pragma unroll
        for (int j = 0; j < kPer; ++j) {
            const int d = lane + 64 * j;
            if (d < head_dim) dot += qr[j] * kr[d];
        }
        const float s = wave_sum(dot) * scale;
        const float mn = fmaxf(m, s);
        const float corr = expf(m - mn), p = expf(s - mn);       // exp(-inf) = 0 on the first position
        const float* vr = vb + (int64_t)t * head_dim;
        l = l * corr + p;
#pragma unroll
        for (int j = 0; j < kPer; ++j) {
            const int d = lane + 64 * j;
            if (d < head_dim) acc[j] = acc[j] * corr + p * vr[d];
        }
        m = mn;
    }
    if (lane == 0) {
        sm[wave] = m;
        sl[wave] = l;
    }
#pragma unroll
    for (int j = 0; j < kPer; ++j) sacc[wave][lane + 64 * j] = acc[j];
    __syncthreads();
    if (wave == 0) {
        float mm = -INFINITY;
#pragma unroll
        for (int w = 0; w < kAttnWaves; ++w) mm = fmaxf(mm, sm[w]);
        float ll = 0.f;
        float out[kPer];
#pragma unroll
        for (int j = 0; j < kPer; ++j) out[j] = 0.f;
#pragma unroll
        for (int w = 0; w < kAttnWaves; ++w) {
            const float f = sm[w] == -INFINITY ? 0.f : expf(sm[w] - mm);     // a wavefront without positions
            ll += sl[w] * f;
#pragma unroll
            for (int j = 0; j < kPer; ++j) out[j] += sacc[w][lane + 64 * j] * f;
        }
        float* dst = partial + ((int64_t)h * gridDim.y + split) * (kMaxHeadDim + 2);
        if (lane == 0) {
            dst[0] = mm;
            dst[1] = ll;
        }
#pragma unroll
        for (int j = 0; j < kPer; ++j) dst[2 + lane + 64 * j] = out[j];
    }
}

__global__ void __launch_bounds__(64) attn_combine_kernel(const float* __restrict__ partial, int splits, int head_dim,
                                                          float* __restrict__ out)
{
    const int h = blockIdx.x, lane = threadIdx.x;
    const float* base = partial + (int64_t)h * splits * (kMaxHeadDim + 2);
    float mm = -INFINITY;
    for (int s = 0; s < splits; ++s) mm = fmaxf(mm, base[(int64_t)s * (kMaxHeadDim + 2)]);
    float ll = 0.f;
    for (int s = 0; s < splits; ++s) {
        const float* p = base + (int64_t)s * (kMaxHeadDim + 2);
        ll += p[1] * expf(p[0] - mm);
    }
    for (int d = lane; d < head_dim; d += 64) {
        float acc = 0.f;
        for (int s = 0; s < splits; ++s) {
            const float* p = base + (int64_t)s * (kMaxHeadDim + 2);
            acc += p[2 + d] * expf(p[0] - mm);
        }
        out[(int64_t)h * head_dim + d] = acc / ll;
    }
}

}  // namespace

size_t attention_decode_ws_bytes(int num_heads, int total)
{
    const int splits = (total + kSplit - 1) / kSplit;
    return (size_t)num_heads * splits * (kMaxHeadDim + 2) * sizeof(float);
}

bool launch_qkv_post(const float* qkv, int num_heads, int num_kv_heads, int head_dim, const float* q_norm_w, const float* k_norm_w,
                     float eps, int position, float rope_base, float rope_freq_scale, int rope_mode, float* q_out, float* k_cache,
                     float* v_cache, int max_seq_len, hipStream_t stream)
{
    if (head_dim <= 0 || head_dim > kMaxHeadDim || (head_dim & 1)) {
        set_last_error("layer decode: head_dim must be even and at most 256.");
        return false;
    }
    if (rope_mode != 0 && rope_mode != 2) {
        set_last_error("layer decode: rope mode must be 0 (adjacent pairs) or 2 (NeoX halves).");
        return false;
    }
    const float theta_scale = powf(rope_base, -2.0f / (float)head_dim);           // ggml-cpu/ops.cpp:5711
    hipLaunchKernelGGL(qkv_post_kernel, dim3(num_heads + 2 * num_kv_heads), dim3(64), 0, stream, qkv, num_heads, num_kv_heads, head_dim,
                       q_norm_w, k_norm_w, eps, position, theta_scale, rope_freq_scale, rope_mode == 2 ? 1 : 0, q_out, k_cache,
                       v_cache, max_seq_len);
    return hip_ok(hipGetLastError(), "qkv post launch");
}

bool launch_attention_decode(const float* q, const float* k_cache, const float* v_cache, int num_heads, int num_kv_heads,
                             int head_dim, int max_seq_len, int total, float* partial_ws, float* out, hipStream_t stream)
{
    if (num_kv_heads <= 0 || num_heads % num_kv_heads != 0 || total <= 0 || total > max_seq_len) {
        set_last_error("layer decode: bad head counts or position.");
        return false;
    }
    const int splits = (total + kSplit - 1) / kSplit;
    if (splits > 65535) {
        set_last_error("layer decode: context too long for one launch.");
        return false;
    }
    const float scale = 1.0f / sqrtf((float)head_dim);
    hipLaunchKernelGGL(attn_decode_kernel, dim3(num_heads, splits), dim3(kAttnWaves * 64), 0, stream, q, k_cache, v_cache, head_dim,
                       num_heads / num_kv_heads, max_seq_len, total, scale, partial_ws);
    if (!hip_ok(hipGetLastError(), "attention launch")) return false;
    hipLaunchKernelGGL(attn_combine_kernel, dim3(num_heads), dim3(64), 0, stream, partial_ws, splits, head_dim, out);
    return hip_ok(hipGetLastError(), "attention combine launch");
}

}  // namespace tship
