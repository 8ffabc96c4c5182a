// MoE support kernels for the GPT-OSS expert stage: routing, grouping by expert, SwiGLU-OAI, combine.
// The expert matmuls themselves are the GEMV / GEMM kernels (with an expert indirection / tile table).
//
// Semantics restated from TensorSharp.Models/Models/GptOss/GptOssModel.cs:
//   MoERoute :814-865, MoEForwardBatched :737-812 (stable grouping by expert, ascending-expert
//   accumulation), MoEForwardSingleToken :718-735 (selection-order accumulation), ExpertFFN :867-898,
//   ApplySwiGluOaiInPlace :901-934 (scalar form), LinearForwardWithBias :974-994.
#include "tship_internal.h"

namespace tship {
namespace {

constexpr int kMaxK = 16;

// one wavefront per token
__global__ void __launch_bounds__(64) moe_route_kernel(const float* __restrict__ logits, int64_t ld, int E, int k,
                                                       int* __restrict__ ids, float* __restrict__ weights)
{
    const int t = blockIdx.x, lane = threadIdx.x;
    const float* row = logits + (int64_t)t * ld;
    int sel[kMaxK];
    float val[kMaxK];
#pragma unroll
    for (int s = 0; s < kMaxK; ++s) {
        sel[s] = -1;
        val[s] = 0.f;
    }
#pragma unroll
    for (int s = 0; s < kMaxK; ++s) {
        if (s < k) {
            float best = -INFINITY;
            int bi = 0x7fffffff;
            for (int i = lane; i < E; i += 64) {
                bool taken = false;
#pragma unroll
                for (int j = 0; j < kMaxK; ++j) taken = taken || (j < s && sel[j] == i);
                const float v = row[i];
                if (!taken && v > best) {   // strict: the first maximum wins
                    best = v;
                    bi = i;
                }
            }
            for (int o = 32; o > 0; o >>= 1) {
                const float ov = __shfl_xor(best, o);
                const int oi = __shfl_xor(bi, o);
                if (ov > best || (ov == best && oi < bi)) {
                    best = ov;
                    bi = oi;
                }
            }
            if (bi == 0x7fffffff) {   // nothing comparable left (all -inf / NaN): the reference keeps index 0
                bi = 0;
                best = row[0];
            }
            sel[s] = bi;
            val[s] = best;
        }
    }
    float mx = -INFINITY;
#pragma unroll
    for (int s = 0; s < kMaxK; ++s)
        if (s < k && val[s] > mx) mx = val[s];
    float sum = 0.f;
#pragma unroll
    for (int s = 0; s < kMaxK; ++s)
        if (s < k) {
            val[s] = expf(val[s] - mx);
            sum += val[s];
        }
#pragma unroll
    for (int s = 0; s < kMaxK; ++s)
        if (s < k && lane == 0) {
            ids[(int64_t)t * k + s] = sel[s];
            weights[(int64_t)t * k + s] = sum > 0.f ? val[s] / sum : val[s];
        }
}

// single workgroup: histogram, exclusive scan, stable placement (one wavefront per expert at a time), tile table
__global__ void __launch_bounds__(1024) moe_group_kernel(const int* __restrict__ ids, int A, int k, int E, int bm, int max_tiles,
                                                         MoeMaps M)
{
    extern __shared__ int sh[];      // cnt[E], off[E + 1], tbeg[E + 1]
    int* cnt = sh;
    int* off = sh + E;
    int* tbeg = sh + 2 * E + 1;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nw = blockDim.x >> 6;
    for (int e = tid; e < E; e += blockDim.x) cnt[e] = 0;
    __syncthreads();
    for (int i = tid; i < A; i += blockDim.x) {
        const int e = ids[i];
        if (e >= 0 && e < E) atomicAdd(&cnt[e], 1);
        else M.pos_of[i] = -1;
    }
    __syncthreads();
    if (tid == 0) {
        int o = 0, tb = 0;
        for (int e = 0; e < E; ++e) {
            off[e] = o;
            tbeg[e] = tb;
            o += cnt[e];
            tb += (cnt[e] + bm - 1) / bm;
        }
        off[E] = o;
        tbeg[E] = tb;
    }
    __syncthreads();
    for (int e = tid; e <= E; e += blockDim.x) M.offsets[e] = off[e];
    for (int j = tbeg[E] + tid; j < max_tiles; j += blockDim.x) {
        M.tile_expert[j] = 0;
        M.tile_row0[j] = 0;
        M.tile_rows[j] = 0;
    }
    for (int e = wave; e < E; e += nw) {
        int base = off[e];
        for (int c = 0; c < A; c += 64) {
            const int i = c + lane;
            const bool match = i < A && ids[i] == e;
            const unsigned long long mask = __ballot(match);
            if (match) {
                const int pos = base + __popcll(mask & ((1ull << lane) - 1ull));
                M.token_of[pos] = i / k;
                M.expert_of[pos] = e;
                M.pos_of[i] = pos;
            }
            base += __popcll(mask);
        }
        const int nt = (cnt[e] + bm - 1) / bm;
        for (int j = lane; j < nt; j += 64) {
            M.tile_expert[tbeg[e] + j] = e;
            M.tile_row0[tbeg[e] + j] = off[e] + j * bm;
            M.tile_rows[tbeg[e] + j] = min(bm, cnt[e] - j * bm);
        }
    }
}

__global__ void __launch_bounds__(256) moe_swiglu_kernel(const float* __restrict__ gu, const float* __restrict__ bias,
                                                         const int* __restrict__ expert_of, int F, float alpha, float limit,
                                                         float* __restrict__ act)
{
    const int r = blockIdx.y;
    const int f = blockIdx.x * 256 + threadIdx.x;
    if (f >= F) return;
    const float* g = gu + (int64_t)r * 2 * F;
    float gate = g[f], up = g[F + f];
    if (bias) {
        const float* b = bias + (int64_t)expert_of[r] * 2 * F;
        gate += b[f];
        up += b[F + f];
    }
    const float x = fminf(gate, limit);
    const float y = fminf(fmaxf(up, -limit), limit);
    const float glu = x / (1.0f + expf(alpha * (-x)));
    act[(int64_t)r * F + f] = glu * (y + 1.0f);
}

__global__ void __launch_bounds__(256) moe_combine_kernel(const float* __restrict__ dn, const float* __restrict__ bias,
                                                          const int* __restrict__ ids, const float* __restrict__ weights,
                                                          const int* __restrict__ pos_of, int k, int H, int slot_order,
                                                          float* __restrict__ out, int64_t ldo)
{
    const int t = blockIdx.y;
    const int h = blockIdx.x * 256 + threadIdx.x;
    if (h >= H) return;
    int order[kMaxK];
#pragma unroll
    for (int s = 0; s < kMaxK; ++s) order[s] = s;
    if (!slot_order) {
        // ascending expert id, ties in slot order (insertion sort, k <= 16)
#pragma unroll
        for (int a = 1; a < kMaxK; ++a) {
            if (a < k) {
#pragma unroll
                for (int b = kMaxK - 1; b > 0; --b) {
                    if (b <= a && ids[(int64_t)t * k + order[b]] < ids[(int64_t)t * k + order[b - 1]]) {
                        const int tmp = order[b];
                        order[b] = order[b - 1];
                        order[b - 1] = tmp;
                    }
                }
            }
        }
    }
    float acc = 0.f;
#pragma unroll
    for (int j = 0; j < kMaxK; ++j) {
        if (j < k) {
            const int s = order[j];
            const int64_t a = (int64_t)t * k + s;
            const int pos = pos_of ? pos_of[a] : (int)a;
            if (pos >= 0) {
                float v = dn[(int64_t)pos * H + h];
                if (bias) v += bias[(int64_t)ids[a] * H + h];
                acc += weights[a] * v;
            }
        }
    }
    out[(int64_t)t * ldo + h] = acc;
}

}  // namespace

bool launch_moe_route(const float* logits, int64_t ld, int T, int E, int k, int* ids, float* weights, hipStream_t stream)
{
    if (k < 1 || k > kMaxK || k > E) {
        set_last_error("moe_route: k out of range (1..16, <= number of experts).");
        return false;
    }
    hipLaunchKernelGGL(moe_route_kernel, dim3(T), dim3(64), 0, stream, logits, ld, E, k, ids, weights);
    return hip_ok(hipGetLastError(), "moe_route launch");
}

bool launch_moe_group(const int* ids, int A, int k, int E, int bm, int max_tiles, const MoeMaps& maps, hipStream_t stream)
{
    if (E > 4096) {
        set_last_error("moe_group: more than 4096 experts.");
        return false;
    }
    const size_t lds = (size_t)(3 * E + 2) * sizeof(int);
    hipLaunchKernelGGL(moe_group_kernel, dim3(1), dim3(1024), lds, stream, ids, A, k, E, bm, max_tiles, maps);
    return hip_ok(hipGetLastError(), "moe_group launch");
}

bool launch_moe_swiglu(const float* gu, const float* bias, const int* expert_of, int rows, int F, float alpha, float limit,
                       float* act, hipStream_t stream)
{
    hipLaunchKernelGGL(moe_swiglu_kernel, dim3((F + 255) / 256, rows), dim3(256), 0, stream, gu, bias, expert_of, F, alpha, limit, act);
    return hip_ok(hipGetLastError(), "moe_swiglu launch");
}

bool launch_moe_combine(const float* dn, const float* bias, const int* ids, const float* weights, const int* pos_of, int T,
                        int k, int H, bool slot_order, float* out, int64_t ldo, hipStream_t stream)
{
    if (k > kMaxK) {
        set_last_error("moe_combine: k > 16.");
        return false;
    }
    hipLaunchKernelGGL(moe_combine_kernel, dim3((H + 255) / 256, T), dim3(256), 0, stream, dn, bias, ids, weights, pos_of, k, H,
                       slot_order ? 1 : 0, out, ldo);
    return hip_ok(hipGetLastError(), "moe_combine launch");
}

}  // namespace tship
