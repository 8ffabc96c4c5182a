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
constexpr int kGroupLdsIds = 8192;     // assignments whose ids the grouping kernel keeps in LDS (32 KiB)

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

// single workgroup: histogram, exclusive scan, placement, tile table
__global__ void __launch_bounds__(1024) moe_group_kernel(const int* __restrict__ ids, int A, int k, int E, int bm, int max_tiles,
                                                         MoeMaps M)
{
    extern __shared__ int sh[];      // cnt[E], off[E + 1], tbeg[E + 1], then a copy of the ids if it fits
    int* cnt = sh;
    int* off = sh + E;
    int* tbeg = sh + 2 * E + 1;
    int* ids_lds = sh + 3 * E + 2;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nw = blockDim.x >> 6;
    const bool in_lds = A <= kGroupLdsIds;       // the placement pass below reads every id once per expert
    for (int e = tid; e < E; e += blockDim.x) cnt[e] = 0;
    __syncthreads();
    for (int i = tid; i < A; i += blockDim.x) {
        const int e = ids[i];
        if (in_lds) ids_lds[i] = e;
        if (e >= 0 && e < E) atomicAdd(&cnt[e], 1);
        else M.pos_of[i] = -1;
    }
    __syncthreads();
    // exclusive scans of the row counts and of the tile counts: one wavefront, 64 experts per step
    if (wave == 0) {
        int carry_o = 0, carry_t = 0;
        for (int e0 = 0; e0 < E; e0 += 64) {
            const int e = e0 + lane;
            const int c = e < E ? cnt[e] : 0;
            const int nt = (c + bm - 1) / bm;
            int so = c, st = nt;
#pragma unroll
            for (int d = 1; d < 64; d <<= 1) {
                const int vo = __shfl_up(so, d), vt = __shfl_up(st, d);
                if (lane >= d) {
                    so += vo;
                    st += vt;
                }
            }
            if (e < E) {
                off[e] = carry_o + so - c;
                tbeg[e] = carry_t + st - nt;
            }
            carry_o += __shfl(so, 63);
            carry_t += __shfl(st, 63);
        }
        if (lane == 0) {
            off[E] = carry_o;
            tbeg[E] = carry_t;
        }
    }
    __syncthreads();
    for (int e = tid; e <= E; e += blockDim.x) M.offsets[e] = off[e];
    // assignments with an id outside the table take no sorted row: the rows past the last expert's stay unused, but
    // the activation converts walk over all A rows, so those rows name a valid token and expert
    for (int i = off[E] + tid; i < A; i += blockDim.x) {
        M.token_of[i] = 0;
        M.expert_of[i] = 0;
    }
    for (int j = tbeg[E] + tid; j < max_tiles; j += blockDim.x) {
        M.tile_expert[j] = 0;
        M.tile_row0[j] = 0;
        M.tile_rows[j] = 0;
    }
    // Placement: the rows of an expert are handed out by an LDS counter, in no particular order (every result row
    // depends on its own activation row only, so the order inside an expert does not show in the output).
    __syncthreads();
    for (int e = tid; e < E; e += blockDim.x) cnt[e] = 0;            // reused as the fill counters
    __syncthreads();
    for (int i = tid; i < A; i += blockDim.x) {
        const int e = in_lds ? ids_lds[i] : ids[i];
        if (e >= 0 && e < E) {
            const int pos = off[e] + atomicAdd(&cnt[e], 1);
            M.token_of[pos] = i / k;
            M.expert_of[pos] = e;
            M.pos_of[i] = pos;
        }
    }
    for (int e = wave; e < E; e += nw) {
        const int rows = off[e + 1] - off[e];
        const int nt = (rows + bm - 1) / bm;
        for (int j = lane; j < nt; j += 64) {
            M.tile_expert[tbeg[e] + j] = e;
            M.tile_row0[tbeg[e] + j] = off[e] + j * bm;
            M.tile_rows[tbeg[e] + j] = min(bm, rows - j * bm);
        }
    }
}

// VEC consecutive columns per thread (4: rows and pointers 16-byte aligned)
template <int VEC>
__global__ void __launch_bounds__(256) moe_combine_kernel(const float* __restrict__ dn, const float* __restrict__ bias,
                                                          const int* __restrict__ ids, const float* __restrict__ weights,
                                                          const int* __restrict__ pos_of, int k, int E, int H, int slot_order,
                                                          float* __restrict__ out, int64_t ldo)
{
    const int t = blockIdx.y;
    const int h = (blockIdx.x * 256 + threadIdx.x) * VEC;
    if (h >= H) return;
    // the token's (expert, slot) pairs in registers
    int id[kMaxK], slot[kMaxK];
#pragma unroll
    for (int s = 0; s < kMaxK; ++s) {
        id[s] = s < k ? ids[(int64_t)t * k + s] : 0x7fffffff;
        slot[s] = s;
    }
    if (!slot_order) {
        // ascending expert id, ties in slot order (insertion sort, k <= 16)
#pragma unroll
        for (int a = 1; a < kMaxK; ++a) {
            if (a < k) {
#pragma unroll
                for (int b = a; b > 0; --b) {
                    if (id[b] < id[b - 1]) {
                        const int ti = id[b], ts = slot[b];
                        id[b] = id[b - 1];
                        slot[b] = slot[b - 1];
                        id[b - 1] = ti;
                        slot[b - 1] = ts;
                    }
                }
            }
        }
    }
    float acc[VEC];
#pragma unroll
    for (int v = 0; v < VEC; ++v) acc[v] = 0.f;
#pragma unroll
    for (int j = 0; j < kMaxK; ++j) {
        if (j < k) {
            const int64_t a = (int64_t)t * k + slot[j];
            const int pos = pos_of ? pos_of[a] : (int)a;
            if (pos >= 0 && id[j] >= 0 && id[j] < E) {     // an id outside the expert table contributes nothing
                const float w = weights[a];
                const float* dp = dn + (int64_t)pos * H + h;
                const float* bp = bias ? bias + (int64_t)id[j] * H + h : nullptr;
                if constexpr (VEC == 4) {
                    float4 v = *reinterpret_cast<const float4*>(dp);
                    if (bp) {
                        const float4 bv = *reinterpret_cast<const float4*>(bp);
                        v = float4{v.x + bv.x, v.y + bv.y, v.z + bv.z, v.w + bv.w};
                    }
                    acc[0] += w * v.x;
                    acc[1] += w * v.y;
                    acc[2] += w * v.z;
                    acc[3] += w * v.w;
                } else {
                    float v = dp[0];
                    if (bp) v += bp[0];
                    acc[0] += w * v;
                }
            }
        }
    }
    float* op = out + (int64_t)t * ldo + h;
    if constexpr (VEC == 4) *reinterpret_cast<float4*>(op) = float4{acc[0], acc[1], acc[2], acc[3]};
    else op[0] = acc[0];
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
    const size_t lds = (size_t)(3 * E + 2 + (A <= kGroupLdsIds ? A : 0)) * sizeof(int);
    hipLaunchKernelGGL(moe_group_kernel, dim3(1), dim3(1024), lds, stream, ids, A, k, E, bm, max_tiles, maps);
    return hip_ok(hipGetLastError(), "moe_group launch");
}

bool launch_moe_combine(const float* dn, const float* bias, const int* ids, const float* weights, const int* pos_of, int T,
                        int k, int E, int H, bool slot_order, float* out, int64_t ldo, hipStream_t stream)
{
    if (k > kMaxK) {
        set_last_error("moe_combine: k > 16.");
        return false;
    }
    const bool vec = H % 4 == 0 && ldo % 4 == 0 && ((reinterpret_cast<uintptr_t>(dn) | reinterpret_cast<uintptr_t>(bias) |
                                                    reinterpret_cast<uintptr_t>(out)) & 15) == 0;
    if (vec)
        hipLaunchKernelGGL(moe_combine_kernel<4>, dim3((H / 4 + 255) / 256, T), dim3(256), 0, stream, dn, bias, ids, weights, pos_of, k,
                           E, H, slot_order ? 1 : 0, out, ldo);
    else
        hipLaunchKernelGGL(moe_combine_kernel<1>, dim3((H + 255) / 256, T), dim3(256), 0, stream, dn, bias, ids, weights, pos_of, k, E, H,
                           slot_order ? 1 : 0, out, ldo);
    return hip_ok(hipGetLastError(), "moe_combine launch");
}

}  // namespace tship
