// Single-token attention pieces of the whole-layer decode (TensorSharp.GGML.Native/ggml_ops_transformer.cpp:318-470):
// what sits between the fused QKV projection and the output projection.
//
//   attn_decode_kernel   first finishes the projections for the heads it serves - optional RMSNorm over the head
//                        (ggml_rms_norm, then * weight), RoPE at `position` (ggml_rope_ext with n_dims = head_dim,
//                        ext_factor 0, attn_factor 1: ggml-cpu/ops.cpp:5549-5563, :5636-5652); the new k and the
//                        untouched v row go into the fp32 KV cache [kv_head][max_seq_len][head_dim] at row `position`
//                        (written by the workgroup of the last split, which uses them from LDS) - then computes
//                        softmax(q . K^T / sqrt(head_dim)) V over positions 0..position (what ggml_flash_attn_ext
//                        computes for one query row); a workgroup serves the query heads that share a KV head, so K / V
//                        rows are loaded once per group; the positions are cut into splits of 64 or 128, each split
//                        leaves (max, sum, weighted V) behind (a single split writes the result itself)
//   attn_combine_kernel  merges the splits of a head
//
// HBM-bound on the KV cache: 2 * num_kv_heads * (position + 1) * head_dim * 4 bytes per call.
#include "tship_internal.h"

namespace tship {
namespace {

constexpr int kMaxHeadDim = 256;
// positions per workgroup of the attention kernel: one trip of the 16 groups x kInFlight rows while the context is
// short (the kernel is latency bound: more, shorter workgroups), two trips beyond
int attn_split_len(int total) { return total <= 2048 ? 64 : 128; }
constexpr int kInFlight = 4;         // K / V rows a 16-lane group loads before it uses the first
constexpr int kAttnWaves = 4;

__device__ __forceinline__ float wave_sum(float v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
    return v;
}
// (register permutations on both halves of the value; a shuffle of a double is two trips through the LDS crossbar)
__device__ __forceinline__ double wave_sum(double v)
{
    typedef uint32_t u2_t __attribute__((ext_vector_type(2)));
    auto moved = [](double d, auto perm) { return __hiloint2double(perm(__double2hiint(d)), perm(__double2loint(d))); };
    v += moved(v, [](int x) { return __builtin_amdgcn_update_dpp(0, x, 0xb1, 0xf, 0xf, true); });
    v += moved(v, [](int x) { return __builtin_amdgcn_update_dpp(0, x, 0x4e, 0xf, 0xf, true); });
    v += moved(v, [](int x) { return __builtin_amdgcn_update_dpp(0, x, 0x141, 0xf, 0xf, true); });
    v += moved(v, [](int x) { return __builtin_amdgcn_update_dpp(0, x, 0x140, 0xf, 0xf, true); });
    {
        const u2_t hi = __builtin_amdgcn_permlane16_swap((uint32_t)__double2hiint(v), (uint32_t)__double2hiint(v), false, false);
        const u2_t lo = __builtin_amdgcn_permlane16_swap((uint32_t)__double2loint(v), (uint32_t)__double2loint(v), false, false);
        v = __hiloint2double((int)hi.x, (int)lo.x) + __hiloint2double((int)hi.y, (int)lo.y);
    }
    {
        const u2_t hi = __builtin_amdgcn_permlane32_swap((uint32_t)__double2hiint(v), (uint32_t)__double2hiint(v), false, false);
        const u2_t lo = __builtin_amdgcn_permlane32_swap((uint32_t)__double2loint(v), (uint32_t)__double2loint(v), false, false);
        v = __hiloint2double((int)hi.x, (int)lo.x) + __hiloint2double((int)hi.y, (int)lo.y);
    }
    return v;
}

// What the attention kernel needs to finish the projections itself: the raw output of the QKV matmul
// ([q heads | k heads | v heads], head_dim each), the optional per-head RMSNorm weights, the rotation, and the caches
// whose row `position` it writes.
struct AttnFront {
    const float* qkv;
    const float* q_norm_w;
    const float* k_norm_w;
    float eps, theta_scale, freq_scale;
    int neox;
    int num_heads, num_kv_heads;
    float* k_cache;
    float* v_cache;
};

// Merge of two online-softmax states (max, sum, weighted values).
template <int N>
__device__ __forceinline__ void softmax_merge(float& m, float& l, float (&acc)[N], float m2, float l2, const float (&acc2)[N])
{
    const float mm = fmaxf(m, m2);
    const float f1 = m == -INFINITY ? 0.f : expf(m - mm), f2 = m2 == -INFINITY ? 0.f : expf(m2 - mm);
    l = l * f1 + l2 * f2;
#pragma unroll
    for (int j = 0; j < N; ++j) acc[j] = acc[j] * f1 + acc2[j] * f2;
    m = mm;
}

// Sum over the 16 lanes of a group, every lane gets it: four register permutations (pairs inside a quad, quads, mirrored
// eights, mirrored sixteen) instead of four trips through the LDS crossbar.
__device__ __forceinline__ float sum16(float v)
{
    auto moved = [](float x, auto perm) { return __int_as_float(perm(__float_as_int(x))); };
    v += moved(v, [](int x) { return __builtin_amdgcn_update_dpp(0, x, 0xb1, 0xf, 0xf, true); });     // quad_perm [1,0,3,2]
    v += moved(v, [](int x) { return __builtin_amdgcn_update_dpp(0, x, 0x4e, 0xf, 0xf, true); });     // quad_perm [2,3,0,1]
    v += moved(v, [](int x) { return __builtin_amdgcn_update_dpp(0, x, 0x141, 0xf, 0xf, true); });    // lane i <-> 7 - i of each 8
    v += moved(v, [](int x) { return __builtin_amdgcn_update_dpp(0, x, 0x140, 0xf, 0xf, true); });    // lane i <-> 15 - i of each 16
    return v;
}

// grid (num_kv_heads, splits, q-head chunks): one workgroup serves G query heads that share a KV head, so every K / V
// row is loaded once for all of them.  4 wavefronts x 4 groups of 16 lanes; a group takes positions g, g + 16, ... of
// the split, kInFlight at a time (all their loads are issued before the first is used: the loop is latency bound), lane l of
// a group holds the head dimensions l, l + 16, ... (PER of them).  Groups, then wavefronts, merge their softmax states.
template <int PER, int G>
__global__ void __launch_bounds__(kAttnWaves * 64) attn_decode_kernel(float* k_cache, float* v_cache, const float* qkv, int group,
                                                                       int max_seq_len, int total, int split_len, float scale, int splits,
                                                                       int num_heads, float* __restrict__ partial, const AttnFront F,
                                                                       float* __restrict__ out_direct, const float* pre0, const float* pre1,
                                                                       int pre_floats)
{
    // (what the first loads need - the caches, the projections, the geometry - are leading scalar arguments: the hardware
    // delivers the first 14 dwords in SGPRs at wave launch, the rest is read from the argument block)
    constexpr int HD = 16 * PER;
    __shared__ float sm[kAttnWaves][G], sl[kAttnWaves][G], sacc[kAttnWaves][G][HD];
    __shared__ float sq[G][HD], sk[HD], sv[HD], tmp[kAttnWaves][HD];
    const int kvh = blockIdx.x, split = blockIdx.y;
    if (split == splits) {
        // One more row of workgroups than there are splits: they only read the vectors that the launches after this one
        // ask for first (the norm weights of the FFN and of the next layer) and leave.  Read from HBM by this kernel's
        // spare workgroups, the vectors wait in the memory-side cache (and, consecutive workgroups being dealt to
        // consecutive XCDs, in every L2) instead of queueing up behind a launch's first weight requests: 1.25 us per
        // RMSNorm launch, measured by leaving the vector out.
        if (blockIdx.z == 0) {
            for (int i = (int)threadIdx.x * 4; i < pre_floats; i += kAttnWaves * 64 * 4) {
                typedef float f4_t __attribute__((ext_vector_type(4)));
                f4_t a, b;                                     // never used: the loads are for the caches
                if (pre0) asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(a) : "v"(pre0 + i) : "memory");
                if (pre1) asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(b) : "v"(pre1 + i) : "memory");
            }
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        }
        return;
    }
    const int h0 = kvh * group + blockIdx.z * G;                     // first query head of this workgroup
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int lg = lane & 15, grp = (wave << 2) | (lane >> 4);       // 16 groups per workgroup
    const float* kb = k_cache + (int64_t)kvh * max_seq_len * HD;
    const float* vb = v_cache + (int64_t)kvh * max_seq_len * HD;
    const int position = total - 1;
    const bool last = split == splits - 1;                           // the split that holds the new position
    // kInFlight rows of K and of V per group, all requested before the first is used; the first set is requested
    // here, ahead of the work on the projections below, which does not depend on it
    const int t_end = min(total, (split + 1) * split_len);
    float kr[kInFlight][PER], vr[kInFlight][PER];
    auto load_rows = [&](int t0) {
#pragma unroll
        for (int u = 0; u < kInFlight; ++u) {
            const int64_t row = (int64_t)min(t0 + 16 * u, t_end - 1) * HD + lg;      // rows past the split: a valid row, unused
#pragma unroll
            for (int j = 0; j < PER; ++j) {
                kr[u][j] = kb[row + 16 * j];
                vr[u][j] = vb[row + 16 * j];
            }
        }
    };
    int t0 = split * split_len + grp;
    load_rows(t0);

    // ---- the projections' last steps, per head: RMSNorm over the head (ggml_rms_norm, then * weight), RoPE at
    // `position` (ggml_rope_ext with n_dims = head_dim: ggml-cpu/ops.cpp:5549-5563, :5636-5652).  Every workgroup
    // prepares its own query heads; the workgroup of the last split also prepares the new key / value row, uses it
    // from LDS and (query-head chunk 0 only) writes it to the caches.
    {
        constexpr int kPer = (HD + 63) / 64, kPairs = (HD / 2 + 63) / 64;
        constexpr int half = HD / 2;
        const int nprep = G + (last ? 1 : 0);
        auto head_src = [&](int hh) { return qkv + (int64_t)(hh < G ? h0 + hh : num_heads + kvh) * HD; };
        // the wavefront's first head is requested before the angles are worked out
        float xv[kPer];
#pragma unroll
        for (int j = 0; j < kPer; ++j) {
            const int d = lane + 64 * j;
            xv[j] = (wave < nprep && d < HD) ? head_src(wave)[d] : 0.f;
        }
        float cs[kPairs], sn[kPairs];
        {
            // the reference builds theta by repeated multiplication; the same float products in the same order.  One
            // uniform chain of half - 1 products, every lane keeping the value of its own pair (a loop of lane-dependent
            // length costs several times as many instructions per product).
            // theta_i = theta_(i-1) * theta_scale, i = lane + 64 j: every step each lane takes its lower neighbour's value
            // times theta_scale (lane 0: its own value times one), so that after 63 steps lane i has been through exactly
            // the products 1 .. i of the chain - one instruction per step instead of a multiply, a compare and a select.
            const float factor = lane == 0 ? 1.0f : F.theta_scale;
            float chain = (float)position;
#pragma unroll
            for (int j = 0; j < kPairs; ++j) {
                if (j > 0) chain = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(chain), 63)) * F.theta_scale;
                const int steps = min(half - 64 * j, 64) - 1;
                for (int i = 0; i < steps; ++i) {
                    const int below = __builtin_amdgcn_update_dpp(__float_as_int(chain), __float_as_int(chain), 0x138, 0xf, 0xf, false);   // wave_shr:1
                    chain = __int_as_float(below) * factor;
                }
                cs[j] = chain;
            }
#pragma unroll
            for (int j = 0; j < kPairs; ++j) {
                const float ang = F.freq_scale * cs[j];
                sincosf(ang, &sn[j], &cs[j]);
            }
        }
        for (int hh = wave; hh < nprep; hh += kAttnWaves) {          // uniform per wavefront
            const bool is_q = hh < G;
            const float* src = head_src(hh);
            const float* nw = is_q ? F.q_norm_w : F.k_norm_w;
            if (hh != wave) {
#pragma unroll
                for (int j = 0; j < kPer; ++j) {
                    const int d = lane + 64 * j;
                    xv[j] = d < HD ? src[d] : 0.f;
                }
            }
            float rs = 1.f;
            if (nw) {
                // ggml-cpu/ops.cpp:3646-3695: sum of squares in double, scale = 1 / sqrtf(mean + eps)
                double ss = 0.0;
#pragma unroll
                for (int j = 0; j < kPer; ++j) ss += (double)(xv[j] * xv[j]);
                ss = wave_sum(ss);
                rs = 1.0f / sqrtf((float)(ss / (double)HD) + F.eps);
            }
#pragma unroll
            for (int j = 0; j < kPer; ++j) {
                const int d = lane + 64 * j;
                if (d < HD) tmp[wave][d] = nw ? (xv[j] * rs) * nw[d] : xv[j];
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");   // the wavefront's own LDS writes before its reads
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            float* dst = is_q ? sq[hh] : sk;
            float* cache = (!is_q && blockIdx.z == 0) ? k_cache + ((int64_t)kvh * max_seq_len + position) * HD : nullptr;
#pragma unroll
            for (int j = 0; j < kPairs; ++j) {
                const int p = lane + 64 * j;
                if (p < half) {
                    const int i0 = F.neox ? p : 2 * p, i1 = F.neox ? p + half : 2 * p + 1;
                    const float x0 = tmp[wave][i0], x1 = tmp[wave][i1];
                    const float r0 = x0 * cs[j] - x1 * sn[j], r1 = x0 * sn[j] + x1 * cs[j];
                    dst[i0] = r0;
                    dst[i1] = r1;
                    if (cache) {
                        cache[i0] = r0;
                        cache[i1] = r1;
                    }
                }
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");   // tmp is reused by this wavefront's next head
            __builtin_amdgcn_wave_barrier();
        }
        if (last) {
            const float* src = qkv + (int64_t)(num_heads + F.num_kv_heads + kvh) * HD;
            float* cache = blockIdx.z == 0 ? v_cache + ((int64_t)kvh * max_seq_len + position) * HD : nullptr;
            for (int d = threadIdx.x; d < HD; d += kAttnWaves * 64) {
                const float v = src[d];
                sv[d] = v;
                if (cache) cache[d] = v;
            }
        }
        __syncthreads();
    }
    float qr[G][PER], acc[G][PER], m[G], l[G];
#pragma unroll
    for (int g = 0; g < G; ++g) {
        m[g] = -INFINITY;
        l[g] = 0.f;
#pragma unroll
        for (int j = 0; j < PER; ++j) {
            qr[g][j] = sq[g][lg + 16 * j] * scale;
            acc[g][j] = 0.f;
        }
    }
    for (; t0 < t_end; t0 += 16 * kInFlight) {
        bool live[kInFlight];
#pragma unroll
        for (int u = 0; u < kInFlight; ++u) live[u] = t0 + 16 * u < t_end;
        if (last) {       // uniform: the new position's row is not in the caches yet (another workgroup may be writing it)
#pragma unroll
            for (int u = 0; u < kInFlight; ++u) {
                const bool fresh = t0 + 16 * u == position;
#pragma unroll
                for (int j = 0; j < PER; ++j) {
                    kr[u][j] = fresh ? sk[lg + 16 * j] : kr[u][j];
                    vr[u][j] = fresh ? sv[lg + 16 * j] : vr[u][j];
                }
            }
        }
        // Slots past the split hold a clamped row (in the last split the row being written by this very launch, or
        // whatever the cache memory held): their values must not reach the sums, not even multiplied by a zero
        // weight (0 * NaN), so they are replaced, not scaled.
#pragma unroll
        for (int u = 0; u < kInFlight; ++u)
#pragma unroll
            for (int j = 0; j < PER; ++j) {
                kr[u][j] = live[u] ? kr[u][j] : 0.f;
                vr[u][j] = live[u] ? vr[u][j] : 0.f;
            }
#pragma unroll
        for (int g = 0; g < G; ++g) {
            float d[kInFlight];
#pragma unroll
            for (int u = 0; u < kInFlight; ++u) {
                d[u] = 0.f;
#pragma unroll
                for (int j = 0; j < PER; ++j) d[u] += qr[g][j] * kr[u][j];
            }
#pragma unroll
            for (int u = 0; u < kInFlight; ++u) d[u] = sum16(d[u]);
            float mn = m[g];
#pragma unroll
            for (int u = 0; u < kInFlight; ++u) {
                if (!live[u]) d[u] = -INFINITY;
                mn = fmaxf(mn, d[u]);
            }
            const float corr = expf(m[g] - mn);                    // exp(-inf) = 0 on the first rows
            float p[kInFlight], psum = 0.f;
#pragma unroll
            for (int u = 0; u < kInFlight; ++u) {
                p[u] = expf(d[u] - mn);
                psum += p[u];
            }
            l[g] = l[g] * corr + psum;
#pragma unroll
            for (int j = 0; j < PER; ++j) {
                float a = acc[g][j] * corr;
#pragma unroll
                for (int u = 0; u < kInFlight; ++u) a += p[u] * vr[u][j];
                acc[g][j] = a;
            }
            m[g] = mn;
        }
        if (t0 + 16 * kInFlight < t_end) load_rows(t0 + 16 * kInFlight);
    }
    // the four groups of a wavefront
#pragma unroll
    for (int g = 0; g < G; ++g) {
        // rows 0 | 1 and 2 | 3 of the wavefront, then the two halves: a lane gets the state of the even and of the odd
        // member of its pair (register swaps between rows) and merges them, so every lane ends with the same result
#pragma unroll
        for (int level = 0; level < 2; ++level) {
            typedef uint32_t u2_t __attribute__((ext_vector_type(2)));
            auto both = [&](float x, float& even, float& odd) {
                const u2_t r = level == 0 ? __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false)
                                          : __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
                even = __uint_as_float(r.x);
                odd = __uint_as_float(r.y);
            };
            float m1, m2, l1, l2, a1[PER], a2[PER];
            both(m[g], m1, m2);
            both(l[g], l1, l2);
#pragma unroll
            for (int j = 0; j < PER; ++j) both(acc[g][j], a1[j], a2[j]);
            softmax_merge<PER>(m1, l1, a1, m2, l2, a2);
            m[g] = m1;
            l[g] = l1;
#pragma unroll
            for (int j = 0; j < PER; ++j) acc[g][j] = a1[j];
        }
        if (lane < 16) {
            if (lane == 0) {
                sm[wave][g] = m[g];
                sl[wave][g] = l[g];
            }
#pragma unroll
            for (int j = 0; j < PER; ++j) sacc[wave][g][lg + 16 * j] = acc[g][j];
        }
    }
    __syncthreads();
    // the four wavefronts: thread (g, d) of the first G * HD threads
    for (int i = threadIdx.x; i < G * HD; i += kAttnWaves * 64) {
        const int g = i / HD, d = i - g * HD;
        float mm = -INFINITY;
#pragma unroll
        for (int w = 0; w < kAttnWaves; ++w) mm = fmaxf(mm, sm[w][g]);
        float ll = 0.f, out = 0.f;
#pragma unroll
        for (int w = 0; w < kAttnWaves; ++w) {
            const float f = sm[w][g] == -INFINITY ? 0.f : expf(sm[w][g] - mm);
            ll += sl[w][g] * f;
            out += sacc[w][g][d] * f;
        }
        if (out_direct) {
            out_direct[(int64_t)(h0 + g) * HD + d] = out / ll;       // a single split: this is the result
            continue;
        }
        float* dst = partial + ((int64_t)(h0 + g) * splits + split) * (kMaxHeadDim + 2);
        if (d == 0) {
            dst[0] = mm;
            dst[1] = ll;
        }
        dst[2 + d] = out;
    }
}

// one workgroup per head: wavefront w merges splits w, w + 4, ... (four rows in flight), the wavefronts meet in LDS
__global__ void __launch_bounds__(kAttnWaves * 64) attn_combine_kernel(const float* __restrict__ partial, int splits, int head_dim,
                                                                        float* __restrict__ out)
{
    constexpr int kPer = kMaxHeadDim / 64, kRow = kMaxHeadDim + 2;
    __shared__ float sacc[kAttnWaves][kMaxHeadDim], sl[kAttnWaves];
    const int h = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const float* base = partial + (int64_t)h * splits * kRow;
    float ms[4], ls[4], v[4][kPer];
    auto load_rows = [&](int s0) {
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int s = s0 + u * kAttnWaves;
            const bool live = s < splits;
            const float* p = base + (int64_t)(live ? s : s0) * kRow;
            ms[u] = live ? p[0] : -INFINITY;
            ls[u] = live ? p[1] : 0.f;
#pragma unroll
            for (int j = 0; j < kPer; ++j) {
                const int d = lane + 64 * j;
                v[u][j] = (live && d < head_dim) ? p[2 + d] : 0.f;
            }
        }
    };
    // When one batch of rows per wavefront covers the splits (up to 1024 positions), it is requested before the maximum
    // over all splits is worked out (every wavefront computes it: independent loads, one pass), so that the two round
    // trips overlap: 0.35 us per layer.  (With more batches the early request measured 0.3 us slower.)
    constexpr int kBatch = 4 * kAttnWaves;
    const bool early = splits <= kBatch;
    if (early && wave < splits) load_rows(wave);
    float mm = -INFINITY;
    for (int s = lane; s < splits; s += 64) mm = fmaxf(mm, base[(int64_t)s * kRow]);
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) mm = fmaxf(mm, __shfl_xor(mm, o));
    float acc[kPer], ll = 0.f;
#pragma unroll
    for (int j = 0; j < kPer; ++j) acc[j] = 0.f;
    for (int s0 = wave; s0 < splits; s0 += kBatch) {
        if (!early) load_rows(s0);
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const float f = ms[u] == -INFINITY ? 0.f : expf(ms[u] - mm);
            ll += ls[u] * f;
#pragma unroll
            for (int j = 0; j < kPer; ++j) acc[j] += v[u][j] * f;
        }
    }
    if (lane == 0) sl[wave] = ll;
#pragma unroll
    for (int j = 0; j < kPer; ++j) sacc[wave][lane + 64 * j] = acc[j];
    __syncthreads();
    if (wave == 0) {
        float lt = 0.f;
#pragma unroll
        for (int w = 0; w < kAttnWaves; ++w) lt += sl[w];
#pragma unroll
        for (int j = 0; j < kPer; ++j) {
            const int d = lane + 64 * j;
            float a = 0.f;
#pragma unroll
            for (int w = 0; w < kAttnWaves; ++w) a += sacc[w][d];
            if (d < head_dim) out[(int64_t)h * head_dim + d] = a / lt;
        }
    }
}

}  // namespace

size_t attention_decode_ws_bytes(int num_heads, int total)
{
    const int split_len = attn_split_len(total);
    const int splits = (total + split_len - 1) / split_len;
    return (size_t)num_heads * splits * (kMaxHeadDim + 2) * sizeof(float);
}

bool launch_attention_decode(const float* qkv, const float* q_norm_w, const float* k_norm_w, float eps, float rope_base,
                             float rope_freq_scale, int rope_mode, float* k_cache, float* v_cache, int num_heads, int num_kv_heads,
                             int head_dim, int max_seq_len, int position, float* partial_ws, float* out, hipStream_t stream,
                             const float* prefetch0, const float* prefetch1, int prefetch_floats)
{
    const int total = position + 1;
    if (num_kv_heads <= 0 || num_heads % num_kv_heads != 0 || total <= 0 || total > max_seq_len) {
        set_last_error("layer decode: bad head counts or position.");
        return false;
    }
    if (rope_mode != 0 && rope_mode != 2) {
        set_last_error("layer decode: rope mode must be 0 (adjacent pairs) or 2 (NeoX halves).");
        return false;
    }
    AttnFront front{};
    front.qkv = qkv;
    front.q_norm_w = q_norm_w;
    front.k_norm_w = k_norm_w;
    front.eps = eps;
    front.theta_scale = powf(rope_base, -2.0f / (float)head_dim);           // ggml-cpu/ops.cpp:5711
    front.freq_scale = rope_freq_scale;
    front.neox = rope_mode == 2 ? 1 : 0;
    front.num_heads = num_heads;
    front.num_kv_heads = num_kv_heads;
    front.k_cache = k_cache;
    front.v_cache = v_cache;
    const int split_len = attn_split_len(total);
    const int splits = (total + split_len - 1) / split_len;
    if (splits > 65535) {
        set_last_error("layer decode: context too long for one launch.");
        return false;
    }
    const float scale = 1.0f / sqrtf((float)head_dim);
    const int group = num_heads / num_kv_heads;
    // query heads per workgroup: as many as share the KV head (its rows are then loaded once), fewer while that leaves
    // the launch with too few workgroups to hide its latency
    int g = group % 8 == 0 ? 8 : group % 4 == 0 ? 4 : group % 2 == 0 ? 2 : 1;
    while (g > 2 && num_kv_heads * splits * (group / g) < 128) g >>= 1;
    // (vectors to prefetch: whole float4s at 16-byte aligned addresses, else none)
    const bool pre = (prefetch0 || prefetch1) && prefetch_floats > 0 && prefetch_floats % 4 == 0 && splits < 65535 &&
                     ((reinterpret_cast<uintptr_t>(prefetch0) | reinterpret_cast<uintptr_t>(prefetch1)) & 15) == 0;
    const dim3 grid(num_kv_heads, splits + (pre ? 1 : 0), group / g), block(kAttnWaves * 64);
#define TSHIP_ATTN_LAUNCH(PER, GG)                                                                                              \
    hipLaunchKernelGGL((attn_decode_kernel<PER, GG>), grid, block, 0, stream, front.k_cache, front.v_cache, front.qkv, group,     \
                       max_seq_len, total, split_len, scale, splits, num_heads, partial_ws, front, splits == 1 ? out : nullptr,           \
                       pre ? prefetch0 : nullptr, pre ? prefetch1 : nullptr, pre ? prefetch_floats : 0)
#define TSHIP_ATTN_G(PER)                                                    \
    switch (g) {                                                             \
    case 8: TSHIP_ATTN_LAUNCH(PER, 8); break;                                \
    case 4: TSHIP_ATTN_LAUNCH(PER, 4); break;                                \
    case 2: TSHIP_ATTN_LAUNCH(PER, 2); break;                                \
    default: TSHIP_ATTN_LAUNCH(PER, 1); break;                               \
    }
    switch (head_dim) {
    case 64: TSHIP_ATTN_G(4) break;
    case 80: TSHIP_ATTN_G(5) break;
    case 96: TSHIP_ATTN_G(6) break;
    case 128: TSHIP_ATTN_G(8) break;
    case 192: TSHIP_ATTN_G(12) break;
    case 256: TSHIP_ATTN_G(16) break;
    default: set_last_error("layer decode: head_dim must be one of 64, 80, 96, 128, 192, 256."); return false;
    }
#undef TSHIP_ATTN_G
#undef TSHIP_ATTN_LAUNCH
    if (!hip_ok(hipGetLastError(), "attention launch")) return false;
    if (splits == 1) return true;
    hipLaunchKernelGGL(attn_combine_kernel, dim3(num_heads), dim3(kAttnWaves * 64), 0, stream, partial_ws, splits, head_dim, out);
    return hip_ok(hipGetLastError(), "attention combine launch");
}

}  // namespace tship
