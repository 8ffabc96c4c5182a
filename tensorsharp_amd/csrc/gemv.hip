// Decode GEMV  y[N] = W[N x K] * x[K]  over raw GGUF blocks (Q8_0 / Q4_K / MXFP4) for gfx950.
//
// Shape of the kernel (all three formats):
//   * persistent workgroups of 4 wavefronts; each workgroup stages x once into LDS in the
//     layout its format's unpack order wants (fp16 pairs for Q4_K / MXFP4, fp32 for Q8_0),
//     padded so that a ds_read_b128 per lane is bank-conflict free;
//   * a wavefront owns R consecutive weight rows at a time (a contiguous byte range of W).
//     The range is cut into "units" (Q8_0: one 34-byte block, Q4_K: one 64-weight group =
//     32 quant bytes + the super-block header, MXFP4: one 17-byte block); lane l takes units
//     l, l+64, ... so consecutive lanes read consecutive bytes of the raw blocks with
//     128-bit loads.  Unaligned units (34 B / 17 B) are fetched as aligned dwords and
//     re-aligned in registers with v_alignbyte;
//   * dequantization happens in registers: Q8_0 int8 -> fp32 (sign-extending byte select),
//     Q4_K nibbles masked in place are fp16 subnormals (q * 2^-24) feeding v_dot2_f32_f16,
//     MXFP4 E2M1 pairs -> fp16 with v_cvt_scalef32_pk_f16_fp4 feeding v_dot2_f32_f16;
//     block scales (fp16 d, 6-bit K-quant scales/mins, E8M0) are applied once per unit in fp32;
//   * R row sums per lane are reduced with DPP inside each row of 16 lanes and four
//     v_readlane across rows.
//
// Arithmetic restated from TensorSharp.Models/ManagedQuantizedOps.cs:156-200 (dot of a
// dequantised row with the activation row); activations are rounded to fp16 for the
// 4-bit formats (power-of-two pre-scaled so that no value overflows or underflows).
#include "tship_internal.h"

#include <algorithm>
#include <cstring>

namespace tship {
namespace {

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));

constexpr int kWaves = 4;
constexpr int kThreads = kWaves * 64;
constexpr int kMaxGroup = 8;

// one GEMV
struct GemvProblem {
    const uint8_t* w;
    int64_t w_bytes;
    const float* x;
    float* y;
    int N;
    int K;
};

// up to kMaxGroup independent GEMVs served by one launch; workgroups [wg_begin[i], wg_begin[i+1])
// work on problem i.  Passed by value as the kernel argument (no device-side descriptor memory).
struct GemvGroup {
    GemvProblem p[kMaxGroup];
    int wg_begin[kMaxGroup + 1];
    int count;
};

union H2U {
    uint32_t u;
    half2_t h;
};

__device__ __forceinline__ half2_t as_half2(uint32_t u)
{
    H2U c;
    c.u = u;
    return c.h;
}

__device__ __forceinline__ uint32_t pack_half2(float a, float b)
{
    H2U c;
    c.h = half2_t{(_Float16)a, (_Float16)b};
    return c.u;
}

__device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float acc)
{
    return __builtin_amdgcn_fdot2(as_half2(a), as_half2(b), acc, false);
}

// sum over the 64 lanes; result valid in every lane
__device__ __forceinline__ float wave_sum(float v)
{
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xb1, 0xf, 0xf, true));   // quad_perm [1,0,3,2]
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4e, 0xf, 0xf, true));   // quad_perm [2,3,0,1]
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xf, 0xf, true));  // row_half_mirror
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xf, 0xf, true));  // row_mirror
    const int iv = __float_as_int(v);
    return __int_as_float(__builtin_amdgcn_readlane(iv, 0)) + __int_as_float(__builtin_amdgcn_readlane(iv, 16)) +
           __int_as_float(__builtin_amdgcn_readlane(iv, 32)) + __int_as_float(__builtin_amdgcn_readlane(iv, 48));
}

// dword `idx` of the 4-byte aligned window starting at `al`, assembled from byte loads that stay
// inside [p, p + len): used only for the last unit of a tensor, where a full 128-bit load
// would read past the end of the weight bytes.
__device__ __forceinline__ uint32_t window_dword(uintptr_t al, int idx, uintptr_t p, int len)
{
    uint32_t v = 0;
#pragma unroll
    for (int b = 0; b < 4; ++b) {
        const uintptr_t addr = al + 4 * idx + b;
        if (addr >= p && addr < p + len) v |= (uint32_t)(*reinterpret_cast<const uint8_t*>(addr)) << (8 * b);
    }
    return v;
}

// max |x| over the workgroup -> power-of-two divisor that brings it into [2^13, 2^14) for fp16.
// Returns the inverse scale (to multiply x with) and writes the scale itself to *scale_out.
__device__ float block_prescale(const float* __restrict__ x, int K, float* red /* kWaves floats in LDS */,
                                float* scale_out)
{
    float amax = 0.f;
    for (int i = threadIdx.x; i < K; i += kThreads) amax = fmaxf(amax, fabsf(x[i]));
    // wave max with the same DPP ladder as wave_sum
    amax = fmaxf(amax, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(amax), 0xb1, 0xf, 0xf, true)));
    amax = fmaxf(amax, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(amax), 0x4e, 0xf, 0xf, true)));
    amax = fmaxf(amax, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(amax), 0x141, 0xf, 0xf, true)));
    amax = fmaxf(amax, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(amax), 0x140, 0xf, 0xf, true)));
    const int iv = __float_as_int(amax);
    const float wmax = fmaxf(fmaxf(__int_as_float(__builtin_amdgcn_readlane(iv, 0)), __int_as_float(__builtin_amdgcn_readlane(iv, 16))),
                             fmaxf(__int_as_float(__builtin_amdgcn_readlane(iv, 32)), __int_as_float(__builtin_amdgcn_readlane(iv, 48))));
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = wmax;
    __syncthreads();
    float m = red[0];
    for (int w = 1; w < kWaves; ++w) m = fmaxf(m, red[w]);
    // exponent of m (0 for zero / subnormal input); scale = 2^(exp - 13) so m/scale in [2^13, 2^14)
    int e = (int)((__float_as_uint(m) >> 23) & 0xffu);
    if (!(m < 3.0e38f)) e = 127;  // inf/NaN activations: leave unscaled, they propagate
    if (e < 14) e = 14;           // do not amplify tiny vectors beyond fp32 normal range handling
    const int se = e - 13;        // biased exponent of scale, >= 1
    *scale_out = __uint_as_float((uint32_t)se << 23);
    return __uint_as_float((uint32_t)(254 - se) << 23);
}

// ------------------------------------------------------------------------------------------
// Q4_K
// LDS unit (one 64-weight group, 144 B): 32 dwords of fp16 pairs in unpack order, then the two
// fp32 sums of the fp16-rounded activations of its two 32-weight sub-blocks, then 8 B pad.
// Unpack order of quant dword j (bytes 4j..4j+3 of the group's 32 quant bytes):
//   dword 4j+0 = (x[4j], x[4j+2])      low nibbles of bytes 0 and 2
//   dword 4j+1 = (x[4j+1], x[4j+3])    low nibbles of bytes 1 and 3
//   dword 4j+2 = (x[32+4j], x[32+4j+2])   high nibbles
//   dword 4j+3 = (x[32+4j+1], x[32+4j+3])
// ------------------------------------------------------------------------------------------
__device__ void stage_x_q4k(const float* __restrict__ x, int K, uint32_t* lds, float inv_scale)
{
    // one work item = 4 consecutive activations (one float4): items are coalesced across lanes
    const int items = K >> 2;
    for (int base = 0; base < items; base += kThreads) {
        // every lane of a wave stays in the loop together so the 8-lane sum below is well defined
        const int it = base + threadIdx.x;
        const bool live = it < items;
        float4 v = live ? reinterpret_cast<const float4*>(x)[it] : float4{0.f, 0.f, 0.f, 0.f};
        const int e = it << 2;        // first element
        const int g = e >> 6;         // group
        const int r = e & 63;
        const int sub = r >> 5;
        const int j = (r & 31) >> 2;
        const _Float16 h0 = (_Float16)(v.x * inv_scale), h1 = (_Float16)(v.y * inv_scale);
        const _Float16 h2 = (_Float16)(v.z * inv_scale), h3 = (_Float16)(v.w * inv_scale);
        H2U a, b;
        a.h = half2_t{h0, h2};
        b.h = half2_t{h1, h3};
        float s = ((float)h0 + (float)h1) + ((float)h2 + (float)h3);
        // sum over the 8 lanes that share a 32-weight sub-block (xor 1, 2, 4 inside a row of 16)
        s += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(s), 0xb1, 0xf, 0xf, true));
        s += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(s), 0x4e, 0xf, 0xf, true));
        s += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(s), 0x141, 0xf, 0xf, true));
        if (live) {
            uint32_t* unit = lds + g * 36;
            uint2 w2;
            w2.x = a.u;
            w2.y = b.u;
            *reinterpret_cast<uint2*>(unit + 4 * j + 2 * sub) = w2;
            if ((threadIdx.x & 7) == 0) reinterpret_cast<float*>(unit)[32 + sub] = s;
        }
    }
}

template <int R>
__device__ __forceinline__ void gemv_q4k_body(const GemvProblem& P, int wg, int nwg, uint32_t* lds, float* red)
{
    const uint8_t* __restrict__ W = P.w;
    const float* __restrict__ x = P.x;
    float* __restrict__ y = P.y;
    const int N = P.N, K = P.K;
    float xscale;
    const float inv = block_prescale(x, K, red, &xscale);
    stage_x_q4k(x, K, lds, inv);
    __syncthreads();

    const int lane = threadIdx.x & 63;
    const int upr = K >> 6;  // units per row
    const int64_t row_bytes = (int64_t)(K >> 8) * 144;
    const int nrb = (N + R - 1) / R;
    const int wave_stride = nwg * kWaves;
    for (int rb = wg * kWaves + (threadIdx.x >> 6); rb < nrb; rb += wave_stride) {
        const int row0 = rb * R;
        const int rows = min(R, N - row0);
        const int total = rows * upr;
        const uint8_t* base = W + (int64_t)row0 * row_bytes;
        float acc[R];
#pragma unroll
        for (int i = 0; i < R; ++i) acc[i] = 0.f;
        int r = 0, g = lane;
        for (int u = lane; u < total; u += 64) {
            while (g >= upr) {
                g -= upr;
                ++r;
            }
            const uint8_t* blk = base + (int64_t)r * row_bytes + (g >> 2) * 144;
            const int g4 = g & 3;
            const uint4 hdr = *reinterpret_cast<const uint4*>(blk);
            const uint4 qa = *reinterpret_cast<const uint4*>(blk + 16 + g4 * 32);
            const uint4 qb = *reinterpret_cast<const uint4*>(blk + 32 + g4 * 32);
            const uint4* xu = reinterpret_cast<const uint4*>(lds + g * 36);

            float lo = 0.f, hi = 0.f;
            const uint32_t qw[8] = {qa.x, qa.y, qa.z, qa.w, qb.x, qb.y, qb.z, qb.w};
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const uint4 xv = xu[j];
                const uint32_t w = qw[j];
                const uint32_t w8 = w >> 8;
                // a nibble left in place is an fp16 subnormal: q * 2^-24 (low) or 16q * 2^-24 (high);
                // v_dot2_f32_f16 honours fp16 denormals, so the integer values enter the dot exactly
                lo = dot2(w & 0x000f000fu, xv.x, lo);
                lo = dot2(w8 & 0x000f000fu, xv.y, lo);
                hi = dot2(w & 0x00f000f0u, xv.z, hi);
                hi = dot2(w8 & 0x00f000f0u, xv.w, hi);
            }
            const uint4 tail = xu[8];
            const float s1 = __uint_as_float(tail.x), s2 = __uint_as_float(tail.y);
            const float dl = lo * 16777216.f;   // 2^24
            const float dh = hi * 1048576.f;    // 2^24 / 16

            // 6-bit scales / mins of sub-blocks 2*g4 and 2*g4+1 (ggml-quants.c:703-710)
            const int sh = (g4 & 1) * 16;
            const uint32_t a = hdr.y >> sh, b = hdr.z >> sh, c = hdr.w >> sh;
            uint32_t sc1, sc2, m1, m2;
            if (g4 < 2) {
                sc1 = a & 63u;
                sc2 = (a >> 8) & 63u;
                m1 = b & 63u;
                m2 = (b >> 8) & 63u;
            } else {
                sc1 = (c & 0x0fu) | ((a >> 2) & 0x30u);
                sc2 = ((c >> 8) & 0x0fu) | ((a >> 10) & 0x30u);
                m1 = ((c >> 4) & 0x0fu) | ((b >> 2) & 0x30u);
                m2 = ((c >> 12) & 0x0fu) | ((b >> 10) & 0x30u);
            }
            const half2_t dm = as_half2(hdr.x);
            const float d = (float)dm.x, dmin = (float)dm.y;
            const float part = d * ((float)sc1 * dl + (float)sc2 * dh) - dmin * ((float)m1 * s1 + (float)m2 * s2);
#pragma unroll
            for (int i = 0; i < R; ++i) acc[i] += (r == i) ? part : 0.f;
            g += 64;
        }
#pragma unroll
        for (int i = 0; i < R; ++i) {
            const float t = wave_sum(acc[i]);
            if (lane == 0 && i < rows) y[row0 + i] = t * xscale;
        }
    }
}

// ------------------------------------------------------------------------------------------
// MXFP4
// LDS unit (one 32-weight block, 80 B): 16 dwords (x[j], x[j+16]) as fp16 pairs, 16 B pad.
// ------------------------------------------------------------------------------------------
__device__ void stage_x_mxfp4(const float* __restrict__ x, int K, uint32_t* lds, float inv_scale)
{
    // one work item = x[b*32 + 4i .. +3] and x[b*32 + 16 + 4i .. +3]  -> 4 dwords
    const int items = K >> 3;
    for (int it = threadIdx.x; it < items; it += kThreads) {
        const int b = it >> 2, i = it & 3;
        const float4 lo = *reinterpret_cast<const float4*>(x + b * 32 + 4 * i);
        const float4 hi = *reinterpret_cast<const float4*>(x + b * 32 + 16 + 4 * i);
        uint4 o;
        o.x = pack_half2(lo.x * inv_scale, hi.x * inv_scale);
        o.y = pack_half2(lo.y * inv_scale, hi.y * inv_scale);
        o.z = pack_half2(lo.z * inv_scale, hi.z * inv_scale);
        o.w = pack_half2(lo.w * inv_scale, hi.w * inv_scale);
        *reinterpret_cast<uint4*>(lds + b * 20 + 4 * i) = o;
    }
}

// E2M1 pair (low nibble, high nibble of byte `sel`) -> fp16 pair, exact
template <int SEL>
__device__ __forceinline__ uint32_t fp4_pair(uint32_t w)
{
    H2U c;
    c.h = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, 1.0f, SEL);
    return c.u;
}

template <int R>
__device__ __forceinline__ void gemv_mxfp4_body(const GemvProblem& P, int wg, int nwg, uint32_t* lds, float* red)
{
    const uint8_t* __restrict__ W = P.w;
    const int64_t w_bytes = P.w_bytes;
    const float* __restrict__ x = P.x;
    float* __restrict__ y = P.y;
    const int N = P.N, K = P.K;
    float xscale;
    const float inv = block_prescale(x, K, red, &xscale);
    stage_x_mxfp4(x, K, lds, inv);
    __syncthreads();

    const int lane = threadIdx.x & 63;
    const int upr = K >> 5;
    const int64_t row_bytes = (int64_t)upr * 17;
    const int nrb = (N + R - 1) / R;
    const int wave_stride = nwg * kWaves;
    const uintptr_t w_end = reinterpret_cast<uintptr_t>(W) + (uintptr_t)w_bytes;
    for (int rb = wg * kWaves + (threadIdx.x >> 6); rb < nrb; rb += wave_stride) {
        const int row0 = rb * R;
        const int rows = min(R, N - row0);
        const int total = rows * upr;
        const uint8_t* base = W + (int64_t)row0 * row_bytes;
        float acc[R];
#pragma unroll
        for (int i = 0; i < R; ++i) acc[i] = 0.f;
        int r = 0, g = lane;
        for (int u = lane; u < total; u += 64) {
            while (g >= upr) {
                g -= upr;
                ++r;
            }
            const uintptr_t p = reinterpret_cast<uintptr_t>(base) + (uintptr_t)((int64_t)r * row_bytes + (int64_t)g * 17);
            const uintptr_t al = p & ~(uintptr_t)3;
            const uint32_t o = (uint32_t)(p & 3);
            uint32_t a0, a1, a2, a3, a4;
            if (al + 20 <= w_end) {
                const uint4 v = *reinterpret_cast<const uint4*>(al);  // 4-byte aligned 128-bit global load
                a0 = v.x; a1 = v.y; a2 = v.z; a3 = v.w;
                a4 = *reinterpret_cast<const uint32_t*>(al + 16);
            } else {
                // last unit of the tensor: never read past the end of the weight bytes
                a0 = window_dword(al, 0, p, 17); a1 = window_dword(al, 1, p, 17); a2 = window_dword(al, 2, p, 17);
                a3 = window_dword(al, 3, p, 17); a4 = window_dword(al, 4, p, 17);
            }
            const uint32_t e = (a0 >> (8 * o)) & 0xffu;
            // quant bytes start at byte o+1 of the aligned window
            const bool wrap = o == 3;
            const uint32_t b0 = wrap ? a1 : a0, b1 = wrap ? a2 : a1, b2 = wrap ? a3 : a2, b3 = wrap ? a4 : a3;
            const uint32_t b4 = a4;
            const uint32_t shb = (o + 1) & 3;
            const uint32_t q0 = __builtin_amdgcn_alignbyte(b1, b0, shb);
            const uint32_t q1 = __builtin_amdgcn_alignbyte(b2, b1, shb);
            const uint32_t q2 = __builtin_amdgcn_alignbyte(b3, b2, shb);
            const uint32_t q3 = __builtin_amdgcn_alignbyte(b4, b3, shb);

            const uint4* xu = reinterpret_cast<const uint4*>(lds + g * 20);
            const uint4 x0 = xu[0], x1 = xu[1], x2 = xu[2], x3 = xu[3];
            float s = 0.f;
            s = dot2(fp4_pair<0>(q0), x0.x, s); s = dot2(fp4_pair<1>(q0), x0.y, s);
            s = dot2(fp4_pair<2>(q0), x0.z, s); s = dot2(fp4_pair<3>(q0), x0.w, s);
            s = dot2(fp4_pair<0>(q1), x1.x, s); s = dot2(fp4_pair<1>(q1), x1.y, s);
            s = dot2(fp4_pair<2>(q1), x1.z, s); s = dot2(fp4_pair<3>(q1), x1.w, s);
            s = dot2(fp4_pair<0>(q2), x2.x, s); s = dot2(fp4_pair<1>(q2), x2.y, s);
            s = dot2(fp4_pair<2>(q2), x2.z, s); s = dot2(fp4_pair<3>(q2), x2.w, s);
            s = dot2(fp4_pair<0>(q3), x3.x, s); s = dot2(fp4_pair<1>(q3), x3.y, s);
            s = dot2(fp4_pair<2>(q3), x3.z, s); s = dot2(fp4_pair<3>(q3), x3.w, s);
            // table value = 2 * E2M1, block scale = 2^(e-128)  ->  E2M1 * 2^(e-127)
            const float scale = __uint_as_float(e == 0 ? 0x00400000u : (e << 23));
            const float part = s * scale;
#pragma unroll
            for (int i = 0; i < R; ++i) acc[i] += (r == i) ? part : 0.f;
            g += 64;
        }
#pragma unroll
        for (int i = 0; i < R; ++i) {
            const float t = wave_sum(acc[i]);
            if (lane == 0 && i < rows) y[row0 + i] = t * xscale;
        }
    }
}

// ------------------------------------------------------------------------------------------
// Q8_0
// LDS unit (one 32-weight block, 144 B): 32 fp32 activations, 16 B pad.  fp32 throughout.
// ------------------------------------------------------------------------------------------
__device__ void stage_x_q80(const float* __restrict__ x, int K, float* lds)
{
    const int items = K >> 2;
    for (int it = threadIdx.x; it < items; it += kThreads) {
        const float4 v = reinterpret_cast<const float4*>(x)[it];
        *reinterpret_cast<float4*>(lds + (it >> 3) * 36 + (it & 7) * 4) = v;
    }
}

__device__ __forceinline__ float dot4_i8(uint32_t q, float4 xv, float acc)
{
    acc += (float)(int8_t)(q & 0xffu) * xv.x;
    acc += (float)(int8_t)((q >> 8) & 0xffu) * xv.y;
    acc += (float)(int8_t)((q >> 16) & 0xffu) * xv.z;
    acc += (float)(int8_t)(q >> 24) * xv.w;
    return acc;
}

template <int R>
__device__ __forceinline__ void gemv_q80_body(const GemvProblem& P, int wg, int nwg, uint32_t* lds, float* /*red*/)
{
    const uint8_t* __restrict__ W = P.w;
    const int64_t w_bytes = P.w_bytes;
    const float* __restrict__ x = P.x;
    float* __restrict__ y = P.y;
    const int N = P.N, K = P.K;
    float* xl = reinterpret_cast<float*>(lds);
    stage_x_q80(x, K, xl);
    __syncthreads();

    const int lane = threadIdx.x & 63;
    const int upr = K >> 5;
    const int64_t row_bytes = (int64_t)upr * 34;
    const int nrb = (N + R - 1) / R;
    const int wave_stride = nwg * kWaves;
    const uintptr_t w_end = reinterpret_cast<uintptr_t>(W) + (uintptr_t)w_bytes;
    for (int rb = wg * kWaves + (threadIdx.x >> 6); rb < nrb; rb += wave_stride) {
        const int row0 = rb * R;
        const int rows = min(R, N - row0);
        const int total = rows * upr;
        const uint8_t* base = W + (int64_t)row0 * row_bytes;
        float acc[R];
#pragma unroll
        for (int i = 0; i < R; ++i) acc[i] = 0.f;
        int r = 0, g = lane;
        for (int u = lane; u < total; u += 64) {
            while (g >= upr) {
                g -= upr;
                ++r;
            }
            const uintptr_t p = reinterpret_cast<uintptr_t>(base) + (uintptr_t)((int64_t)r * row_bytes + (int64_t)g * 34);
            const uintptr_t al = p & ~(uintptr_t)3;
            const bool odd = (p & 2) != 0;  // blocks are 2-byte aligned: window offset is 0 or 2
            uint32_t a[9];
            if (al + 36 <= w_end) {
                const uint4 v0 = *reinterpret_cast<const uint4*>(al);
                const uint4 v1 = *reinterpret_cast<const uint4*>(al + 16);
                a[0] = v0.x; a[1] = v0.y; a[2] = v0.z; a[3] = v0.w;
                a[4] = v1.x; a[5] = v1.y; a[6] = v1.z; a[7] = v1.w;
                a[8] = *reinterpret_cast<const uint32_t*>(al + 32);
            } else {
#pragma unroll
                for (int i = 0; i < 9; ++i) a[i] = window_dword(al, i, p, 34);
            }
            const uint32_t dbits = odd ? (a[0] >> 16) : (a[0] & 0xffffu);
            H2U dh;
            dh.u = dbits;
            const float d = (float)dh.h.x;
            const float4* xu = reinterpret_cast<const float4*>(xl + g * 36);
            float s = 0.f;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const uint32_t q = odd ? a[i + 1] : __builtin_amdgcn_alignbyte(a[i + 1], a[i], 2);
                s = dot4_i8(q, xu[i], s);
            }
            const float part = s * d;
#pragma unroll
            for (int i = 0; i < R; ++i) acc[i] += (r == i) ? part : 0.f;
            g += 64;
        }
#pragma unroll
        for (int i = 0; i < R; ++i) {
            const float t = wave_sum(acc[i]);
            if (lane == 0 && i < rows) y[row0 + i] = t;
        }
    }
}

template <int TYPE, int R>
__global__ void __launch_bounds__(kThreads) gemv_kernel(const GemvGroup G)
{
    extern __shared__ uint32_t lds[];
    __shared__ float red[kWaves];
    int i = 0;
#pragma unroll
    for (int j = 1; j < kMaxGroup; ++j)
        if (j < G.count && (int)blockIdx.x >= G.wg_begin[j]) i = j;
    const int wg = (int)blockIdx.x - G.wg_begin[i];
    const int nwg = G.wg_begin[i + 1] - G.wg_begin[i];
    if (TYPE == kTypeQ4_K) gemv_q4k_body<R>(G.p[i], wg, nwg, lds, red);
    else if (TYPE == kTypeMXFP4) gemv_mxfp4_body<R>(G.p[i], wg, nwg, lds, red);
    else gemv_q80_body<R>(G.p[i], wg, nwg, lds, red);
}

size_t lds_bytes_for(int type, int K)
{
    switch (type) {
    case kTypeQ8_0: return (size_t)(K / 32) * 144;
    case kTypeQ4_K: return (size_t)(K / 64) * 144;
    case kTypeMXFP4: return (size_t)(K / 32) * 80;
    default: return 0;
    }
}

constexpr size_t kMaxLds = 160 * 1024 - 1024;

template <int TYPE, int R>
bool launch_instance(const GemvGroup& g, int grid, size_t lds, hipStream_t stream)
{
    auto kern = gemv_kernel<TYPE, R>;
    if (lds > 64 * 1024 &&
        !hip_ok(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                    (int)lds),
                "gemv: raising the dynamic LDS limit"))
        return false;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(kThreads), lds, stream, g);
    return hip_ok(hipGetLastError(), "gemv launch");
}

template <int TYPE>
bool launch_type(const GemvGroup& g, int R, int grid, size_t lds, hipStream_t stream)
{
    if (R == 4) return launch_instance<TYPE, 4>(g, grid, lds, stream);
    if (R == 2) return launch_instance<TYPE, 2>(g, grid, lds, stream);
    return launch_instance<TYPE, 1>(g, grid, lds, stream);
}

}  // namespace

int gemv_max_k(int type)
{
    switch (type) {
    case kTypeQ8_0: return (int)(kMaxLds / 144) * 32;
    case kTypeQ4_K: return (int)(kMaxLds / 144) * 64;
    case kTypeMXFP4: return (int)(kMaxLds / 80) * 32;
    default: return 0;
    }
}

int gemv_max_group() { return kMaxGroup; }

bool launch_gemv_group(int type, int count, const GemvArgs* args, hipStream_t stream)
{
    if (count < 1 || count > kMaxGroup) {
        set_last_error("gemv: group size out of range.");
        return false;
    }
    if (type != kTypeQ8_0 && type != kTypeQ4_K && type != kTypeMXFP4) {
        set_last_error("gemv: unsupported type.");
        return false;
    }
    const DeviceInfo& di = device_info();
    size_t lds = 0;
    int64_t total_rows = 0;
    double total_bytes = 0;
    for (int i = 0; i < count; ++i) {
        if (args[i].K > gemv_max_k(type)) {
            set_last_error("gemv: K exceeds what one workgroup can stage in LDS.");
            return false;
        }
        lds = std::max(lds, lds_bytes_for(type, args[i].K));
        total_rows += args[i].N;
        total_bytes += (double)args[i].w_bytes;
    }
    // rows per wavefront step: keep at least ~16 waves per CU worth of row blocks
    int R = 4;
    while (R > 1 && total_rows / R < (int64_t)di.num_cus * 16) R >>= 1;
    int per_cu = (int)std::min<size_t>(8, (160 * 1024) / (lds + 256));
    if (per_cu < 1) per_cu = 1;
    const int budget = di.num_cus * per_cu;

    GemvGroup g;
    std::memset(&g, 0, sizeof(g));
    g.count = count;
    int begin = 0;
    for (int i = 0; i < count; ++i) {
        g.p[i].w = static_cast<const uint8_t*>(args[i].w);
        g.p[i].w_bytes = args[i].w_bytes;
        g.p[i].x = args[i].x;
        g.p[i].y = args[i].y;
        g.p[i].N = args[i].N;
        g.p[i].K = args[i].K;
        const int nrb = (args[i].N + R - 1) / R;
        const int wg_needed = (nrb + kWaves - 1) / kWaves;
        // workgroups in proportion to the bytes each problem streams
        int share = (int)((double)budget * (double)args[i].w_bytes / total_bytes + 0.5);
        share = std::max(1, std::min(share, wg_needed));
        g.wg_begin[i] = begin;
        begin += share;
    }
    for (int i = count; i <= kMaxGroup; ++i) g.wg_begin[i] = begin;
    const int grid = begin;
    switch (type) {
    case kTypeQ4_K: return launch_type<kTypeQ4_K>(g, R, grid, lds, stream);
    case kTypeMXFP4: return launch_type<kTypeMXFP4>(g, R, grid, lds, stream);
    default: return launch_type<kTypeQ8_0>(g, R, grid, lds, stream);
    }
}

bool launch_gemv(int type, const void* w, int64_t w_bytes, const float* x, float* y, int N, int K, hipStream_t stream)
{
    GemvArgs a{w, w_bytes, x, y, N, K};
    return launch_gemv_group(type, 1, &a, stream);
}

}  // namespace tship
