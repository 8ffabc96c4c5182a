// Bit-exact dequantization of raw GGUF blocks to fp32 on gfx950.
//
// The arithmetic is the managed dequantizers' (TensorSharp.Models/ManagedQuantizedOps.cs:411-427 Q8_0, :429-445 Q8_1,
// :447-479 Q4_K, :579-598 MXFP4; :268-409 and :481-577 for F16, BF16, Q4_0, Q4_1, Q5_0, Q5_1, Q5_K, Q6_K, IQ4_NL):
// every product is exact in fp32, the subtract of Q4_K / Q5_K and the add of Q4_1 / Q5_1 are the one rounding.
// Contraction is switched off so the multiply and the subtract stay separately rounded operations.
// fp16 scales are widened with integer arithmetic, so the result does not depend on the wave's
// denormal mode.
#include "tship_internal.h"

#pragma clang fp contract(off)

namespace tship {
namespace {

__device__ __forceinline__ float half_bits_to_float(uint32_t h)
{
    const uint32_t sign = (h & 0x8000u) << 16;
    const uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    uint32_t bits;
    if (exp == 0x1fu) {
        bits = sign | 0x7f800000u | (man << 13);
    } else if (exp != 0) {
        bits = sign | ((exp + 112u) << 23) | (man << 13);
    } else if (man == 0) {
        bits = sign;
    } else {
        const int lz = __clz(man) - 21;  // leading zeros inside the 11-bit field
        man = (man << lz) & 0x3ffu;
        bits = sign | ((uint32_t)(113 - lz) << 23) | (man << 13);
    }
    return __uint_as_float(bits);
}

// 2^(e-128): ggml-impl.h:471-489, ManagedQuantizedOps.cs:678-682
__device__ __forceinline__ float e8m0_half_scale(uint32_t e)
{
    return __uint_as_float(e < 2 ? (0x00200000u << e) : ((e - 1u) << 23));
}

__device__ __forceinline__ float mxfp4_value(uint32_t nib)
{
    // doubled E2M1 table {0,1,2,3,4,6,8,12, 0,-1,-2,-3,-4,-6,-8,-12} as signed bytes
    // (ggml-common.h:1094-1096); the integer route keeps code 8 at +0 like the reference.
    const uint64_t pos = 0x0c08060403020100ull;
    const uint64_t neg = 0xf4f8fafcfdfeff00ull;
    const uint64_t tab = (nib & 8u) ? neg : pos;
    return (float)(int)(int8_t)((tab >> ((nib & 7u) * 8)) & 0xffu);
}

// Q8_1 (ggml-common.h block_q8_1: fp16 d, fp16 s = d * sum(q), int8 qs[32] = 36 bytes): y = q * d, s is not read
__device__ __forceinline__ float4 dequant4_q8_1(const uint8_t* src, int64_t e0)
{
    const uint8_t* blk = src + (e0 >> 5) * 36;
    const int j = (int)(e0 & 31);
    const float d = half_bits_to_float((uint32_t)blk[0] | ((uint32_t)blk[1] << 8));
    float4 o;
    o.x = (float)(int8_t)blk[4 + j] * d;
    o.y = (float)(int8_t)blk[5 + j] * d;
    o.z = (float)(int8_t)blk[6 + j] * d;
    o.w = (float)(int8_t)blk[7 + j] * d;
    return o;
}

// 4 consecutive outputs starting at element e0 (a multiple of 4) of the block sequence at src
__device__ __forceinline__ float4 dequant4_q8_0(const uint8_t* src, int64_t e0)
{
    const uint8_t* blk = src + (e0 >> 5) * 34;
    const int j = (int)(e0 & 31);
    const float d = half_bits_to_float((uint32_t)blk[0] | ((uint32_t)blk[1] << 8));
    float4 o;
    o.x = (float)(int8_t)blk[2 + j] * d;
    o.y = (float)(int8_t)blk[3 + j] * d;
    o.z = (float)(int8_t)blk[4 + j] * d;
    o.w = (float)(int8_t)blk[5 + j] * d;
    return o;
}

__device__ __forceinline__ float4 dequant4_q4_K(const uint8_t* src, int64_t e0)
{
    const uint8_t* blk = src + (e0 >> 8) * 144;
    const int r = (int)(e0 & 255);
    const int g = r >> 6;          // 64-group
    const int hi = (r >> 5) & 1;   // 0: low nibbles, 1: high nibbles
    const int l = r & 31;
    const int j = 2 * g + hi;      // sub-block
    const float d = half_bits_to_float((uint32_t)blk[0] | ((uint32_t)blk[1] << 8));
    const float dmin = half_bits_to_float((uint32_t)blk[2] | ((uint32_t)blk[3] << 8));
    const uint8_t* p = blk + 4;
    uint32_t sc, mn;
    if (j < 4) {
        sc = p[j] & 63u;
        mn = p[j + 4] & 63u;
    } else {
        sc = (p[j + 4] & 0x0fu) | ((uint32_t)(p[j - 4] >> 6) << 4);
        mn = (uint32_t)(p[j + 4] >> 4) | ((uint32_t)(p[j] >> 6) << 4);
    }
    const float d1 = d * (float)sc;
    const float m1 = dmin * (float)mn;
    const uint8_t* q = blk + 16 + 32 * g + l;
    const int sh = hi * 4;
    float4 o;
    o.x = d1 * (float)((q[0] >> sh) & 0x0fu) - m1;
    o.y = d1 * (float)((q[1] >> sh) & 0x0fu) - m1;
    o.z = d1 * (float)((q[2] >> sh) & 0x0fu) - m1;
    o.w = d1 * (float)((q[3] >> sh) & 0x0fu) - m1;
    return o;
}

__device__ __forceinline__ float4 dequant4_mxfp4(const uint8_t* src, int64_t e0)
{
    const uint8_t* blk = src + (e0 >> 5) * 17;
    const int j = (int)(e0 & 31);
    const int sh = (j >> 4) * 4;
    const uint8_t* q = blk + 1 + (j & 15);
    const float d = e8m0_half_scale(blk[0]);
    float4 o;
    o.x = d * mxfp4_value((q[0] >> sh) & 0x0fu);
    o.y = d * mxfp4_value((q[1] >> sh) & 0x0fu);
    o.z = d * mxfp4_value((q[2] >> sh) & 0x0fu);
    o.w = d * mxfp4_value((q[3] >> sh) & 0x0fu);
    return o;
}


// ---- formats used for dequantization / embedding gather only (ManagedQuantizedOps.cs:268-409, :481-577) ----
__device__ __forceinline__ uint32_t rd16u(const uint8_t* p) { return (uint32_t)p[0] | ((uint32_t)p[1] << 8); }
__device__ __forceinline__ uint32_t rd32u(const uint8_t* p) { return rd16u(p) | (rd16u(p + 2) << 16); }

__device__ __forceinline__ float4 dequant4_f16(const uint8_t* src, int64_t e0)
{
    const uint8_t* p = src + e0 * 2;
    return float4{half_bits_to_float(rd16u(p)), half_bits_to_float(rd16u(p + 2)), half_bits_to_float(rd16u(p + 4)),
                  half_bits_to_float(rd16u(p + 6))};
}

__device__ __forceinline__ float4 dequant4_bf16(const uint8_t* src, int64_t e0)
{
    const uint8_t* p = src + e0 * 2;
    return float4{__uint_as_float(rd16u(p) << 16), __uint_as_float(rd16u(p + 2) << 16), __uint_as_float(rd16u(p + 4) << 16),
                  __uint_as_float(rd16u(p + 6) << 16)};
}

// Q4_0 / Q4_1 / Q5_0 / Q5_1 / IQ4_NL: 32 weights, low nibbles are elements 0..15, high nibbles 16..31;
// HDR bytes of scales (and the 32 fifth bits) in front of the 16 quant bytes
template <int TYPE>
__device__ __forceinline__ float4 dequant4_legacy(const uint8_t* src, int64_t e0)
{
    constexpr int kHdr = TYPE == kTypeQ4_0 || TYPE == kTypeIQ4_NL ? 2 : TYPE == kTypeQ4_1 ? 4 : TYPE == kTypeQ5_0 ? 6 : 8;
    constexpr bool kMin = TYPE == kTypeQ4_1 || TYPE == kTypeQ5_1;
    constexpr bool kFive = TYPE == kTypeQ5_0 || TYPE == kTypeQ5_1;
    const uint8_t* blk = src + (e0 >> 5) * (kHdr + 16);
    const int j = (int)(e0 & 31);
    const int sh = (j >> 4) * 4;
    const uint8_t* q = blk + kHdr + (j & 15);
    const float d = half_bits_to_float(rd16u(blk));
    const float m = kMin ? half_bits_to_float(rd16u(blk + 2)) : 0.f;
    const uint32_t qh = kFive ? rd32u(blk + kHdr - 4) : 0u;
    float o[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        int v = (q[i] >> sh) & 0x0f;
        if (kFive) v |= (int)((qh >> (j + i)) & 1u) << 4;
        if (TYPE == kTypeIQ4_NL) {
            // {-127,-104,-83,-65,-49,-35,-22,-10, 1,13,25,38,53,69,89,113} as signed bytes (ManagedQuantizedOps.cs:30-33)
            const uint64_t tab = (v & 8) ? 0x7159453526190d01ull : 0xf6eaddcfbfad9881ull;
            o[i] = d * (float)(int)(int8_t)((tab >> ((v & 7) * 8)) & 0xffu);
        } else if (kMin) {
            o[i] = (float)v * d + m;
        } else {
            o[i] = (float)(v - (kFive ? 16 : 8)) * d;
        }
    }
    return float4{o[0], o[1], o[2], o[3]};
}

// Q5_K: d, dmin, scales[12], qh[32], ql[128]; y = (d*sc) * (nibble + 16*bit) - (dmin*m)
__device__ __forceinline__ float4 dequant4_q5_K(const uint8_t* src, int64_t e0)
{
    const uint8_t* blk = src + (e0 >> 8) * 176;
    const int r = (int)(e0 & 255);
    const int g = r >> 6, hi = (r >> 5) & 1, l = r & 31;
    const int j = 2 * g + hi;
    const float d = half_bits_to_float(rd16u(blk));
    const float dmin = half_bits_to_float(rd16u(blk + 2));
    const uint8_t* p = blk + 4;
    uint32_t sc, mn;
    if (j < 4) {
        sc = p[j] & 63u;
        mn = p[j + 4] & 63u;
    } else {
        sc = (p[j + 4] & 0x0fu) | ((uint32_t)(p[j - 4] >> 6) << 4);
        mn = (uint32_t)(p[j + 4] >> 4) | ((uint32_t)(p[j] >> 6) << 4);
    }
    const float d1 = d * (float)sc;
    const float m1 = dmin * (float)mn;
    const uint8_t* qh = blk + 16 + l;
    const uint8_t* q = blk + 48 + 32 * g + l;
    const int sh = hi * 4;
    float o[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = d1 * (float)(((q[i] >> sh) & 0x0fu) + (((qh[i] >> j) & 1u) << 4)) - m1;
    return float4{o[0], o[1], o[2], o[3]};
}

// Q6_K: ql[128], qh[64], int8 scales[16], fp16 d; y = d * scale * (q - 32)
__device__ __forceinline__ float4 dequant4_q6_K(const uint8_t* src, int64_t e0)
{
    const uint8_t* blk = src + (e0 >> 8) * 210;
    const int r = (int)(e0 & 255);
    const int half = r >> 7, grp = (r >> 5) & 3, l = r & 31;
    const uint8_t* ql = blk + 64 * half + 32 * (grp & 1) + l;
    const uint8_t* qh = blk + 128 + 32 * half + l;
    const float d = half_bits_to_float(rd16u(blk + 208));
    const float ds = d * (float)(int)(int8_t)blk[192 + 8 * half + 2 * grp + (l >> 4)];
    const int sh = (grp >> 1) * 4;
    float o[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int q = (int)(((ql[i] >> sh) & 0x0fu) | (((qh[i] >> (2 * grp)) & 3u) << 4)) - 32;
        o[i] = ds * (float)q;
    }
    return float4{o[0], o[1], o[2], o[3]};
}

template <int TYPE>
__device__ __forceinline__ float4 dequant4(const uint8_t* src, int64_t e0)
{
    if (TYPE == kTypeQ8_0) return dequant4_q8_0(src, e0);
    if (TYPE == kTypeQ8_1) return dequant4_q8_1(src, e0);
    if (TYPE == kTypeQ4_K) return dequant4_q4_K(src, e0);
    if (TYPE == kTypeMXFP4) return dequant4_mxfp4(src, e0);
    if (TYPE == kTypeF16) return dequant4_f16(src, e0);
    if (TYPE == kTypeBF16) return dequant4_bf16(src, e0);
    if (TYPE == kTypeQ4_0 || TYPE == kTypeQ4_1 || TYPE == kTypeQ5_0 || TYPE == kTypeQ5_1 || TYPE == kTypeIQ4_NL)
        return dequant4_legacy<TYPE>(src, e0);
    if (TYPE == kTypeQ5_K) return dequant4_q5_K(src, e0);
    if (TYPE == kTypeQ6_K) return dequant4_q6_K(src, e0);
    const float* f = reinterpret_cast<const float*>(src) + e0;      // F32 rows: plain copy
    return float4{f[0], f[1], f[2], f[3]};
}

// one thread -> 4 consecutive outputs
template <int TYPE>
__global__ void __launch_bounds__(256) dequant_kernel(const uint8_t* __restrict__ src, float* __restrict__ dst, int64_t n4)
{
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (t >= n4) return;
    reinterpret_cast<float4*>(dst)[t] = dequant4<TYPE>(src, t * 4);
}

constexpr int kWideItems = 1;      // items of 8 weights per thread in the wide dequantization kernels (2 and 4 measured slower)

// A little-endian dword / word at any byte address (global memory takes unaligned addresses; where the compiler may
// not assume that, it falls back to byte loads by itself).
__device__ __forceinline__ uint32_t load_u32(const uint8_t* p)
{
    uint32_t v;
    __builtin_memcpy(&v, p, 4);
    return v;
}
__device__ __forceinline__ uint32_t load_u16(const uint8_t* p)
{
    uint16_t v;
    __builtin_memcpy(&v, p, 2);
    return v;
}

// Q8_0: one thread takes a quarter of a block: the scale and eight quants (two dwords) -> 32 contiguous output bytes.
// y = q * d (ManagedQuantizedOps.cs:411-427).
__global__ void __launch_bounds__(256) dequant_q8_0_wide_kernel(const uint8_t* __restrict__ src, float* __restrict__ dst, int64_t n8)
{
    // kWideItems quarter blocks per thread, 256 apart, all loads issued before the first store
    const int64_t t0 = (int64_t)blockIdx.x * (256 * kWideItems) + threadIdx.x;
    uint32_t dh[kWideItems], q0[kWideItems], q1[kWideItems];
#pragma unroll
    for (int u = 0; u < kWideItems; ++u) {
        const int64_t t = t0 + 256 * u;
        if (t < n8) {
            const uint8_t* blk = src + (t >> 2) * 34;
            const int part = (int)(t & 3);
            dh[u] = load_u16(blk);
            q0[u] = load_u32(blk + 2 + 8 * part);
            q1[u] = load_u32(blk + 6 + 8 * part);
        }
    }
#pragma unroll
    for (int u = 0; u < kWideItems; ++u) {
        const int64_t t = t0 + 256 * u;
        if (t < n8) {
            const float d = half_bits_to_float(dh[u]);
            float4 a, b;
            a.x = (float)(int8_t)(q0[u] & 0xffu) * d;
            a.y = (float)(int8_t)((q0[u] >> 8) & 0xffu) * d;
            a.z = (float)(int8_t)((q0[u] >> 16) & 0xffu) * d;
            a.w = (float)(int8_t)(q0[u] >> 24) * d;
            b.x = (float)(int8_t)(q1[u] & 0xffu) * d;
            b.y = (float)(int8_t)((q1[u] >> 8) & 0xffu) * d;
            b.z = (float)(int8_t)((q1[u] >> 16) & 0xffu) * d;
            b.w = (float)(int8_t)(q1[u] >> 24) * d;
            float4* o = reinterpret_cast<float4*>(dst + t * 8);
            o[0] = a;
            o[1] = b;
        }
    }
}

// MXFP4: one thread takes the scale byte and one dword of a block's quants: four weights in the low nibbles
// (elements 4 part ..) and four in the high nibbles (elements 16 + 4 part ..).  value = table[nibble] * 2^(e - 128)
// (ManagedQuantizedOps.cs:579-598).
__global__ void __launch_bounds__(256) dequant_mxfp4_wide_kernel(const uint8_t* __restrict__ src, float* __restrict__ dst, int64_t n8)
{
    const int64_t t0 = (int64_t)blockIdx.x * (256 * kWideItems) + threadIdx.x;
    uint32_t e[kWideItems], q[kWideItems];
#pragma unroll
    for (int u = 0; u < kWideItems; ++u) {
        const int64_t t = t0 + 256 * u;
        if (t < n8) {
            const uint8_t* blk = src + (t >> 2) * 17;
            e[u] = blk[0];
            q[u] = load_u32(blk + 1 + 4 * (int)(t & 3));
        }
    }
#pragma unroll
    for (int u = 0; u < kWideItems; ++u) {
        const int64_t t = t0 + 256 * u;
        if (t < n8) {
            const float d = e8m0_half_scale(e[u]);
            const uint32_t v = q[u];
            float4 lo, hi;
            lo.x = d * mxfp4_value(v & 0x0fu);
            lo.y = d * mxfp4_value((v >> 8) & 0x0fu);
            lo.z = d * mxfp4_value((v >> 16) & 0x0fu);
            lo.w = d * mxfp4_value((v >> 24) & 0x0fu);
            hi.x = d * mxfp4_value((v >> 4) & 0x0fu);
            hi.y = d * mxfp4_value((v >> 12) & 0x0fu);
            hi.z = d * mxfp4_value((v >> 20) & 0x0fu);
            hi.w = d * mxfp4_value(v >> 28);
            float* o = dst + (t >> 2) * 32 + 4 * (int)(t & 3);
            *reinterpret_cast<float4*>(o) = lo;
            *reinterpret_cast<float4*>(o + 16) = hi;
        }
    }
}

// Q4_K with 16-byte aligned blocks: one thread takes one dword of a block's quants (four bytes = four weights of an even
// sub-block in the low nibbles and four of the odd sub-block after it in the high nibbles) and the block's 16-byte
// header: two loads, two 16-byte stores.  Eight neighbouring threads write 128 contiguous bytes of each sub-block.
// Same arithmetic as dequant4_q4_K (ManagedQuantizedOps.cs:447-479): (d * sc) * q - dmin * m.
__global__ void __launch_bounds__(256) dequant_q4k_wide_kernel(const uint8_t* __restrict__ src, float* __restrict__ dst, int64_t n8)
{
    const int64_t t0 = (int64_t)blockIdx.x * (256 * kWideItems) + threadIdx.x;
    uint4 hd[kWideItems];
    uint32_t qd[kWideItems];
#pragma unroll
    for (int u = 0; u < kWideItems; ++u) {
        const int64_t t = t0 + 256 * u;
        if (t < n8) {
            const uint8_t* blk = src + (t >> 5) * 144;
            hd[u] = *reinterpret_cast<const uint4*>(blk);
            qd[u] = *reinterpret_cast<const uint32_t*>(blk + 16 + 4 * (int)(t & 31));
        }
    }
#pragma unroll
    for (int u = 0; u < kWideItems; ++u) {
        const int64_t t = t0 + 256 * u;
        if (t >= n8) continue;
        const int64_t b = t >> 5;
        const int i = (int)(t & 31), g = i >> 3, l = (i & 7) * 4;
        const uint4 hdr = hd[u];
        const uint32_t q = qd[u];
        const float d = half_bits_to_float(hdr.x & 0xffffu), dmin = half_bits_to_float(hdr.x >> 16);
        // scales[12] = hdr.y, hdr.z, hdr.w; sub-blocks j = 2 g and 2 g + 1 (get_scale_min_k4, ggml-quants.c:703-710)
        uint32_t sc[2], mn[2];
#pragma unroll
        for (int k = 0; k < 2; ++k) {
            const int j = 2 * g + k;
            const uint32_t pj = ((j < 4 ? hdr.y : hdr.z) >> (8 * (j & 3))) & 0xffu;      // scales[j]
            const uint32_t pj4 = ((j < 4 ? hdr.z : hdr.w) >> (8 * (j & 3))) & 0xffu;     // scales[j + 4]
            const uint32_t pjm4 = (hdr.y >> (8 * (j & 3))) & 0xffu;                      // scales[j - 4], used for j >= 4
            sc[k] = j < 4 ? (pj & 63u) : ((pj4 & 0x0fu) | ((pjm4 >> 6) << 4));
            mn[k] = j < 4 ? (pj4 & 63u) : ((pj4 >> 4) | ((pj >> 6) << 4));
        }
        const float d1 = d * (float)sc[0], m1 = dmin * (float)mn[0];
        const float d2 = d * (float)sc[1], m2 = dmin * (float)mn[1];
        float4 lo, hi;
        lo.x = d1 * (float)(q & 0x0fu) - m1;
        lo.y = d1 * (float)((q >> 8) & 0x0fu) - m1;
        lo.z = d1 * (float)((q >> 16) & 0x0fu) - m1;
        lo.w = d1 * (float)((q >> 24) & 0x0fu) - m1;
        hi.x = d2 * (float)((q >> 4) & 0x0fu) - m2;
        hi.y = d2 * (float)((q >> 12) & 0x0fu) - m2;
        hi.z = d2 * (float)((q >> 20) & 0x0fu) - m2;
        hi.w = d2 * (float)(q >> 28) - m2;
        float* o = dst + b * 256 + 64 * g + l;
        *reinterpret_cast<float4*>(o) = lo;
        *reinterpret_cast<float4*>(o + 32) = hi;
    }
}

// dst[i, :] = dequantized row ids[i] of the weight; rows with an index outside [0, ne1) become zeros
template <int TYPE>
__global__ void __launch_bounds__(256) get_rows_kernel(const uint8_t* __restrict__ src, int64_t row_bytes, int64_t ne1,
                                                       const int32_t* __restrict__ ids, float* __restrict__ dst, int64_t ldd, int k4)
{
    const int t = (int)blockIdx.x * 256 + (int)threadIdx.x;
    if (t >= k4) return;
    const int64_t i = blockIdx.y;
    const int64_t row = ids[i];
    float4 o = float4{0.f, 0.f, 0.f, 0.f};
    if (row >= 0 && row < ne1) o = dequant4<TYPE>(src + row * row_bytes, (int64_t)t * 4);
    float* d = dst + i * ldd + (int64_t)t * 4;
    d[0] = o.x;
    d[1] = o.y;
    d[2] = o.z;
    d[3] = o.w;
}

}  // namespace

bool launch_dequant(int type, const void* src, int64_t n, float* dst, hipStream_t stream)
{
    if (n == 0) return true;
    const int64_t n4 = n / 4;  // block sizes are multiples of 4
    const int64_t blocks = (n4 + 255) / 256;
    if (blocks > 0x7fffffff) {
        set_last_error("dequantize: tensor too large for one launch.");
        return false;
    }
    const dim3 grid((unsigned)blocks), block(256);
    const uint8_t* s = static_cast<const uint8_t*>(src);
    switch (type) {
    case kTypeQ8_0:
    case kTypeMXFP4:
        if ((reinterpret_cast<uintptr_t>(dst) & 15) == 0) {
            const int64_t n8 = n / 8;
            const dim3 wide((unsigned)((n8 + 256 * kWideItems - 1) / (256 * kWideItems)));
            if (type == kTypeQ8_0) hipLaunchKernelGGL(dequant_q8_0_wide_kernel, wide, block, 0, stream, s, dst, n8);
            else hipLaunchKernelGGL(dequant_mxfp4_wide_kernel, wide, block, 0, stream, s, dst, n8);
        } else if (type == kTypeQ8_0) {
            hipLaunchKernelGGL(dequant_kernel<kTypeQ8_0>, grid, block, 0, stream, s, dst, n4);
        } else {
            hipLaunchKernelGGL(dequant_kernel<kTypeMXFP4>, grid, block, 0, stream, s, dst, n4);
        }
        break;
    case kTypeQ4_K:
        if ((reinterpret_cast<uintptr_t>(s) & 15) == 0 && (reinterpret_cast<uintptr_t>(dst) & 15) == 0) {
            const int64_t n8 = n / 8;
            hipLaunchKernelGGL(dequant_q4k_wide_kernel, dim3((unsigned)((n8 + 256 * kWideItems - 1) / (256 * kWideItems))), block, 0, stream, s, dst, n8);
        } else {
            hipLaunchKernelGGL(dequant_kernel<kTypeQ4_K>, grid, block, 0, stream, s, dst, n4);
        }
        break;
#define TSHIP_DEQUANT_CASE(T) case T: hipLaunchKernelGGL(dequant_kernel<T>, grid, block, 0, stream, s, dst, n4); break;
    TSHIP_DEQUANT_CASE(kTypeF16) TSHIP_DEQUANT_CASE(kTypeBF16) TSHIP_DEQUANT_CASE(kTypeQ4_0) TSHIP_DEQUANT_CASE(kTypeQ4_1)
    TSHIP_DEQUANT_CASE(kTypeQ5_0) TSHIP_DEQUANT_CASE(kTypeQ5_1) TSHIP_DEQUANT_CASE(kTypeQ5_K) TSHIP_DEQUANT_CASE(kTypeQ6_K)
    TSHIP_DEQUANT_CASE(kTypeIQ4_NL) TSHIP_DEQUANT_CASE(kTypeQ8_1)
#undef TSHIP_DEQUANT_CASE
    default: set_last_error("dequantize: unsupported type."); return false;
    }
    return hip_ok(hipGetLastError(), "dequantize launch");
}

// Embedding-style gather (ggml_get_rows on a quantized source, ggml_ops_matmul.cpp:519-668): n_ids rows of K
// floats.  type kTypeF32 copies fp32 rows.
bool launch_get_rows(int type, const void* src, int64_t row_bytes, int64_t ne1, const int32_t* ids, int64_t n_ids, int64_t K,
                     float* dst, int64_t ldd, hipStream_t stream)
{
    if (n_ids == 0 || K == 0) return true;
    if (n_ids > 65535) {
        set_last_error("get_rows: more than 65535 indices per call.");
        return false;
    }
    const int k4 = (int)(K / 4);
    const dim3 grid((unsigned)((k4 + 255) / 256), (unsigned)n_ids), block(256);
    const uint8_t* s = static_cast<const uint8_t*>(src);
    switch (type) {
    case kTypeF32: hipLaunchKernelGGL(get_rows_kernel<kTypeF32>, grid, block, 0, stream, s, row_bytes, ne1, ids, dst, ldd, k4); break;
    case kTypeQ8_0: hipLaunchKernelGGL(get_rows_kernel<kTypeQ8_0>, grid, block, 0, stream, s, row_bytes, ne1, ids, dst, ldd, k4); break;
    case kTypeQ4_K: hipLaunchKernelGGL(get_rows_kernel<kTypeQ4_K>, grid, block, 0, stream, s, row_bytes, ne1, ids, dst, ldd, k4); break;
    case kTypeMXFP4: hipLaunchKernelGGL(get_rows_kernel<kTypeMXFP4>, grid, block, 0, stream, s, row_bytes, ne1, ids, dst, ldd, k4); break;
#define TSHIP_ROWS_CASE(T) case T: hipLaunchKernelGGL(get_rows_kernel<T>, grid, block, 0, stream, s, row_bytes, ne1, ids, dst, ldd, k4); break;
    TSHIP_ROWS_CASE(kTypeF16) TSHIP_ROWS_CASE(kTypeBF16) TSHIP_ROWS_CASE(kTypeQ4_0) TSHIP_ROWS_CASE(kTypeQ4_1)
    TSHIP_ROWS_CASE(kTypeQ5_0) TSHIP_ROWS_CASE(kTypeQ5_1) TSHIP_ROWS_CASE(kTypeQ5_K) TSHIP_ROWS_CASE(kTypeQ6_K)
    TSHIP_ROWS_CASE(kTypeIQ4_NL) TSHIP_ROWS_CASE(kTypeQ8_1)
#undef TSHIP_ROWS_CASE
    default: set_last_error("get_rows: unsupported type."); return false;
    }
    return hip_ok(hipGetLastError(), "get_rows launch");
}

}  // namespace tship
