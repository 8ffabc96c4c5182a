// Bit-exact dequantization of raw GGUF blocks to fp32 on gfx950.
//
// The arithmetic is the managed dequantizers' (TensorSharp.Models/ManagedQuantizedOps.cs:411-427 Q8_0,
// :447-479 Q4_K, :579-598 MXFP4): every product is exact in fp32, the Q4_K subtract is the one rounding.
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

template <int TYPE>
__device__ __forceinline__ float4 dequant4(const uint8_t* src, int64_t e0)
{
    if (TYPE == kTypeQ8_0) return dequant4_q8_0(src, e0);
    if (TYPE == kTypeQ4_K) return dequant4_q4_K(src, e0);
    if (TYPE == kTypeMXFP4) return dequant4_mxfp4(src, e0);
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
    case kTypeQ8_0: hipLaunchKernelGGL(dequant_kernel<kTypeQ8_0>, grid, block, 0, stream, s, dst, n4); break;
    case kTypeQ4_K: hipLaunchKernelGGL(dequant_kernel<kTypeQ4_K>, grid, block, 0, stream, s, dst, n4); break;
    case kTypeMXFP4: hipLaunchKernelGGL(dequant_kernel<kTypeMXFP4>, grid, block, 0, stream, s, dst, n4); break;
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
    default: set_last_error("get_rows: unsupported type."); return false;
    }
    return hip_ok(hipGetLastError(), "get_rows launch");
}

}  // namespace tship
