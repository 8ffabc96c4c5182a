// Prefill GEMM  C[M x N] = X[M x K] * W[N x K]^T  over raw GGUF blocks (Q8_0 / Q4_K / MXFP4) on
// the gfx950 matrix cores.
//
//   1. convert_x_kernel: fp32 activations -> fp16, one power-of-two scale per row (so no input
//      magnitude overflows or underflows fp16), written in the k-order in which the weight
//      format unpacks (so the dequantizer never has to shuffle lanes), zero-padded to a
//      multiple of the k-tile.  Optionally gathers rows through an index (MoE).
//   2. gemm_slim_kernel (32 rows per tile: activations in registers, K split over the wavefronts, long K in
//      chunks; used up to a few hundred rows, see gemm_tile_m) and gemm_kernel (128 / 256 rows per tile):
//      BM x 256 x 64 tiles, eight wavefronts, each owning 32 output columns.  The fp16
//      activation k-tiles and the RAW quantized bytes of 256 weight rows (one 144-byte window per row
//      covering four k-tiles of Q4_K / MXFP4 or two of Q8_0) are copied from global memory straight
//      into LDS (buffer_load ... lds, range-checked), double-buffered.  Every lane unpacks its own
//      MFMA B operands from those raw bytes into registers with packed-fp16 VALU, one k-tile ahead
//      and in the shadow of the matrix pipe, so a weight is unpacked exactly once per tile and
//      dequantized weights never pass through LDS; A operands come from LDS one MFMA ahead.
//      v_mfma_f32_32x32x16_f16, fp32 accumulation, XCD-aware tile order, one barrier per k-tile.
//   3. epilogue: fp32 accumulators times the row scale -> C (optionally scattered through a row
//      index).
//
// Arithmetic: dequantised values follow ManagedQuantizedOps.cs:411-427 / :447-479 / :579-598 and
// are then rounded to fp16 operands (Q4_K: d*sc and dmin*m rounded to fp16 first); the contraction
// is TensorSharp.Models/ModelBase.cs:924-991 with fp32 accumulation on the matrix cores.
#include "tship_internal.h"

#include <algorithm>
#include <mutex>
#include <type_traits>

namespace tship {
namespace {

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef uint32_t uint4_t __attribute__((ext_vector_type(4)));

constexpr int kBK = 64;                 // k-tile
constexpr uint32_t kDeadOffset = 0x80000000u;

union H2U {
    uint32_t u;
    half2_t h;
};
__device__ __forceinline__ uint32_t pk_add(uint32_t a, uint32_t b)
{
    H2U x, y, r;
    x.u = a;
    y.u = b;
    r.h = x.h + y.h;
    return r.u;
}
__device__ __forceinline__ uint32_t pk_mul(uint32_t a, uint32_t b)
{
    H2U x, y, r;
    x.u = a;
    y.u = b;
    r.h = x.h * y.h;
    return r.u;
}
__device__ __forceinline__ uint32_t pk_fma(uint32_t a, uint32_t b, uint32_t c)
{
    H2U x, y, z, r;
    x.u = a;
    y.u = b;
    z.u = c;
    r.h = x.h * y.h + z.h;
    return r.u;
}
__device__ __forceinline__ uint32_t pack2(float a, float b)
{
    H2U r;
    r.h = half2_t{(_Float16)a, (_Float16)b};
    return r.u;
}
__device__ __forceinline__ uint32_t splat(float a) { return pack2(a, a); }

// Range of the fp16 weight operands.  A dequantised weight enters the matrix cores as an fp16 number, so a block scale
// near the ends of its own range would overflow fp16 or lose bits as an fp16 subnormal, where the reference
// (ManagedQuantizedOps.cs:411-598) is exact in fp32 for every scale.  Weights of trained models are far below one, so
// the operands carry the weight times 2^kWShift (the activations' row scale carries 2^-kWShift, see convert_x_kernel):
// the smallest fp16 scale (2^-24) then gives a normal fp16 operand, and only scales ABOVE a per-format limit
// (weights of magnitude about 32 and more; MXFP4: block exponents outside 94 .. 130) cannot be represented.  The
// unpackers keep a high-water mark of the scales they met in `bad` (out_of_range() reads it), and the kernels then
// store NaN in the columns such a block belongs to instead of a wrong number.
constexpr int kWShift = 10;
constexpr float kWUp = 1024.f;                   // 2^kWShift
constexpr uint32_t kWUp2 = 0x64006400u;          // the same as two fp16
constexpr uint32_t kNaNBits = 0x7fc00000u;
typedef uint16_t ushort2_t __attribute__((ext_vector_type(2)));
// high-water mark of the magnitude bits of two fp16 numbers (the order of the bits is the order of the magnitudes)
__device__ __forceinline__ void mark2(uint32_t& mark, uint32_t two_halfs)
{
    mark = __builtin_bit_cast(uint32_t, __builtin_elementwise_max(__builtin_bit_cast(ushort2_t, mark),
                                                                  __builtin_bit_cast(ushort2_t, two_halfs & 0x7fff7fffu)));
}
__device__ __forceinline__ bool over2(uint32_t mark, uint32_t limit_lo, uint32_t limit_hi)
{
    return (mark & 0xffffu) > limit_lo || (mark >> 16) > limit_hi;
}

// Position inside a k-tile at which activation k (0..63) is stored, per weight format.  MFMA k-step ks
// (0..3) takes positions [16 ks, 16 ks + 16): the first eight from the lanes with k-half h = 0, the
// next eight from h = 1, and element e of those eight pairs with element e of the lane's B operand,
// i.e. half (e & 1) of dword (4 ks + e / 2) in the order in which dequant() unpacks the raw bytes.
template <int TYPE>
__device__ __forceinline__ int k_slot(int k)
{
    if (TYPE == kTypeQ4_K) {      // also the order of Q5_K
        // sub-block k/32; quant byte c of the lane's 16-byte chunk; dword c/4 unpacks as (b0,b2),(b1,b3)
        const int sub = k >> 5, hh = (k >> 4) & 1, c = k & 15, b = c & 3;
        const int idx = sub * 8 + 2 * (c >> 2) + (b & 1);
        return (idx >> 2) * 16 + hh * 8 + 2 * (idx & 3) + (b >> 1);
    }
    if (TYPE == kTypeMXFP4) {     // also the order of Q4_0, Q4_1, Q5_0, Q5_1, IQ4_NL
        // block k/32; quant byte i = k%16 holds elements i (low nibble) and i + 16 (high nibble)
        const int hh = k >> 5, i = k & 15, hi = (k >> 4) & 1;
        return (i >> 2) * 16 + hh * 8 + 2 * (i & 3) + hi;
    }
    // Q8_0 and Q6_K: 32-element group k/32, natural order
    const int hh = k >> 5, tt = k & 31;
    return (tt >> 3) * 16 + hh * 8 + (tt & 7);
}

// ------------------------------------------------------------------------------------------
// activations: fp32 [M x K] (row stride ldx) -> fp16 [M x Kp] in unpack order, per-row scale
// ------------------------------------------------------------------------------------------
constexpr int kCvtHold = 8;      // float4 per thread kept in registers: rows up to THREADS * 32 elements are read once

// How a row of activations is formed while it is read.
struct ConvertSrc {
    const float* x;          // rows (kSrcSwiglu: gate | up rows of 2 K floats)
    int64_t ldx;
    const int* row_map;      // optional gather: source row of activation row m
    const float* norm_w;     // kSrcPlain: optional RMSNorm weight
    float eps;
    const float* bias;       // kSrcSwiglu: optional [experts x 2 K] bias, picked through expert_of
    const int* expert_of;
    float alpha, limit;
};
constexpr int kSrcPlain = 0, kSrcSwiglu = 1;

// SwiGLU of the gpt-oss experts (ggml-cpu/ops.cpp swiglu_oai: x = min(gate, limit), y = clamp(up, +-limit),
// x / (1 + exp(-alpha x)) * (y + 1))
__device__ __forceinline__ float swiglu_oai(float gate, float up, float alpha, float limit)
{
    const float x = fminf(gate, limit);
    const float y = fminf(fmaxf(up, -limit), limit);
    return x / (1.0f + expf(alpha * (-x))) * (y + 1.0f);
}

template <int TYPE, int THREADS, int SRC>
__global__ void __launch_bounds__(THREADS) convert_x_kernel(const ConvertSrc S, int K, int Kp, int ldo, _Float16* __restrict__ out,
                                                            float* __restrict__ scales)
{
    const int m = blockIdx.x;
    const int tid = threadIdx.x;
    const float* src = S.x + (int64_t)(S.row_map ? S.row_map[m] : m) * S.ldx;
    const float* norm_w = SRC == kSrcPlain ? S.norm_w : nullptr;
    const float* bias = (SRC == kSrcSwiglu && S.bias) ? S.bias + (int64_t)S.expert_of[m] * 2 * K : nullptr;
    __shared__ float red[THREADS / 64];
    __shared__ double redd[THREADS / 64];
    const int k4 = K >> 2;                       // K is a multiple of 32
    constexpr int kHeld = kCvtHold * THREADS * 4;
    // element k of the row as it enters the product (before the optional RMSNorm)
    auto raw4 = [&](int q) -> float4 {
        if (SRC == kSrcSwiglu) {
            float4 g = reinterpret_cast<const float4*>(src)[q], u = reinterpret_cast<const float4*>(src + K)[q];
            if (bias) {
                const float4 bg = reinterpret_cast<const float4*>(bias)[q], bu = reinterpret_cast<const float4*>(bias + K)[q];
                g = float4{g.x + bg.x, g.y + bg.y, g.z + bg.z, g.w + bg.w};
                u = float4{u.x + bu.x, u.y + bu.y, u.z + bu.z, u.w + bu.w};
            }
            return float4{swiglu_oai(g.x, u.x, S.alpha, S.limit), swiglu_oai(g.y, u.y, S.alpha, S.limit),
                          swiglu_oai(g.z, u.z, S.alpha, S.limit), swiglu_oai(g.w, u.w, S.alpha, S.limit)};
        }
        return reinterpret_cast<const float4*>(src)[q];
    };
    auto raw1 = [&](int k) -> float {
        if (SRC == kSrcSwiglu) return swiglu_oai(src[k] + (bias ? bias[k] : 0.f), src[K + k] + (bias ? bias[K + k] : 0.f), S.alpha, S.limit);
        return src[k];
    };
    auto held = [&](int i) -> int { return tid + i * THREADS; };      // which float4 of the row register i holds
    float4 hold[kCvtHold];
#pragma unroll
    for (int i = 0; i < kCvtHold; ++i) {
        const int q = held(i);
        hold[i] = q < k4 ? raw4(q) : float4{0.f, 0.f, 0.f, 0.f};
    }
    // optional RMSNorm prologue (ggml-cpu/ops.cpp:3646-3695: sum of squares in double, scale = 1/sqrtf(mean + eps),
    // then the multiply by the norm weight: (x * scale) * w)
    float rms = 1.f;
    if (norm_w) {
        double ss = 0.0;
#pragma unroll
        for (int i = 0; i < kCvtHold; ++i)
            ss += (double)(hold[i].x * hold[i].x) + (double)(hold[i].y * hold[i].y) + (double)(hold[i].z * hold[i].z) +
                  (double)(hold[i].w * hold[i].w);
        for (int k = kHeld + tid; k < K; k += THREADS) ss += (double)(src[k] * src[k]);
        for (int o = 32; o > 0; o >>= 1) ss += __shfl_xor(ss, o);
        if ((tid & 63) == 0) redd[tid >> 6] = ss;
        __syncthreads();
        double tot = 0.0;
#pragma unroll
        for (int i = 0; i < THREADS / 64; ++i) tot += redd[i];
        rms = 1.0f / sqrtf((float)(tot / (double)K) + S.eps);
#pragma unroll
        for (int i = 0; i < kCvtHold; ++i) {
            const int q = held(i);
            if (q < k4) {
                const float4 wv = reinterpret_cast<const float4*>(norm_w)[q];
                hold[i] = float4{(hold[i].x * rms) * wv.x, (hold[i].y * rms) * wv.y, (hold[i].z * rms) * wv.z, (hold[i].w * rms) * wv.w};
            }
        }
    }
    auto tail_value = [&](int k) { return norm_w ? (src[k] * rms) * norm_w[k] : raw1(k); };
    float amax = 0.f;
#pragma unroll
    for (int i = 0; i < kCvtHold; ++i)
        amax = fmaxf(amax, fmaxf(fmaxf(fabsf(hold[i].x), fabsf(hold[i].y)), fmaxf(fabsf(hold[i].z), fabsf(hold[i].w))));
    for (int k = kHeld + tid; k < K; k += THREADS) amax = fmaxf(amax, fabsf(tail_value(k)));
    for (int o = 32; o > 0; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o));
    if ((tid & 63) == 0) red[tid >> 6] = amax;
    __syncthreads();
    amax = 0.f;
#pragma unroll
    for (int i = 0; i < THREADS / 64; ++i) amax = fmaxf(amax, red[i]);
    // power-of-two scale bringing amax into [2^13, 2^14)
    int e = (int)((__float_as_uint(amax) >> 23) & 0xffu);
    if (e == 255) e = 127;
    if (e < 14) e = 14;
    const int se = e - 13;
    const float inv = __uint_as_float((uint32_t)(254 - se) << 23);
    // the weight operands carry 2^kWShift (see kWShift), the row scale takes it back
    if (tid == 0) scales[m] = __uint_as_float((uint32_t)se << 23) * (1.0f / kWUp);
    _Float16* dst = out + (int64_t)m * ldo;
    auto put = [&](int k, float v) { dst[(k & ~(kBK - 1)) | k_slot<TYPE>(k & (kBK - 1))] = (_Float16)(v * inv); };
    // Four consecutive activations land in one aligned 8-byte piece of the k-tile: in the K-quant order as
    // (x0, x2, x1, x3), in the natural order as they are, and in the split-nibble order interleaved with the four
    // activations 16 further on, which the lane four to the right (left) holds - the pair swaps them and each stores
    // one half of the 16 bytes.
#pragma unroll
    for (int i = 0; i < kCvtHold; ++i) {
        const int q = tid + i * THREADS;
        const float4 v = float4{hold[i].x * inv, hold[i].y * inv, hold[i].z * inv, hold[i].w * inv};
        uint2 o;
        int slot;
        if (TYPE == kTypeQ4_K) {
            o.x = pack2(v.x, v.z);
            o.y = pack2(v.y, v.w);
            slot = k_slot<TYPE>((4 * q) & (kBK - 1));
        } else if (TYPE == kTypeMXFP4) {
            // uniform trip count: lanes past the row take part in the exchange with zeros
            const float4 p = float4{__shfl_xor(v.x, 4), __shfl_xor(v.y, 4), __shfl_xor(v.z, 4), __shfl_xor(v.w, 4)};
            const bool upper = (q & 4) != 0;             // this lane holds the activations paired with high nibbles
            o.x = upper ? pack2(p.z, v.z) : pack2(v.x, p.x);
            o.y = upper ? pack2(p.w, v.w) : pack2(v.y, p.y);
            slot = k_slot<TYPE>((4 * (q & ~4)) & (kBK - 1)) + (upper ? 4 : 0);
        } else {
            o.x = pack2(v.x, v.y);
            o.y = pack2(v.z, v.w);
            slot = k_slot<TYPE>((4 * q) & (kBK - 1));
        }
        if (q < k4) *reinterpret_cast<uint2*>(dst + (((4 * q) & ~(kBK - 1)) | slot)) = o;
    }
    for (int k = kHeld + tid; k < K; k += THREADS) put(k, tail_value(k));
    for (int k = K + tid; k < Kp; k += THREADS) dst[(k & ~(kBK - 1)) | k_slot<TYPE>(k & (kBK - 1))] = (_Float16)0.f;
}

// ------------------------------------------------------------------------------------------
// activations for gemm_mx_kernel / gemm_slim_mx_kernel: fp32 [M x K] -> two block-scaled fp6 (E2M3) terms per
// activation, x = hi * 2^Eh + lo * 2^El with lo the same encoding of the rest x - hi * 2^Eh: what is left is below 2^-9
// of the block's largest magnitude.  The exponents are absolute (E8M0), so the row scale is one.
// A k-tile of a row is 128 bytes = 8 pieces of 16: term p (hi, lo) of block g keeps the first 16 bytes of its 24-byte
// stream of 32 six-bit fields in piece 3 p + 2 g and the last 8 in half g of piece 3 p + 1; piece 6 holds the scale
// bytes (hi, lo) of block g in the low bytes of dword g.  Field f of a stream pairs with nibble f of the weight block:
// element f / 2 (f even) or 16 + f / 2 (f odd) - the order in which v_cvt_scalef32_2xpk16_fp6_f32 packs its two
// sixteen-float sources, so a thread converts a whole block with one instruction per term (round to nearest even)
// and one more (v_cvt_scalef32_pk32_f32_fp6) for the values of the hi term that the rest is taken against.
// A workgroup takes kMxCvtBlocks consecutive blocks of one row: its threads read them float4 by float4 (coalesced),
// pass them through LDS (144 bytes per block: the 16-byte reads of sixteen threads cover the banks once) and each
// thread converts one block.
// ------------------------------------------------------------------------------------------
constexpr int kMxCvtBlocks = 128;
typedef float float16v_t __attribute__((ext_vector_type(16)));
typedef float float32v_t __attribute__((ext_vector_type(32)));
typedef uint32_t uint6_t __attribute__((ext_vector_type(6)));

// One block of 32 activations (a: elements 0 .. 15, b: 16 .. 31) as its two fp6 streams and their biased exponents.
// A block that is not live (past K inside the last k-tile) gives zero streams under a scale of one.
struct MxBlock {
    uint6_t hi, lo;
    int eh, el;
};
__device__ __forceinline__ MxBlock mx_encode_block(float16v_t a, float16v_t b, bool live)
{
    // Largest magnitude as an integer maximum of the bit patterns: an infinity or a NaN anywhere in the block comes out
    // on top.  Biased exponent E + 127 that brings it into (3.75, 7.5]; 127 for an empty block, 255 (NaN) for inf / NaN.
    auto top = [](const float16v_t& x, const float16v_t& y) -> uint32_t {
        uint32_t t = 0u;
#pragma unroll
        for (int i = 0; i < 16; ++i) t = max(t, max(__float_as_uint(x[i]) & 0x7fffffffu, __float_as_uint(y[i]) & 0x7fffffffu));
        return t;
    };
    auto block_exp = [](uint32_t u) -> int {
        const int ex = (int)(u >> 23);
        if (ex == 255) return 255;
        if (u == 0u) return 127;
        const int eb = ex - ((u & 0x7fffffu) > 0x700000u ? 1 : 2);      // a mantissa above 1.875 would round up to 8
        return eb < 1 ? 1 : eb;                                            // at most 253
    };
    auto pow2 = [](int biased) { return __uint_as_float((uint32_t)biased << 23); };      // biased 1 .. 254
    MxBlock r;
    r.eh = r.el = 127;
    r.hi = r.lo = uint6_t{0u, 0u, 0u, 0u, 0u, 0u};
    if (live) {
        r.eh = block_exp(top(a, b));
        if (r.eh != 255) {
            const float sc_h = pow2(r.eh);
            r.hi = __builtin_amdgcn_cvt_scalef32_2xpk16_fp6_f32(a, b, sc_h);
            const float32v_t back = __builtin_amdgcn_cvt_scalef32_pk32_f32_fp6(r.hi, sc_h);      // in field order
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                a[i] -= back[2 * i];
                b[i] -= back[2 * i + 1];
            }
            r.el = block_exp(top(a, b));
            r.lo = __builtin_amdgcn_cvt_scalef32_2xpk16_fp6_f32(a, b, pow2(r.el));
        }
    }
    return r;
}
// block g (0, 1) of the k-tile whose 128 bytes start at `tile`
__device__ __forceinline__ void mx_store_block(uint8_t* tile, int g, const MxBlock& r)
{
    *reinterpret_cast<uint4_t*>(tile + (2 * g) * 16) = uint4_t{r.hi[0], r.hi[1], r.hi[2], r.hi[3]};
    *reinterpret_cast<uint2*>(tile + 16 + 8 * g) = uint2{r.hi[4], r.hi[5]};
    *reinterpret_cast<uint4_t*>(tile + (3 + 2 * g) * 16) = uint4_t{r.lo[0], r.lo[1], r.lo[2], r.lo[3]};
    *reinterpret_cast<uint2*>(tile + 64 + 8 * g) = uint2{r.lo[4], r.lo[5]};
    *reinterpret_cast<uint32_t*>(tile + 96 + 4 * g) = (uint32_t)r.eh | ((uint32_t)r.el << 8);
}

template <int SRC>
__global__ void __launch_bounds__(kMxCvtBlocks) convert_x_mx_kernel(const ConvertSrc S, int K, int Kp, int ldo, int chunks,
                                                                     _Float16* __restrict__ out, float* __restrict__ scales)
{
    constexpr int T = kMxCvtBlocks;
    __shared__ float4 stage[T * 9];
    __shared__ double redd[T / 64];
    const int m = blockIdx.x / chunks, chunk = blockIdx.x - m * chunks;
    const int tid = threadIdx.x;
    const float* src = S.x + (int64_t)(S.row_map ? S.row_map[m] : m) * S.ldx;
    const float* norm_w = SRC == kSrcPlain ? S.norm_w : nullptr;
    const float* bias = (SRC == kSrcSwiglu && S.bias) ? S.bias + (int64_t)S.expert_of[m] * 2 * K : nullptr;
    const int k4 = K >> 2;                       // K is a multiple of 32
    if (chunk == 0 && tid == 0) scales[m] = 1.0f;
    // optional RMSNorm prologue (ggml-cpu/ops.cpp:3646-3695: sum of squares in double, scale = 1/sqrtf(mean + eps),
    // then the multiply by the norm weight: (x * scale) * w); every workgroup of the row sums the whole row
    float rms = 1.f;
    if (norm_w) {
        double ss = 0.0;
        for (int q = tid; q < k4; q += T) {
            const float4 v = reinterpret_cast<const float4*>(src)[q];
            ss += (double)(v.x * v.x) + (double)(v.y * v.y) + (double)(v.z * v.z) + (double)(v.w * v.w);
        }
        for (int o = 32; o > 0; o >>= 1) ss += __shfl_xor(ss, o);
        if ((tid & 63) == 0) redd[tid >> 6] = ss;
        __syncthreads();
        double tot = 0.0;
#pragma unroll
        for (int i = 0; i < T / 64; ++i) tot += redd[i];
        rms = 1.0f / sqrtf((float)(tot / (double)K) + S.eps);
    }
    const int q0 = chunk * T * 8;                // first float4 of the chunk
    // every load of the thread is issued before the first value is used: no branch between them (float4s past the row
    // read its last one and become zeros afterwards)
    float4 v[8], w[8];
    int qs[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) qs[j] = min(q0 + tid + j * T, k4 - 1);
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = reinterpret_cast<const float4*>(src)[qs[j]];
    if (SRC == kSrcSwiglu) {
#pragma unroll
        for (int j = 0; j < 8; ++j) w[j] = reinterpret_cast<const float4*>(src + K)[qs[j]];
        if (bias) {
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const float4 bg = reinterpret_cast<const float4*>(bias)[qs[j]], bu = reinterpret_cast<const float4*>(bias + K)[qs[j]];
                v[j] = float4{v[j].x + bg.x, v[j].y + bg.y, v[j].z + bg.z, v[j].w + bg.w};
                w[j] = float4{w[j].x + bu.x, w[j].y + bu.y, w[j].z + bu.z, w[j].w + bu.w};
            }
        }
#pragma unroll
        for (int j = 0; j < 8; ++j)
            v[j] = float4{swiglu_oai(v[j].x, w[j].x, S.alpha, S.limit), swiglu_oai(v[j].y, w[j].y, S.alpha, S.limit),
                          swiglu_oai(v[j].z, w[j].z, S.alpha, S.limit), swiglu_oai(v[j].w, w[j].w, S.alpha, S.limit)};
    } else if (norm_w) {
#pragma unroll
        for (int j = 0; j < 8; ++j) w[j] = reinterpret_cast<const float4*>(norm_w)[qs[j]];
#pragma unroll
        for (int j = 0; j < 8; ++j)
            v[j] = float4{(v[j].x * rms) * w[j].x, (v[j].y * rms) * w[j].y, (v[j].z * rms) * w[j].z, (v[j].w * rms) * w[j].w};
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const int ql = tid + j * T;
        stage[(ql >> 3) * 9 + (ql & 7)] = q0 + ql < k4 ? v[j] : float4{0.f, 0.f, 0.f, 0.f};
    }
    __syncthreads();
    const int blk = chunk * T + tid;             // this thread's block of the row
    const bool in_row = blk < (Kp >> 5);
    MxBlock r;
    if (in_row) {
        float16v_t a, b;                         // elements 0 .. 15 and 16 .. 31 of the block
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float4 va = stage[tid * 9 + j], vb = stage[tid * 9 + 4 + j];
            a[4 * j] = va.x, a[4 * j + 1] = va.y, a[4 * j + 2] = va.z, a[4 * j + 3] = va.w;
            b[4 * j] = vb.x, b[4 * j + 1] = vb.y, b[4 * j + 2] = vb.z, b[4 * j + 3] = vb.w;
        }
        r = mx_encode_block(a, b, blk < (K >> 5));      // blocks past K inside the last k-tile: zeros
    }
    // The k-tiles of the chunk are put together in LDS and leave as whole 16-byte pieces, thread after thread: stored
    // from the threads' own registers (4 .. 16 bytes each, 64 bytes apart) the same bytes took five times as long.
    __syncthreads();                             // every block has been read: the staging area takes the k-tiles
    uint8_t* const tiles = reinterpret_cast<uint8_t*>(stage);
    if (in_row) {
        mx_store_block(tiles + (tid >> 1) * 128, tid & 1, r);
        if (tid & 1) {                           // the bytes no kernel reads, as zeros
            *reinterpret_cast<uint2*>(tiles + (tid >> 1) * 128 + 104) = uint2{0u, 0u};
            *reinterpret_cast<uint4_t*>(tiles + (tid >> 1) * 128 + 112) = uint4_t{0u, 0u, 0u, 0u};
        }
    }
    __syncthreads();
    const int pieces = min(T / 2, (Kp >> 6) - chunk * (T / 2)) * 8;      // 16-byte pieces of this chunk's k-tiles
    uint4_t* const dst = reinterpret_cast<uint4_t*>(reinterpret_cast<uint8_t*>(out + (int64_t)m * ldo) + (int64_t)chunk * (T / 2) * 128);
#pragma unroll
    for (int j = 0; j < 4; ++j)
        if (tid + j * T < pieces) dst[tid + j * T] = reinterpret_cast<const uint4_t*>(tiles)[tid + j * T];
}

// ------------------------------------------------------------------------------------------
// weight formats: a "super-tile" is kSup consecutive k-tiles of one weight row, kept RAW in LDS as a window of
// kRawRow bytes (16-byte chunks copied from a 4-byte aligned address at or just below the first block).  `delta`
// is the distance from the window start to that first block.
//   fetch():   the raw dwords one lane needs for its (row, k-half) of k-tile t of the window
//   dequant(): those dwords -> 16 packed fp16 pairs, o[4 ks .. 4 ks + 3] being the lane's B operand
//              of MFMA k-step ks
//   sup_offset() / sup_delta(): where super-tile s starts (4-byte aligned) relative to the row's first window and
//              the delta inside that window; window_bytes() / tile_offset(): the same for windows of any number
//              of k-tiles (the register-resident kernel)
// ------------------------------------------------------------------------------------------
struct GQ4K {
    static constexpr int kRegs = 8;
    static constexpr int kSup = 4;            // one 256-element super-block
    static constexpr int kRawRow = 144;       // LDS bytes of one row's super-tile window
    static constexpr int kTileStep = 4;       // a wavefront's K range starts at a multiple of this many k-tiles
    static constexpr uint32_t sup_offset(int s) { return (uint32_t)s * 144u; }            // window start of super-tile s
    static __device__ __forceinline__ uint32_t sup_delta(uint32_t delta, int /*s*/) { return delta; }
    static constexpr int window_bytes(int ktw) { return ktw * 36; }                       // of ktw consecutive k-tiles
    static constexpr uint32_t tile_offset(int kt0) { return (uint32_t)kt0 * 36u; }        // kt0 a multiple of kTileStep
    static __device__ __forceinline__ void fetch(const uint8_t* rp, int t, int h, uint32_t /*delta*/, uint32_t (&r)[kRegs])
    {
        rp += (t >> 2) * 144;
        const int j = t & 3;
        const uint4_t hdr = *reinterpret_cast<const uint4_t*>(rp);
        const uint4_t q = *reinterpret_cast<const uint4_t*>(rp + 16 + j * 32 + h * 16);
        r[0] = hdr.x; r[1] = hdr.y; r[2] = hdr.z; r[3] = hdr.w;
        r[4] = q.x; r[5] = q.y; r[6] = q.z; r[7] = q.w;
    }
    // o[0..7]: low nibbles (sub-block 2j, elements 16h..16h+15), o[8..15]: high nibbles (sub-block 2j+1)
    static constexpr uint32_t kLimit = 0x2c00u;      // |d|, |dmin| <= 2^-4: 15 * 63 * d * 2^kWShift stays finite in fp16
    static __device__ __forceinline__ bool out_of_range(uint32_t mark) { return over2(mark, kLimit, kLimit); }
    // (blocks past the end of K or N arrive as zeros, whose scale is in range: `live` is not needed)
    static __device__ __forceinline__ void dequant(const uint32_t (&r)[kRegs], int j, int /*h*/, uint32_t /*delta*/, bool /*live*/,
                                                   uint32_t (&o)[16], uint32_t& bad)
    {
        const int sh = (j & 1) * 16;
        const uint32_t a = r[1] >> sh, b = r[2] >> sh, c = r[3] >> sh;
        const uint32_t sc_lo = a & 0x3f3fu, m_lo = b & 0x3f3fu;
        const uint32_t sc_hi = (c & 0x0f0fu) | ((a >> 2) & 0x3030u);
        const uint32_t m_hi = ((c >> 4) & 0x0f0fu) | ((b >> 2) & 0x3030u);
        const uint32_t sc = (j & 2) ? sc_hi : sc_lo, mn = (j & 2) ? m_hi : m_lo;
        H2U dm;
        dm.u = r[0];
        mark2(bad, r[0]);
        const float d = (float)dm.h.x, dmin = (float)dm.h.y * kWUp;
        const uint32_t s1 = splat(d * kWUp * (float)(sc & 0xffu)), o1 = splat(-(dmin * (float)(mn & 0xffu)));
        const uint32_t s2 = splat(d * (float)(sc >> 8) * (0.0625f * kWUp)), o2 = splat(-(dmin * (float)(mn >> 8)));
        const uint32_t magic = 0x64006400u, neg1024 = 0xe400e400u;   // 1024.0, -1024.0
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t q = r[4 + i], q8 = q >> 8;
            // 0x6400 | nibble = 1024 + q (low) or 1024 + 16 q (high): exact after subtracting 1024
            o[2 * i] = pk_fma(pk_add((q & 0x000f000fu) | magic, neg1024), s1, o1);
            o[2 * i + 1] = pk_fma(pk_add((q8 & 0x000f000fu) | magic, neg1024), s1, o1);
            o[8 + 2 * i] = pk_fma(pk_add((q & 0x00f000f0u) | magic, neg1024), s2, o2);
            o[8 + 2 * i + 1] = pk_fma(pk_add((q8 & 0x00f000f0u) | magic, neg1024), s2, o2);
        }
    }
};

struct GMXFP4 {
    static constexpr int kRegs = 5;
    static constexpr int kSup = 4;            // eight 17-byte blocks
    static constexpr int kRawRow = 144;
    static constexpr int kTileStep = 2;
    static constexpr uint32_t sup_offset(int s) { return (uint32_t)s * 136u; }
    static __device__ __forceinline__ uint32_t sup_delta(uint32_t delta, int /*s*/) { return delta; }
    static constexpr int window_bytes(int ktw) { return ktw * 34 + 3; }
    static constexpr uint32_t tile_offset(int kt0) { return (uint32_t)kt0 * 34u; }
    static __device__ __forceinline__ void fetch(const uint8_t* rp, int j, int h, uint32_t delta, uint32_t (&r)[kRegs])
    {
        const uint32_t off = delta + (uint32_t)(2 * j + h) * 17u;
        const uint32_t* p = reinterpret_cast<const uint32_t*>(rp + (off & ~3u));
#pragma unroll
        for (int i = 0; i < kRegs; ++i) r[i] = p[i];
    }
    template <int SEL>
    static __device__ __forceinline__ uint32_t cvt(uint32_t q, float scale)
    {
        H2U c;
        c.h = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(q, scale, SEL);
        return c.u;
    }
    // quant byte i of the block -> (element i, element i + 16); o[4 w + s] holds byte 4 w + s
    // block exponents the fp16 operand holds exactly: 0.5 * 2^(e - 127 + kWShift) >= 2^-24 and 6 * 2^(e - 127 + kWShift) < 2^16
    static constexpr uint32_t kMinE = 104 - kWShift, kMaxE = 140 - kWShift;
    // E2M1 * 2^(e - 127) (the doubled table of ggml-common.h:1094-1096 times 2^(e - 128)) times 2^kWShift as a scale operand
    static __device__ __forceinline__ float block_scale(uint32_t e, bool live, uint32_t& bad)
    {
        bad = max(bad, live ? e - kMinE : 0u);          // codes below the window wrap to large numbers
        return live ? __uint_as_float((e + kWShift) << 23) : 0.f;
    }
    static __device__ __forceinline__ bool out_of_range(uint32_t mark) { return mark > kMaxE - kMinE; }
    static __device__ __forceinline__ void dequant(const uint32_t (&r)[kRegs], int j, int h, uint32_t delta, bool live, uint32_t (&o)[16],
                                                   uint32_t& bad)
    {
        const uint32_t sft = (delta + (uint32_t)(2 * j + h) * 17u) & 3u;
        const uint32_t e = (r[0] >> (8 * sft)) & 0xffu;
        const bool wrap = sft == 3;
        const uint32_t b0 = wrap ? r[1] : r[0], b1 = wrap ? r[2] : r[1], b2 = wrap ? r[3] : r[2];
        const uint32_t b3 = wrap ? r[4] : r[3], b4 = r[4];
        const uint32_t shb = (sft + 1) & 3;
        const uint32_t q[4] = {__builtin_amdgcn_alignbyte(b1, b0, shb), __builtin_amdgcn_alignbyte(b2, b1, shb),
                               __builtin_amdgcn_alignbyte(b3, b2, shb), __builtin_amdgcn_alignbyte(b4, b3, shb)};
        // a block past the end of K contributes zeros
        const float scale = block_scale(e, live, bad);
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            o[4 * w] = cvt<0>(q[w], scale);
            o[4 * w + 1] = cvt<1>(q[w], scale);
            o[4 * w + 2] = cvt<2>(q[w], scale);
            o[4 * w + 3] = cvt<3>(q[w], scale);
        }
    }
};

struct GQ80 {
    static constexpr int kRegs = 9;
    static constexpr int kSup = 2;            // four 34-byte blocks
    static constexpr int kRawRow = 144;
    static constexpr int kTileStep = 2;
    static constexpr uint32_t sup_offset(int s) { return (uint32_t)s * 136u; }
    static __device__ __forceinline__ uint32_t sup_delta(uint32_t delta, int /*s*/) { return delta; }
    static constexpr int window_bytes(int ktw) { return ktw * 68 + 3; }
    static constexpr uint32_t tile_offset(int kt0) { return (uint32_t)kt0 * 68u; }
    static __device__ __forceinline__ void fetch(const uint8_t* rp, int j, int h, uint32_t delta, uint32_t (&r)[kRegs])
    {
        const uint32_t off = delta + (uint32_t)(2 * j + h) * 34u;
        const uint32_t* p = reinterpret_cast<const uint32_t*>(rp + (off & ~3u));
#pragma unroll
        for (int i = 0; i < kRegs; ++i) r[i] = p[i];
    }
    static constexpr uint32_t kLimit = 0x37ffu;      // |d| < 0.5: 128 * d * 2^kWShift stays finite in fp16
    static __device__ __forceinline__ bool out_of_range(uint32_t mark) { return over2(mark, kLimit, 0xffffu); }
    static __device__ __forceinline__ void dequant(const uint32_t (&r)[kRegs], int j, int h, uint32_t delta, bool live, uint32_t (&o)[16],
                                                   uint32_t& bad)
    {
        const bool odd = ((delta + (uint32_t)(2 * j + h) * 34u) & 2u) != 0;
        const uint32_t dbits = live ? (odd ? (r[0] >> 16) : (r[0] & 0xffffu)) : 0u;
        mark2(bad, dbits);
        const uint32_t d2 = pk_mul(dbits | (dbits << 16), kWUp2);     // fp16 d * 2^kWShift in both halves
        const uint32_t bias = 0xe480e480u;                              // -1152.0 = -(1024 + 128)
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint32_t q = (odd ? r[i + 1] : __builtin_amdgcn_alignbyte(r[i + 1], r[i], 2)) ^ 0x80808080u;
            // bytes u = q + 128 become fp16 1024 + u: (0x64, u) pairs picked with v_perm
            const uint32_t p0 = __builtin_amdgcn_perm(0x64646464u, q, 0x04010400u);   // (u0, u1)
            const uint32_t p1 = __builtin_amdgcn_perm(0x64646464u, q, 0x04030402u);   // (u2, u3)
            o[2 * i] = pk_mul(pk_add(p0, bias), d2);
            o[2 * i + 1] = pk_mul(pk_add(p1, bias), d2);
        }
    }
};

// Q6_K (ggml-common.h block_q6_K: ql[128], qh[64], int8 scales[16], fp16 d = 210 bytes, 2-byte aligned): k-tile
// t & 3 of a block takes, for k-half h, 32 quant bytes ql[64 (j / 2) + 32 h ..] (low nibbles for even j, high for
// odd), the two bits (2 (j & 1) + h) of qh[32 (j / 2) ..] and two scales.  Values d * scale * (q - 32)
// (ManagedQuantizedOps.cs:520-557) enter the matrix cores as fp16(d * scale) * (q - 32).  Blocks alternate
// between 4-byte aligned and 2 bytes off, so every piece is fetched as aligned dwords and shifted by 0 or 2 bytes.
struct GQ6K {
    static constexpr int kRegs = 20;
    static constexpr int kSup = 4;            // one 256-element block
    static constexpr int kRawRow = 240;       // 60 dwords: the dword reads of 32 rows spread over 16 banks (224 bytes: 8)
    static constexpr int kTileStep = 4;
    static constexpr uint32_t sup_offset(int s) { return ((uint32_t)s * 210u) & ~3u; }
    static __device__ __forceinline__ uint32_t sup_delta(uint32_t delta, int s) { return delta + ((uint32_t)(s & 1) << 1); }
    static constexpr int window_bytes(int ktw) { return ktw / 4 * 210 + 2; }
    static constexpr uint32_t tile_offset(int kt0) { return (uint32_t)(kt0 >> 2) * 210u; }
    static __device__ __forceinline__ void fetch(const uint8_t* rp, int t, int h, uint32_t delta, uint32_t (&r)[kRegs])
    {
        const uint32_t blk = delta + (uint32_t)(t >> 2) * 210u;        // block start inside the window (even)
        const int j = t & 3, nh = j >> 1;
        const uint32_t* a = reinterpret_cast<const uint32_t*>(rp + ((blk + 64u * nh + 32u * h) & ~3u));
        const uint32_t* b = reinterpret_cast<const uint32_t*>(rp + ((blk + 128u + 32u * nh) & ~3u));
#pragma unroll
        for (int i = 0; i < 9; ++i) {
            r[i] = a[i];
            r[9 + i] = b[i];
        }
        r[18] = *reinterpret_cast<const uint32_t*>(rp + ((blk + 192u + 8u * nh + 2u * (2 * (j & 1) + h)) & ~3u));
        r[19] = *reinterpret_cast<const uint32_t*>(rp + ((blk + 208u) & ~3u));
    }
    static constexpr uint32_t kLimit = 0x23ffu;      // |d| < 2^-6: 32 * 128 * d * 2^kWShift stays finite in fp16
    static __device__ __forceinline__ bool out_of_range(uint32_t mark) { return over2(mark, kLimit, 0xffffu); }
    static __device__ __forceinline__ void dequant(const uint32_t (&r)[kRegs], int t, int h, uint32_t delta, bool live, uint32_t (&o)[16],
                                                   uint32_t& bad)
    {
        const uint32_t blk = delta + (uint32_t)(t >> 2) * 210u;
        const int j = t & 3, g4 = 2 * (j & 1) + h;
        const uint32_t sh = (blk & 2u) ? 2u : 0u;                       // byte shift of the block's dwords
        const uint32_t ps = blk + 192u + 8u * (j >> 1) + 2u * g4;
        const uint32_t scw = r[18] >> ((ps & 2u) * 8u);
        const float sc0 = (float)(int)(int8_t)(scw & 0xffu), sc1 = (float)(int)(int8_t)((scw >> 8) & 0xffu);
        H2U dd;
        dd.u = live ? (r[19] >> ((blk & 2u) * 8u)) & 0xffffu : 0u;
        mark2(bad, dd.u);
        const float d = (float)dd.h.x * kWUp;
        const uint32_t s0 = splat(d * sc0), s1 = splat(d * sc1);
        const uint32_t bias = 0xe420e420u;                              // -(1024 + 32)
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint32_t ql = __builtin_amdgcn_alignbyte(r[i + 1], r[i], sh);
            const uint32_t qh = __builtin_amdgcn_alignbyte(r[10 + i], r[9 + i], sh);
            const uint32_t nib = ((j & 1) ? (ql >> 4) : ql) & 0x0f0f0f0fu;
            const uint32_t q6 = nib | (((qh >> (2 * g4)) & 0x03030303u) << 4);
            // bytes u = q become fp16 1024 + u: (0x64, u) pairs picked with v_perm; minus 1056 leaves q - 32 exactly
            const uint32_t p0 = __builtin_amdgcn_perm(0x64646464u, q6, 0x04010400u);
            const uint32_t p1 = __builtin_amdgcn_perm(0x64646464u, q6, 0x04030402u);
            const uint32_t sc = i < 4 ? s0 : s1;                         // elements 0..15 / 16..31 of the group
            o[2 * i] = pk_mul(pk_add(p0, bias), sc);
            o[2 * i + 1] = pk_mul(pk_add(p1, bias), sc);
        }
    }
};

// Q5_K (ggml-common.h block_q5_K: d, dmin, scales[12], qh[32], ql[128] = 176 bytes): Q4_K with a fifth bit per weight,
// bit 2j (low nibbles) / 2j + 1 (high nibbles) of qh[l] for the 64-weight group j (ManagedQuantizedOps.cs:481-518).
struct GQ5K {
    static constexpr int kRegs = 12;
    static constexpr int kSup = 4;
    static constexpr int kRawRow = 176;
    static constexpr int kTileStep = 4;
    static constexpr uint32_t sup_offset(int s) { return (uint32_t)s * 176u; }
    static __device__ __forceinline__ uint32_t sup_delta(uint32_t delta, int /*s*/) { return delta; }
    static constexpr int window_bytes(int ktw) { return ktw * 44; }
    static constexpr uint32_t tile_offset(int kt0) { return (uint32_t)kt0 * 44u; }
    static __device__ __forceinline__ void fetch(const uint8_t* rp, int t, int h, uint32_t /*delta*/, uint32_t (&r)[kRegs])
    {
        rp += (t >> 2) * 176;
        const int j = t & 3;
        const uint4_t hdr = *reinterpret_cast<const uint4_t*>(rp);
        const uint4_t qh = *reinterpret_cast<const uint4_t*>(rp + 16 + h * 16);
        const uint4_t q = *reinterpret_cast<const uint4_t*>(rp + 48 + j * 32 + h * 16);
        r[0] = hdr.x; r[1] = hdr.y; r[2] = hdr.z; r[3] = hdr.w;
        r[4] = q.x; r[5] = q.y; r[6] = q.z; r[7] = q.w;
        r[8] = qh.x; r[9] = qh.y; r[10] = qh.z; r[11] = qh.w;
    }
    static constexpr uint32_t kLimit = 0x2800u;      // |d|, |dmin| <= 2^-5: 31 * 63 * d * 2^kWShift stays finite in fp16
    static __device__ __forceinline__ bool out_of_range(uint32_t mark) { return over2(mark, kLimit, kLimit); }
    static __device__ __forceinline__ void dequant(const uint32_t (&r)[kRegs], int t, int /*h*/, uint32_t /*delta*/, bool /*live*/,
                                                   uint32_t (&o)[16], uint32_t& bad)
    {
        const int j = t & 3;
        const int sh = (j & 1) * 16;
        const uint32_t a = r[1] >> sh, b = r[2] >> sh, c = r[3] >> sh;
        const uint32_t sc_lo = a & 0x3f3fu, m_lo = b & 0x3f3fu;
        const uint32_t sc_hi = (c & 0x0f0fu) | ((a >> 2) & 0x3030u);
        const uint32_t m_hi = ((c >> 4) & 0x0f0fu) | ((b >> 2) & 0x3030u);
        const uint32_t sc = (j & 2) ? sc_hi : sc_lo, mn = (j & 2) ? m_hi : m_lo;
        H2U dm;
        dm.u = r[0];
        mark2(bad, r[0]);
        const float d = (float)dm.h.x * kWUp, dmin = (float)dm.h.y * kWUp;
        const uint32_t s1 = splat(d * (float)(sc & 0xffu)), o1 = splat(-(dmin * (float)(mn & 0xffu)));
        const uint32_t s2 = splat(d * (float)(sc >> 8) * 0.0625f), o2 = splat(-(dmin * (float)(mn >> 8)));
        const uint32_t magic = 0x64006400u, neg1024 = 0xe400e400u;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t q = r[4 + i], q8 = q >> 8;
            const uint32_t bl = r[8 + i] >> (2 * j), bh = r[8 + i] >> (2 * j + 1);    // fifth bits at bit 0 of every byte
            // low group: nibble + 16 bit; high group (kept as 16 * nibble): + 256 bit; both exact above 1024
            o[2 * i] = pk_fma(pk_add((q & 0x000f000fu) | ((bl & 0x00010001u) << 4) | magic, neg1024), s1, o1);
            o[2 * i + 1] = pk_fma(pk_add((q8 & 0x000f000fu) | (((bl >> 8) & 0x00010001u) << 4) | magic, neg1024), s1, o1);
            o[8 + 2 * i] = pk_fma(pk_add((q & 0x00f000f0u) | ((bh & 0x00010001u) << 8) | magic, neg1024), s2, o2);
            o[8 + 2 * i + 1] = pk_fma(pk_add((q8 & 0x00f000f0u) | (((bh >> 8) & 0x00010001u) << 8) | magic, neg1024), s2, o2);
        }
    }
};

// The 32-weight block formats with 16 quant bytes (low nibble = element j, high nibble = element j + 16) behind a
// header: Q4_0 (d), Q4_1 (d, m), Q5_0 (d, 32 fifth bits), Q5_1 (d, m, fifth bits), IQ4_NL (d, table lookup)
// (ManagedQuantizedOps.cs:313-409, :559-577).  Values enter the matrix cores as fp16(d) * q (+ fp16(m)).
template <int TYPE>
struct GLegacy {
    static constexpr int kHdr = TYPE == kTypeQ4_0 || TYPE == kTypeIQ4_NL ? 2 : TYPE == kTypeQ4_1 ? 4 : TYPE == kTypeQ5_0 ? 6 : 8;
    static constexpr int kBlock = kHdr + 16;
    static constexpr bool kMin = TYPE == kTypeQ4_1 || TYPE == kTypeQ5_1;
    static constexpr bool kFive = TYPE == kTypeQ5_0 || TYPE == kTypeQ5_1;
    static constexpr int kWords = (kBlock + 3) / 4;        // aligned dwords of one block
    static constexpr int kRegs = kWords + 1;
    static constexpr int kSup = 2;                          // four blocks
    static constexpr int kRawRow = 112;
    static constexpr int kTileStep = 2;
    static constexpr uint32_t sup_offset(int s) { return (uint32_t)s * (4u * kBlock); }
    static __device__ __forceinline__ uint32_t sup_delta(uint32_t delta, int /*s*/) { return delta; }
    static constexpr int window_bytes(int ktw) { return ktw * 2 * kBlock + 3; }
    static constexpr uint32_t tile_offset(int kt0) { return (uint32_t)kt0 * (2u * kBlock); }
    static __device__ __forceinline__ void fetch(const uint8_t* rp, int t, int h, uint32_t delta, uint32_t (&r)[kRegs])
    {
        const uint32_t off = delta + (uint32_t)(2 * t + h) * kBlock;
        const uint32_t* p = reinterpret_cast<const uint32_t*>(rp + (off & ~3u));
#pragma unroll
        for (int i = 0; i < kRegs; ++i) r[i] = p[i];
    }
    // |d| <= 4 (Q4_0: 8 d), 2 (Q4_1: 15 d + m; Q5_0: 16 d), 1 (Q5_1: 31 d + m), < 0.5 (IQ4_NL: 127 d) and |m| <= 32: the
    // value times 2^kWShift stays finite in fp16
    static constexpr uint32_t kLimitD = TYPE == kTypeQ4_0 ? 0x4400u : TYPE == kTypeQ5_1 ? 0x3c00u : TYPE == kTypeIQ4_NL ? 0x37ffu : 0x4000u;
    static constexpr uint32_t kLimitM = 0x5000u;
    static __device__ __forceinline__ bool out_of_range(uint32_t mark) { return over2(mark, kLimitD, kMin ? kLimitM : 0xffffu); }
    static __device__ __forceinline__ void dequant(const uint32_t (&r)[kRegs], int t, int h, uint32_t delta, bool live, uint32_t (&o)[16],
                                                   uint32_t& bad)
    {
        const uint32_t sft = (delta + (uint32_t)(2 * t + h) * kBlock) & 3u;
        uint32_t b[kWords];                                  // the block from its first byte
#pragma unroll
        for (int i = 0; i < kWords; ++i) b[i] = __builtin_amdgcn_alignbyte(r[i + 1], r[i], sft);
        const uint32_t dbits = live ? b[0] & 0xffffu : 0u;
        const uint32_t d2 = pk_mul(dbits | (dbits << 16), kWUp2);
        uint32_t m2 = 0u;
        if (kMin) {
            const uint32_t mbits = live ? b[0] >> 16 : 0u;
            mark2(bad, dbits | (mbits << 16));
            m2 = pk_mul(mbits | (mbits << 16), kWUp2);
        } else {
            mark2(bad, dbits);
        }
        uint32_t qh = 0u;
        if constexpr (kFive) qh = (kHdr & 3) ? __builtin_amdgcn_alignbyte(b[kHdr / 4], b[kHdr / 4 - 1], 2) : b[kHdr / 4 - 1];
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            // quant bytes 4 w .. 4 w + 3 of the block
            const uint32_t q = (kHdr & 3) ? __builtin_amdgcn_alignbyte(b[kHdr / 4 + w + 1], b[kHdr / 4 + w], 2) : b[kHdr / 4 + w];
            uint32_t lo = q & 0x0f0f0f0fu, hi = (q >> 4) & 0x0f0f0f0fu;
            if (kFive) {
                // bits 4 w .. 4 w + 3 (elements j) and 16 + 4 w .. (elements j + 16) of qh, one per byte, at bit 4
                lo |= ((((qh >> (4 * w)) & 0xfu) * 0x00204081u) & 0x01010101u) << 4;
                hi |= ((((qh >> (16 + 4 * w)) & 0xfu) * 0x00204081u) & 0x01010101u) << 4;
            }
            uint32_t bias;
            if (TYPE == kTypeIQ4_NL) {
                // {-127,-104,-83,-65,-49,-35,-22,-10, 1,13,25,38,53,69,89,113} + 128 as bytes, looked up with v_perm
                const uint32_t t0 = 0x3f2d1801u, t1 = 0x766a5d4fu, t2 = 0xa6998d81u, t3 = 0xf1d9c5b5u;
                const uint32_t ml = ((lo >> 3) & 0x01010101u) * 0xffu, mh = ((hi >> 3) & 0x01010101u) * 0xffu;
                const uint32_t sl = lo & 0x07070707u, shh = hi & 0x07070707u;
                lo = (__builtin_amdgcn_perm(t3, t2, sl) & ml) | (__builtin_amdgcn_perm(t1, t0, sl) & ~ml);
                hi = (__builtin_amdgcn_perm(t3, t2, shh) & mh) | (__builtin_amdgcn_perm(t1, t0, shh) & ~mh);
                bias = 0xe480e480u;                          // -(1024 + 128)
            } else {
                bias = kMin ? 0xe400e400u : kFive ? 0xe410e410u : 0xe408e408u;   // -1024, -(1024 + 16), -(1024 + 8)
            }
#pragma unroll
            for (int s2 = 0; s2 < 4; ++s2) {
                // (element 4 w + s2, element 4 w + s2 + 16) as fp16 1024 + value
                const uint32_t sel = (uint32_t)s2 | 0x0c00u | ((uint32_t)(4 + s2) << 16) | 0x0c000000u;
                const uint32_t pair = __builtin_amdgcn_perm(hi, lo, sel) | 0x64006400u;
                o[4 * w + s2] = pk_fma(pk_add(pair, bias), d2, m2);
            }
        }
    }
};

struct GemmArgs {
    const uint8_t* w;        // weight bytes (of expert 0 for grouped launches)
    int64_t w_bytes;         // bytes of one weight matrix (per expert for grouped launches)
    const _Float16* x16;     // [rows x Kp] converted activations
    int64_t x16_bytes;
    const float* xscale;     // [rows]
    float* c;                // result
    int64_t ldc;
    const int* c_rows;       // optional: result row index per activation row (scatter)
    int M, N, K, Kp;
    int xld;                 // halfs between activation rows of x16 (x_row_halfs)
    int m_tiles, n_tiles;
    // grouped (MoE) launches: m-tiles enumerated through this table
    const int* tile_expert;  // [m_tiles] expert id
    const int* tile_row0;    // [m_tiles] first activation row
    const int* tile_rows;    // [m_tiles] rows in the tile (<= BM)
    int64_t expert_stride;   // bytes between experts
    const int64_t* expert_off;  // optional [experts]: byte offset of each expert from w instead (experts held by pointer)
    int accumulate;          // c += ... instead of c = ...
    // register-resident kernel with K cut into chunks: chunk kc of a row tile writes its sums (already scaled) to
    // partial[kc][activation row][column]; a second kernel adds the chunks in order into c
    float* partial;          // null: one chunk, results go straight to c
    int k_chunks;
    int chunk_kt;            // k-tiles per chunk (8 wavefronts x KTW)
    int x_mx;                // the activations are MX fp6 pairs in gemm_mx_kernel's layout (convert_x_mx_kernel)
    // gemm_slim_mx_kernel<.., .., 1>: bias + SwiGLU-OAI of (gate, up) column pairs, written as MX activation rows
    const float* epi_bias;   // optional [experts x 2 F]
    float epi_alpha, epi_limit;
    uint8_t* epi_out;        // activation rows of the down projection (layout of convert_x_mx_kernel)
    int64_t epi_ld;          // bytes between them
};

// where the weights of m-tile mt's expert start, relative to A.w
__device__ __forceinline__ int64_t expert_offset(const GemmArgs& A, int mt)
{
    const int e = A.tile_expert[mt];
    return A.expert_off ? A.expert_off[e] : (int64_t)e * A.expert_stride;
}

constexpr int kXRow = kBK * 2;               // bytes of one activation row of a k-tile in LDS (no padding, swizzled)

// LDS-direct copy: 64 lanes x 16 bytes land at lds + 16 * lane; out-of-range offsets deliver zeros
__device__ __forceinline__ void copy16_to_lds(__amdgpu_buffer_rsrc_t rs, uint8_t* lds, uint32_t voffset, uint32_t soffset)
{
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (__attribute__((address_space(3))) void*)lds, 16, (int)voffset, (int)soffset, 0, 0);
}

// All but the N youngest LDS-direct copies of this wavefront have landed and its own LDS reads are done;
// then the workgroup barrier.  (A __syncthreads() would wait for every copy in flight.)
template <int N>
__device__ __forceinline__ void wait_copies_and_barrier()
{
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(N) : "memory");
}

// Epilogue of one wavefront: D[row = 32 i + 8 (r / 4) + 4 h + r % 4][column my_n] times the row scale.
// The scales (and scatter indices) of a 32-row block are loaded before its stores: the result may
// alias them as far as the compiler knows, so a load placed after a store would wait for it.
// Plain stores of a wavefront's TMW x NB blocks of 32 x 32 (no scatter, no accumulation).  Loads and stores share one
// counter that retires in order, so row scales loaded from global memory behind a block's stores would wait until those
// stores have been acknowledged, once per row block: the scales come from LDS (tile_scales[row of the tile], put there
// in the kernel's prologue) or are one (kUnitScale), and nothing stands between the stores.
template <int TMW, int NB, bool kUnitScale>
__device__ __forceinline__ void store_wave_tile(const float* tile_scales, const float16_t (&acc)[TMW][NB], float* cdst, int64_t ldc, int N,
                                                int m0, int m_rows, int row_first, int n_first, int h)
{
#pragma unroll
    for (int m = 0; m < TMW; ++m) {
        float sc[16];
#pragma unroll
        for (int r2 = 0; r2 < 16; ++r2) sc[r2] = kUnitScale ? 1.0f : tile_scales[row_first + m * 32 + 8 * (r2 >> 2) + 4 * h + (r2 & 3)];
#pragma unroll
        for (int n = 0; n < NB; ++n) {
            const int my_n = n_first + 32 * n;
            if (my_n >= N) continue;
#pragma unroll
            for (int r2 = 0; r2 < 16; ++r2) {
                const int ml = row_first + m * 32 + 8 * (r2 >> 2) + 4 * h + (r2 & 3);
                if (ml < m_rows) cdst[(int64_t)(m0 + ml) * ldc + my_n] = kUnitScale ? acc[m][n][r2] : acc[m][n][r2] * sc[r2];
            }
        }
    }
}

// A column whose weights held a scale outside the fp16 operand range (kWShift) is stored as NaN.
template <int TM>
__device__ __forceinline__ void poison_column(float16_t (&acc)[TM], bool flagged)
{
    // the two lanes of a column (k-halves) saw different blocks and hold different rows of it
    if (__builtin_amdgcn_ballot_w64(flagged) == 0) return;
    const int bad = (flagged ? 1 : 0) | __shfl_xor(flagged ? 1 : 0, 32);
    if (bad) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][r] = __uint_as_float(kNaNBits);
    }
}

template <int TM>
__device__ __forceinline__ void store_tile(const GemmArgs& A, const float16_t (&acc)[TM], int m0, int m_rows, int my_n, int h,
                                           const float* tile_scales)
{
    if (my_n >= A.N) return;
    if (!A.c_rows && !A.accumulate) {
        // plain stores with the row scales from LDS (tile_scales[row of the tile]): a scale loaded from global memory
        // behind a row block's stores would wait until they have been acknowledged (one counter tracks both)
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            float sc[16];
#pragma unroll
            for (int r = 0; r < 16; ++r) sc[r] = tile_scales[i * 32 + 8 * (r >> 2) + 4 * h + (r & 3)];
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int ml = i * 32 + 8 * (r >> 2) + 4 * h + (r & 3);
                if (ml < m_rows) A.c[(int64_t)(m0 + ml) * A.ldc + my_n] = acc[i][r] * sc[r];
            }
        }
        return;
    }
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        float sc[16], old[16];
        int64_t off[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int ml = i * 32 + 8 * (r >> 2) + 4 * h + (r & 3);
            const int m = m0 + min(ml, m_rows - 1);
            sc[r] = A.xscale[m];
            off[r] = (int64_t)(A.c_rows ? A.c_rows[m] : m) * A.ldc + my_n;
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) old[r] = A.accumulate ? A.c[off[r]] : 0.f;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int ml = i * 32 + 8 * (r >> 2) + 4 * h + (r & 3);
            if (ml < m_rows) A.c[off[r]] = A.accumulate ? old[r] + acc[i][r] * sc[r] : acc[i][r] * sc[r];
        }
    }
}

// Where the sums of K chunks go: a buffer of the caller (the kernels allocate nothing).  A launch whose chunk sums do
// not fit runs with whole K per tile, or fails when the kernel cannot do without chunks.  `need_out` set: nothing is
// launched, the launcher only reports how many bytes it would use.
struct ChunkScratch {
    float* ptr;
    size_t bytes;
    size_t* need_out;
};
inline float* chunk_scratch(const ChunkScratch& cs, size_t bytes) { return bytes <= cs.bytes ? cs.ptr : nullptr; }
__global__ void gemm_chunk_sum_kernel(const float* __restrict__ partial, int k_chunks, int M, int N, const int* __restrict__ c_rows,
                                      float* __restrict__ c, int64_t ldc, int accumulate);
bool launch_chunk_sum(const GemmArgs& a, hipStream_t stream);

// BM x 256 x 64 tiles, eight wavefronts, each owning all BM rows of 32 output columns.
//   * Activation k-tiles (fp16) and raw weight super-tiles go from global memory straight into LDS
//     (buffer_load ... lds, range-checked: rows past M or N arrive as zeros).  Activation rows are 128
//     bytes in LDS with the 16-byte chunk index XORed with (row / 2) % 8, which keeps the ds_read_b128 of
//     the A operands conflict-free without padding, so a k-tile is exactly BM / 8 copies.
//   * Activations run XST - 1 k-tiles ahead in XST LDS stages, weight super-tiles RL super-tiles ahead in
//     RL + 1 buffers.  Every wavefront issues the same number of copies per iteration (surplus copies use
//     an out-of-range source and a dump area), so the wait before the barrier is a vmcnt that leaves the
//     younger copies in flight (XST = 4 keeps three k-tiles of requests outstanding; the configurations in use
//     are double-buffered, XST = 2).
//   * A lane (column n, k-half h) unpacks ITS OWN B operands from the raw bytes into registers one
//     k-tile ahead, so dequantized weights never travel through LDS and every weight is unpacked by
//     exactly one lane of the workgroup.  One barrier per k-tile.
template <typename G, int BM, int XST, int NW>
__global__ void __launch_bounds__(NW * 64) gemm_kernel(const GemmArgs A)
{
    constexpr int BN = NW * 32;                          // output columns per tile
    constexpr int kRawRow = G::kRawRow, kRowChunks = kRawRow / 16;
    constexpr int RT = BN * kRawRow;                     // bytes of one raw super-tile in LDS
    constexpr int RIN = RT / 1024;                       // wavefront-wide 1 KiB copies per raw super-tile
    constexpr int WI = (RIN + NW - 1) / NW;              // per wavefront; the surplus goes to a dump area
    static_assert(RIN * 1024 == RT, "raw tile must be whole KiB");
    constexpr int TM = BM / 32;
    constexpr int D = XST - 1;                           // k-tiles of activation lookahead
    constexpr int RL = (D > 1 && G::kSup == 2) ? 2 : 1;  // weight lookahead in super-tiles
    constexpr int RB = RL + 1;
    constexpr int kXTile = BM * kXRow;
    constexpr int XI = kXTile / 1024 / NW;           // activation copies per wavefront and k-tile
    static_assert(XI >= 1 && XI * NW * 1024 == kXTile, "activation tile must split evenly over the wavefronts");
    static_assert(D == 1 || D == 3, "lookahead of one or three k-tiles");
    extern __shared__ uint8_t smem[];
    uint8_t* const xbuf = smem;                          // XST x kXTile
    uint8_t* const rbuf = smem + XST * kXTile;           // RB x RT
    uint8_t* const dump = rbuf + RB * RT;          // 1 KiB
    float* const tile_scales = reinterpret_cast<float*>(dump + 1024);      // BM row scales for the epilogue

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int col = lane & 31, h = lane >> 5;

    // XCD-aware tile order: workgroup ids go round-robin over the 8 XCDs, so each XCD gets a contiguous
    // run of tiles; consecutive tiles share the activation rows (same m-tile), which then stay in that
    // XCD's L2 while its CUs walk over the weight columns.
    // With K cut into chunks (few tiles, long K: the chunks fill the idle CUs) chunk kc of every tile is one unit.
    const int tiles = A.m_tiles * A.n_tiles;
    const int total = tiles * A.k_chunks;
    int t = blockIdx.x;
    {
        const int per = (total + 7) >> 3;
        const int xcd = t & 7, slot = t >> 3;
        t = xcd * per + slot;
        if (slot >= per || t >= total) return;
    }
    const int kc = t / tiles;
    t -= kc * tiles;
    const int mt = t / A.n_tiles, nt = t - mt * A.n_tiles;
    int m0, m_rows;
    const uint8_t* wbase = A.w;
    if (A.tile_expert) {
        m0 = A.tile_row0[mt];
        m_rows = A.tile_rows[mt];
        if (m_rows <= 0) return;          // table entries past the last tile
        wbase += expert_offset(A, mt);
    } else {
        m0 = mt * BM;
        m_rows = min(BM, A.M - m0);
    }
    const int n0 = nt * BN;

    const uintptr_t wa = reinterpret_cast<uintptr_t>(wbase);
    const uint32_t base_delta = (uint32_t)(wa & 3);
    const __amdgpu_buffer_rsrc_t wrs = __builtin_amdgcn_make_buffer_rsrc(
        reinterpret_cast<void*>(wa & ~(uintptr_t)3), 0, (int)(((uint32_t)A.w_bytes + base_delta + 3u) & ~3u), 0x00020000);
    const __amdgpu_buffer_rsrc_t xrs = __builtin_amdgcn_make_buffer_rsrc(const_cast<_Float16*>(A.x16), 0, (int)A.x16_bytes, 0x00020000);
    const uint32_t row_bytes = (uint32_t)((int64_t)A.w_bytes / A.N);
    const int kt_begin = kc * A.chunk_kt;                               // a multiple of 4: whole super-tiles and stage pairs
    const int nkt = min(A.Kp / kBK, kt_begin + A.chunk_kt);            // end of this unit's K range

    // per-lane source offsets of the LDS-direct copies (constant over the k loop)
    uint32_t x_off[XI], w_off[WI];
#pragma unroll
    for (int i = 0; i < XI; ++i) {
        const int q = (wave + NW * i) * 64 + lane;           // LDS chunk slot: row q / 8, position q % 8
        const int row = q >> 3, chunk = (q & 7) ^ ((row >> 1) & 7);
        x_off[i] = row < m_rows ? (uint32_t)(m0 + row) * (uint32_t)(A.xld * 2) + (uint32_t)chunk * 16u : kDeadOffset;
    }
#pragma unroll
    for (int i = 0; i < WI; ++i) {
        const int c = (wave + NW * i) * 64 + lane;
        const int row = c / kRowChunks, chunk = c - row * kRowChunks;
        w_off[i] = (row < BN && n0 + row < A.N) ? ((base_delta + (uint32_t)(n0 + row) * row_bytes) & ~3u) + (uint32_t)chunk * 16u
                                                  : kDeadOffset;
    }
    // this lane's weight row for the matrix pipe
    const int my_n = n0 + wave * 32 + col;
    const uint32_t my_delta = my_n < A.N ? (base_delta + (uint32_t)my_n * row_bytes) & 3u : 0u;
    const int my_raw = (wave * 32 + col) * kRawRow;

    // every call issues XI (activations) or WI (weights) copies from every wavefront
    auto issue_x = [&](int kt) {
        uint8_t* stage = xbuf + (kt % XST) * kXTile;
        const bool any = kt < nkt;
#pragma unroll
        for (int i = 0; i < XI; ++i) {
            copy16_to_lds(xrs, stage + (wave + NW * i) * 1024, any ? x_off[i] : kDeadOffset, (uint32_t)kt * kXRow);
        }
    };
    auto issue_w = [&](int s) {
        uint8_t* buf = rbuf + (s % RB) * RT;
        const bool any = s * G::kSup < nkt;
#pragma unroll
        for (int i = 0; i < WI; ++i) {
            const int id = wave + NW * i;
            copy16_to_lds(wrs, id < RIN ? buf + id * 1024 : dump, any ? w_off[i] : kDeadOffset, G::sup_offset(s));
        }
    };

    float16_t acc[TM];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][r] = 0.f;

    // A operand of k-step ks: chunk 2 ks + h of row (32 i + col), at its swizzled position
    const int sw = (col >> 1) & 7;
    int a_off[4];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) a_off[ks] = col * kXRow + ((2 * ks + h) ^ sw) * 16;

    int s = kt_begin / G::kSup, j = 0;              // super-tile and k-tile inside it of `kt`
    int xst = kt_begin % XST, rb = s % RB;          // LDS stage of k-tile kt, raw buffer of super-tile s
#pragma unroll
    for (int i = 0; i < RL; ++i) issue_w(s + i);
#pragma unroll
    for (int i = 0; i < D; ++i) issue_x(kt_begin + i);
    for (int i = threadIdx.x; i < BM; i += NW * 64) tile_scales[i] = A.xscale[m0 + min(i, m_rows - 1)];
    __syncthreads();
    uint32_t oc[16], on[16];
    uint32_t bad = 0u;                               // a scale of this lane's column does not fit the fp16 operands
    {
        uint32_t r[G::kRegs];
        G::fetch(rbuf + rb * RT + my_raw, 0, h, G::sup_delta(my_delta, s), r);
        G::dequant(r, 0, h, G::sup_delta(my_delta, s), (kt_begin * 2 + h) * 32 < A.K && my_n < A.N, oc, bad);
    }
    for (int kt = kt_begin; kt < nkt; ++kt) {
        if (j == 0) issue_w(s + RL);
        issue_x(kt + D);
        int jn = j + 1, sn = s, rbn = rb;
        if (jn == G::kSup) { jn = 0; sn = s + 1; rbn = rb + 1 == RB ? 0 : rb + 1; }
        // raw bytes of this lane's operands for k-tile kt + 1 (past the last k-tile: stale LDS, result unused)
        uint32_t r[G::kRegs];
        const uint32_t dn = G::sup_delta(my_delta, sn);
        G::fetch(rbuf + rbn * RT + my_raw, jn, h, dn, r);
        const uint8_t* xs = xbuf + xst * kXTile;
        {
            half8_t a[TM];
#pragma unroll
            for (int i = 0; i < TM; ++i) a[i] = *reinterpret_cast<const half8_t*>(xs + i * 32 * kXRow + a_off[0]);
            __builtin_amdgcn_sched_barrier(0);       // all LDS requests of the k-tile's first step go out before any use
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) {
                const uint4_t bb = {oc[4 * ks], oc[4 * ks + 1], oc[4 * ks + 2], oc[4 * ks + 3]};
                const half8_t b = __builtin_bit_cast(half8_t, bb);
#pragma unroll
                for (int i = 0; i < TM; ++i) {
                    acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[i], b, acc[i], 0, 0, 0);
                    if (ks + 1 < 4) a[i] = *reinterpret_cast<const half8_t*>(xs + i * 32 * kXRow + a_off[(ks + 1) & 3]);
                    // matrix and LDS instructions keep this order (each operand is requested TM - 1 MFMAs
                    // before its use); vector and scalar ALU work may move across
                    __builtin_amdgcn_sched_barrier(0x6);
                }
                // unpack the next k-tile's operands in the shadow of the matrix pipe
                // (past the unit's last k-tile the raw bytes are stale: nothing of them is used)
                if (ks == 0) G::dequant(r, jn, h, dn, kt + 1 < nkt && ((kt + 1) * 2 + h) * 32 < A.K && my_n < A.N, on, bad);
            }
        }
        // Copies that may stay in flight: the activations requested in the last D - 1 iterations and a
        // weight super-tile requested in one of them.
        if constexpr (D == 1) wait_copies_and_barrier<0>();
        else if constexpr (G::kSup == 2) wait_copies_and_barrier<2 * XI + WI>();
        else if (j < 2) wait_copies_and_barrier<2 * XI + WI>();
        else wait_copies_and_barrier<2 * XI>();
#pragma unroll
        for (int i = 0; i < 16; ++i) oc[i] = on[i];
        j = jn;
        s = sn;
        rb = rbn;
        xst = xst + 1 == XST ? 0 : xst + 1;
    }

    poison_column<TM>(acc, G::out_of_range(bad));
    if (A.partial) {
        // chunk sums: [kc][activation row][column], already scaled; a second kernel adds the chunks
        GemmArgs P = A;
        P.c = A.partial + (int64_t)kc * A.M * A.N;
        P.ldc = A.N;
        P.c_rows = nullptr;
        P.accumulate = 0;
        store_tile<TM>(P, acc, m0, m_rows, my_n, h, tile_scales);
    } else {
        store_tile<TM>(A, acc, m0, m_rows, my_n, h, tile_scales);
    }
}

// ------------------------------------------------------------------------------------------
// gemm_xw_kernel: BM x 256 x 64 tiles, eight wavefronts laid out 2 (rows) x 4 (columns); a wavefront owns BM / 2 rows of
// 64 output columns, so one A operand read from LDS feeds two matrix instructions and one B operand feeds BM / 64.
// Every weight of the tile is still unpacked exactly once: wavefront w unpacks columns [32 w, 32 w + 32) of the NEXT
// k-tile from the raw bytes in LDS and leaves the fp16 operands in an exchange area of LDS ([k-step][k-half][column],
// 16 bytes each: the layout in which the matrix instruction wants them, so both the write and the read are
// contiguous 16-byte pieces per lane), double-buffered; the k-tile's one barrier publishes them.
// Raw weights are copied per k-tile (P: which 16-byte pieces of a row belong to k-tile kt), two stages.
// ------------------------------------------------------------------------------------------
struct PQ4K {
    typedef GQ4K G;
    static constexpr int kParts = 3;                  // header + the k-tile's 32 quant bytes
    static constexpr int kRowBytes = 48;
    static __device__ __forceinline__ uint32_t part_base(int part) { return part == 0 ? 0u : 16u * (uint32_t)part; }
    static __device__ __forceinline__ uint32_t part_step(int part) { return part == 0 ? 0u : 32u; }   // times kt % 4
    static __device__ __forceinline__ uint32_t soffset(int kt) { return (uint32_t)(kt >> 2) * 144u; }
    static __device__ __forceinline__ int phase(int kt) { return kt & 3; }
    // rows are 16-byte aligned: the copied window starts at the row, nothing to re-align
    static constexpr bool kAligned = true;
    static __device__ __forceinline__ uint32_t row_window(uint32_t row_start) { return row_start; }
    static __device__ __forceinline__ uint32_t row_delta(uint32_t /*row_start*/) { return 0u; }
    static __device__ __forceinline__ uint32_t delta(uint32_t /*d0*/, int /*kt*/) { return 0u; }
    static __device__ __forceinline__ void fetch(const uint8_t* rp, int h, uint32_t /*delta*/, uint32_t (&r)[G::kRegs])
    {
        const uint4_t hdr = *reinterpret_cast<const uint4_t*>(rp);
        const uint4_t q = *reinterpret_cast<const uint4_t*>(rp + 16 + h * 16);
        r[0] = hdr.x; r[1] = hdr.y; r[2] = hdr.z; r[3] = hdr.w;
        r[4] = q.x; r[5] = q.y; r[6] = q.z; r[7] = q.w;
    }
    // The unpacking of one lane's 32 weights of a k-tile (GQ4K::dequant) cut into kMicro small steps that the kernel
    // places one by one behind its matrix instructions; step I may use what steps < I left in `st` and `o`.
    // Quarter q of `o` (o[4 q .. 4 q + 3], the B operand of k-step q) is complete after step kReady[q].
    static constexpr int kMicro = 17;
    static constexpr int kFirstHalf = 11;             // steps after which quarters 0 and 2 are complete
    struct State {
        uint32_t a, b, c, sc, mn, s1, o1, s2, o2, q8;
        float dmin;                                   // times 2^kWShift
    };
    // constants kept in registers so that mask-and-merge is one instruction (v_and_or_b32 takes one literal at most)
    struct Consts {
        uint32_t magic, lo_mask, hi_mask, neg1024;
        __device__ __forceinline__ Consts() : magic(0x64006400u), lo_mask(0x000f000fu), hi_mask(0x00f000f0u), neg1024(0xe400e400u)
        {
            asm volatile("" : "+v"(magic));
            asm volatile("" : "+s"(lo_mask), "+s"(hi_mask), "+s"(neg1024));
        }
    };
    static __device__ __forceinline__ int ready_after(int quarter) { return quarter == 0 ? 10 : quarter == 2 ? 10 : 16; }
    template <int I>
    static __device__ __forceinline__ void micro(State& st, const uint32_t (&r)[G::kRegs], int j, int /*h*/, uint32_t /*delta*/, bool /*live*/,
                                                 const Consts& K, uint32_t (&o)[16], uint32_t& bad)
    {
        if constexpr (I == 0) {
            const int sh = (j & 1) * 16;
            st.a = r[1] >> sh;
            st.b = r[2] >> sh;
            st.c = r[3] >> sh;
            mark2(bad, r[0]);
        } else if constexpr (I == 1) {
            const uint32_t sc_lo = st.a & 0x3f3fu, sc_hi = (st.c & 0x0f0fu) | ((st.a >> 2) & 0x3030u);
            st.sc = (j & 2) ? sc_hi : sc_lo;
        } else if constexpr (I == 2) {
            const uint32_t m_lo = st.b & 0x3f3fu, m_hi = ((st.c >> 4) & 0x0f0fu) | ((st.b >> 2) & 0x3030u);
            st.mn = (j & 2) ? m_hi : m_lo;
        } else if constexpr (I == 3) {
            H2U dm;
            dm.u = r[0];
            const float d = (float)dm.h.x * kWUp, dmin = (float)dm.h.y * kWUp;
            st.s1 = splat(d * (float)(st.sc & 0xffu));
            st.o1 = splat(-(dmin * (float)(st.mn & 0xffu)));
            st.dmin = dmin;
        } else if constexpr (I == 4) {
            H2U dm;
            dm.u = r[0];
            const float d = (float)dm.h.x;
            st.s2 = splat(d * (float)(st.sc >> 8) * (0.0625f * kWUp));
            st.o2 = splat(-(st.dmin * (float)(st.mn >> 8)));
        } else {
            // raw dword i in three steps: both low nibble pairs; high pair of bytes 0, 2; high pair of bytes 1, 3
            constexpr int i = (I - 5) / 3, part = (I - 5) % 3;
            const uint32_t q = r[4 + i];
            if constexpr (part == 0) {
                st.q8 = q >> 8;
                o[2 * i] = pk_fma(pk_add((q & K.lo_mask) | K.magic, K.neg1024), st.s1, st.o1);
                o[2 * i + 1] = pk_fma(pk_add((st.q8 & K.lo_mask) | K.magic, K.neg1024), st.s1, st.o1);
            } else if constexpr (part == 1) {
                o[8 + 2 * i] = pk_fma(pk_add((q & K.hi_mask) | K.magic, K.neg1024), st.s2, st.o2);
            } else {
                o[8 + 2 * i + 1] = pk_fma(pk_add((st.q8 & K.hi_mask) | K.magic, K.neg1024), st.s2, st.o2);
            }
        }
    }
};

// MXFP4: a k-tile is two 17-byte blocks = 34 bytes of a row that is only byte aligned.  The copied window is the 48 bytes
// from (row start & ~3) + (34 kt & ~3): the blocks then begin 0 .. 5 bytes into it (the row's own misalignment plus the two
// bytes every odd k-tile adds), which GMXFP4's unpacker takes as its byte shift.
struct PMXFP4 {
    typedef GMXFP4 G;
    static constexpr int kParts = 3;
    static constexpr int kRowBytes = 48;
    static __device__ __forceinline__ uint32_t part_base(int part) { return 16u * (uint32_t)part; }
    static __device__ __forceinline__ uint32_t part_step(int /*part*/) { return 0u; }
    static __device__ __forceinline__ uint32_t soffset(int kt) { return ((uint32_t)kt * 34u) & ~3u; }
    static __device__ __forceinline__ int phase(int /*kt*/) { return 0; }
    static constexpr bool kAligned = false;
    static __device__ __forceinline__ uint32_t row_window(uint32_t row_start) { return row_start & ~3u; }
    static __device__ __forceinline__ uint32_t row_delta(uint32_t row_start) { return row_start & 3u; }
    static __device__ __forceinline__ uint32_t delta(uint32_t d0, int kt) { return d0 + (((uint32_t)kt & 1u) << 1); }
    static __device__ __forceinline__ void fetch(const uint8_t* rp, int h, uint32_t delta, uint32_t (&r)[G::kRegs])
    {
        G::fetch(rp, 0, h, delta, r);
    }
    // align + scale; bytes 0-3; bytes 8-11 (quarters 0 and 2 complete); bytes 4-7; bytes 12-15
    static constexpr int kMicro = 5;
    static constexpr int kFirstHalf = 3;
    struct State {
        uint32_t q[4];
        float scale;
    };
    struct Consts {};
    template <int I>
    static __device__ __forceinline__ void micro(State& st, const uint32_t (&r)[G::kRegs], int /*j*/, int h, uint32_t delta, bool live,
                                                 const Consts&, uint32_t (&o)[16], uint32_t& bad)
    {
        if constexpr (I == 0) {
            // the re-alignment of GMXFP4::dequant for block h of the window
            const uint32_t sft = (delta + (uint32_t)h * 17u) & 3u;
            const uint32_t e = (r[0] >> (8 * sft)) & 0xffu;
            const bool wrap = sft == 3;
            const uint32_t b0 = wrap ? r[1] : r[0], b1 = wrap ? r[2] : r[1], b2 = wrap ? r[3] : r[2];
            const uint32_t b3 = wrap ? r[4] : r[3], b4 = r[4];
            const uint32_t shb = (sft + 1) & 3;
            st.q[0] = __builtin_amdgcn_alignbyte(b1, b0, shb);
            st.q[1] = __builtin_amdgcn_alignbyte(b2, b1, shb);
            st.q[2] = __builtin_amdgcn_alignbyte(b3, b2, shb);
            st.q[3] = __builtin_amdgcn_alignbyte(b4, b3, shb);
            st.scale = G::block_scale(e, live, bad);
        } else {
            constexpr int w = I == 1 ? 0 : I == 2 ? 2 : I == 3 ? 1 : 3;
            o[4 * w] = G::template cvt<0>(st.q[w], st.scale);
            o[4 * w + 1] = G::template cvt<1>(st.q[w], st.scale);
            o[4 * w + 2] = G::template cvt<2>(st.q[w], st.scale);
            o[4 * w + 3] = G::template cvt<3>(st.q[w], st.scale);
        }
    }
};

template <typename P, int BM, int WN>
__global__ void __launch_bounds__(128 * WN) gemm_xw_kernel(const GemmArgs A)
{
    typedef typename P::G G;
    constexpr int BN = 256;
    constexpr int NW = 2 * WN;                            // wavefronts: 2 (rows) x WN (columns)
    constexpr int TMW = BM / 64;                          // 32-row blocks of a wavefront (its BM / 2 rows)
    constexpr int NB = BN / (32 * WN);                    // 32-column blocks of a wavefront
    constexpr int DUTY = BN / 32 / NW;                    // 32-column blocks a wavefront unpacks per k-tile
    constexpr int kXTile = BM * kXRow;
    constexpr int XI = kXTile / 1024 / NW;                // activation copies per wavefront and k-tile
    constexpr int kRawTile = BN * P::kRowBytes;
    constexpr int kRawCopies = kRawTile / 1024;
    constexpr int RI = (kRawCopies + NW - 1) / NW;        // raw copies per wavefront and k-tile; the surplus goes to a dump area
    constexpr int kBTile = 4 * 2 * BN * 16;               // exchange area of one k-tile
    static_assert(kRawCopies * 1024 == kRawTile && XI >= 1 && XI * NW * 1024 == kXTile, "tile pieces must be whole KiB");
    extern __shared__ uint8_t smem[];
    constexpr int ST = 2;                                 // copy stages of the activations and of the raw rows
    uint8_t* const xbuf = smem;                           // ST x kXTile
    uint8_t* const rraw = xbuf + ST * kXTile;             // ST x kRawTile
    uint8_t* const bex = rraw + ST * kRawTile;            // 2 x kBTile
    uint8_t* const dump = bex + 2 * kBTile;               // 1 KiB
    float* const tile_scales = reinterpret_cast<float*>(dump + 1024);      // BM row scales for the epilogue
    uint32_t* const col_bad = reinterpret_cast<uint32_t*>(tile_scales + BM);   // BN flags: a scale of the column left the operand range

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WN, wn = wave % WN;
    const int col = lane & 31, h = lane >> 5;

    const int tiles = A.m_tiles * A.n_tiles;
    const int total = tiles * A.k_chunks;
    int t = blockIdx.x;
    {
        const int per = (total + 7) >> 3;
        const int xcd = t & 7, slot = t >> 3;
        t = xcd * per + slot;
        if (slot >= per || t >= total) return;
    }
    const int kc = t / tiles;
    t -= kc * tiles;
    const int mt = t / A.n_tiles, nt = t - mt * A.n_tiles;
    int m0, m_rows;
    const uint8_t* wbase = A.w;
    if (A.tile_expert) {
        m0 = A.tile_row0[mt];
        m_rows = A.tile_rows[mt];
        if (m_rows <= 0) return;
        wbase += expert_offset(A, mt);
    } else {
        m0 = mt * BM;
        m_rows = min(BM, A.M - m0);
    }
    const int n0 = nt * BN;

    // byte-aligned formats: the resource starts at the dword below the weight, offsets carry the difference
    const uintptr_t wa = reinterpret_cast<uintptr_t>(wbase);
    const uint32_t base_delta = P::kAligned ? 0u : (uint32_t)(wa & 3);
    const __amdgpu_buffer_rsrc_t wrs = __builtin_amdgcn_make_buffer_rsrc(
        reinterpret_cast<void*>(wa - base_delta), 0, (int)(((uint32_t)A.w_bytes + base_delta + 3u) & ~3u), 0x00020000);
    const __amdgpu_buffer_rsrc_t xrs = __builtin_amdgcn_make_buffer_rsrc(const_cast<_Float16*>(A.x16), 0, (int)A.x16_bytes, 0x00020000);
    const uint32_t row_bytes = (uint32_t)((int64_t)A.w_bytes / A.N);
    const int kt_begin = kc * A.chunk_kt;
    const int nkt = min(A.Kp / kBK, kt_begin + A.chunk_kt);

    uint32_t x_off[XI], r_off[RI], r_step[RI];
#pragma unroll
    for (int i = 0; i < XI; ++i) {
        const int q = (wave + NW * i) * 64 + lane;
        const int row = q >> 3, chunk = (q & 7) ^ ((row >> 1) & 7);
        x_off[i] = row < m_rows ? (uint32_t)(m0 + row) * (uint32_t)(A.xld * 2) + (uint32_t)chunk * 16u : kDeadOffset;
    }
#pragma unroll
    for (int i = 0; i < RI; ++i) {
        const int q = (wave + NW * i) * 64 + lane;                // 16-byte piece of the raw tile
        const int row = q / P::kParts, part = q - row * P::kParts;
        const bool ok = q < BN * P::kParts && n0 + row < A.N;
        r_off[i] = ok ? P::row_window(base_delta + (uint32_t)(n0 + row) * row_bytes) + P::part_base(part) : kDeadOffset;
        r_step[i] = ok ? P::part_step(part) : 0u;
    }
    // k-tiles past the end: the offset gets its top bit set (out of range: zeros arrive) by data flow, not by a
    // branch, so that the loop body stays one scheduling region
    auto issue_x1 = [&](int kt, int i) {
        const uint32_t past = kt < nkt ? 0u : kDeadOffset;
        copy16_to_lds(xrs, xbuf + (kt & (ST - 1)) * kXTile + (wave + NW * i) * 1024, x_off[i] | past, (uint32_t)kt * kXRow);
    };
    auto issue_raw1 = [&](int kt, int i) {
        const uint32_t past = kt < nkt ? 0u : kDeadOffset;
        const int id = wave + NW * i;
        copy16_to_lds(wrs, id < kRawCopies ? rraw + (kt & (ST - 1)) * kRawTile + id * 1024 : dump,
                      (r_off[i] + r_step[i] * (uint32_t)P::phase(kt)) | past, P::soffset(kt));
    };

    float16_t acc[TMW][NB];
#pragma unroll
    for (int m = 0; m < TMW; ++m)
#pragma unroll
        for (int n = 0; n < NB; ++n)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[m][n][r] = 0.f;

    // LDS addresses of this lane: A operand of k-step ks = 16-byte piece 2 ks + h of row (wm BM/2 + 32 m + col), swizzled;
    // B operand of k-step ks, column block n = piece ((2 ks + h) 256 + 32 NB wn + 32 n + col) of the exchange area
    const int sw = (col >> 1) & 7;
    int a_off[4];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) a_off[ks] = (wm * (BM / 2) + col) * kXRow + ((2 * ks + h) ^ sw) * 16;
    const int b_rd = (h * BN + 32 * NB * wn + col) * 16;
    const int b_wr = (h * BN + 32 * DUTY * wave + col) * 16;
    const int my_raw = (32 * DUTY * wave + col) * P::kRowBytes;
    uint32_t my_d0[DUTY];                                 // byte position of this lane's rows inside their copied windows
#pragma unroll
    for (int u = 0; u < DUTY; ++u) my_d0[u] = P::row_delta(base_delta + (uint32_t)(n0 + 32 * DUTY * wave + 32 * u + col) * row_bytes);
    auto load_ops = [&](int kt, int ks, half8_t (&a)[TMW], half8_t (&b)[NB]) {
        const uint8_t* xs = xbuf + (kt & (ST - 1)) * kXTile;
        const uint8_t* bs = bex + (kt & 1) * kBTile;
#pragma unroll
        for (int m = 0; m < TMW; ++m) a[m] = *reinterpret_cast<const half8_t*>(xs + m * 32 * kXRow + a_off[ks]);
#pragma unroll
        for (int n = 0; n < NB; ++n) b[n] = *reinterpret_cast<const half8_t*>(bs + b_rd + ks * (2 * BN * 16) + n * 32 * 16);
    };

    // The loop is rotated around the k-tile's barrier, which sits between k-steps 2 and 3: by then every operand of the
    // k-tile is in registers, so behind the barrier the stage can take the copy of the k-tile after next, the first
    // operands of the next k-tile are read and its raw bytes fetched while k-step 3 still feeds the matrix pipe.
    //   state behind barrier(kt - 1): activations of k-tile kt and raw bytes of kt + 1 have landed, the exchange area of
    //   kt is complete
#pragma unroll
    for (int i = 0; i < RI; ++i) issue_raw1(kt_begin, i);
#pragma unroll
    for (int i = 0; i < XI; ++i) issue_x1(kt_begin, i);
#pragma unroll
    for (int i = 0; i < RI; ++i) issue_raw1(kt_begin + 1, i);
    if (tid < BM) tile_scales[tid] = A.xscale[m0 + min(tid, m_rows - 1)];
    __syncthreads();
    uint32_t bad[DUTY];                                   // per 32-column block this lane unpacks
    bool in_n[DUTY];
#pragma unroll
    for (int u = 0; u < DUTY; ++u) {
        bad[u] = 0u;
        in_n[u] = n0 + 32 * DUTY * wave + 32 * u + col < A.N;
    }
#pragma unroll
    for (int u = 0; u < DUTY; ++u) {
        uint32_t r0[G::kRegs], o0[16];
        P::fetch(rraw + (kt_begin & (ST - 1)) * kRawTile + my_raw + u * 32 * P::kRowBytes, h, P::delta(my_d0[u], kt_begin), r0);
        G::dequant(r0, P::phase(kt_begin), h, P::delta(my_d0[u], kt_begin), (kt_begin * 2 + h) * 32 < A.K && in_n[u], o0, bad[u]);
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            const uint4_t v = {o0[4 * ks], o0[4 * ks + 1], o0[4 * ks + 2], o0[4 * ks + 3]};
            *reinterpret_cast<uint4_t*>(bex + (kt_begin & 1) * kBTile + b_wr + u * 32 * 16 + ks * (2 * BN * 16)) = v;
        }
    }
    __syncthreads();
    half8_t a0[TMW], b0[NB], a1[TMW], b1[NB];
    uint32_t r[DUTY][G::kRegs];
#pragma unroll
    for (int j = 1; j < ST; ++j) {
#pragma unroll
        for (int i = 0; i < XI; ++i) issue_x1(kt_begin + j, i);
#pragma unroll
        for (int i = 0; i < RI; ++i) issue_raw1(kt_begin + 1 + j, i);
    }
    load_ops(kt_begin, 0, a0, b0);
#pragma unroll
    for (int u = 0; u < DUTY; ++u)
        P::fetch(rraw + ((kt_begin + 1) & (ST - 1)) * kRawTile + my_raw + u * 32 * P::kRowBytes, h, P::delta(my_d0[u], kt_begin + 1), r[u]);

    // One k-step = NM matrix instructions (column block n, row block m in that order).  The other work of the k-tile is
    // placed by hand, piece by piece, behind the matrix instructions (one LDS access and a few vector instructions
    // each) and the scheduler is fenced after every piece, so that it neither clusters the unpacking nor moves an
    // operand read next to its use.
    constexpr int NM = TMW * NB;
    constexpr int kSlots = 3 * NM;                          // matrix instructions of k-steps 0 .. 2
    constexpr int kWorkOne = P::kMicro + 4;                 // unpack steps and the four exchange writes of 32 columns
    constexpr int kWork = DUTY * kWorkOne;
    constexpr int kPer = (kWork + kSlots - 1) / kSlots;
    static_assert(kPer <= 3, "unpack work must fit the slots");
    const typename P::Consts KC;
    for (int kt = kt_begin; kt < nkt; ++kt) {
        uint32_t o[16];
        typename P::State st;
        const int ph = P::phase(kt + 1);
        const bool live_k = kt + 1 < nkt && ((kt + 1) * 2 + h) * 32 < A.K;      // past the unit's end the raw bytes are zeros or stale
        const uint8_t* const xs = xbuf + (kt & (ST - 1)) * kXTile;
        const uint8_t* const bs = bex + (kt & 1) * kBTile + b_rd;
        uint8_t* const bnext = bex + ((kt + 1) & 1) * kBTile + b_wr;
        // work item w of the k-tile's unpacking: per 32 columns P::kMicro unpack steps with the four exchange writes
        // inserted as soon as their quarter is complete (quarters 0 and 2, then 1 and 3)
        auto work = [&](auto w_tag) {
            constexpr int wall = decltype(w_tag)::value;
            if constexpr (wall < kWork) {
                constexpr int u = wall / kWorkOne, w = wall % kWorkOne;
                constexpr int first_ready = P::kFirstHalf, second_ready = P::kMicro;
                uint8_t* const dst = bnext + u * 32 * 16;
                const uint32_t dl = P::delta(my_d0[u], kt + 1);
                const bool live = live_k && in_n[u];
                if constexpr (w < first_ready) {
                    P::template micro<w>(st, r[u], ph, h, dl, live, KC, o, bad[u]);
                } else if constexpr (w == first_ready || w == first_ready + 1) {
                    constexpr int q = w == first_ready ? 0 : 2;
                    const uint4_t v = {o[4 * q], o[4 * q + 1], o[4 * q + 2], o[4 * q + 3]};
                    *reinterpret_cast<uint4_t*>(dst + q * (2 * BN * 16)) = v;
                } else if constexpr (w < second_ready + 2) {
                    P::template micro<w - 2>(st, r[u], ph, h, dl, live, KC, o, bad[u]);
                } else {
                    constexpr int q = w == second_ready + 2 ? 1 : 3;
                    const uint4_t v = {o[4 * q], o[4 * q + 1], o[4 * q + 2], o[4 * q + 3]};
                    *reinterpret_cast<uint4_t*>(dst + q * (2 * BN * 16)) = v;
                }
            }
        };
        auto slot = [&](auto s_tag, const half8_t (&ac)[TMW], const half8_t (&bc)[NB], half8_t (&an)[TMW], half8_t (&bn)[NB], int ks_next) {
            constexpr int sidx = decltype(s_tag)::value;           // 0 .. kSlots - 1
            constexpr int i = sidx % NM, n = i / TMW, m = i % TMW;
            acc[m][n] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ac[m], bc[n], acc[m][n], 0, 0, 0);
            // operands of the next k-step, one read per matrix instruction (two where a k-step has fewer matrix
            // instructions than operands)
            auto read_op = [&](auto idx_tag) {
                constexpr int idx = decltype(idx_tag)::value;
                if constexpr (idx < TMW) an[idx] = *reinterpret_cast<const half8_t*>(xs + idx * 32 * kXRow + a_off[ks_next]);
                else if constexpr (idx < TMW + NB)
                    bn[idx - TMW] = *reinterpret_cast<const half8_t*>(bs + ks_next * (2 * BN * 16) + (idx - TMW) * 32 * 16);
            };
            read_op(std::integral_constant<int, i>{});
            if constexpr (TMW + NB > NM) read_op(std::integral_constant<int, i + NM>{});
            if constexpr (kPer >= 1) work(std::integral_constant<int, sidx * kPer>{});
            if constexpr (kPer >= 2) work(std::integral_constant<int, sidx * kPer + 1>{});
            if constexpr (kPer >= 3) work(std::integral_constant<int, sidx * kPer + 2>{});
            __builtin_amdgcn_sched_barrier(0);
        };
        auto kstep = [&](auto base_tag, const half8_t (&ac)[TMW], const half8_t (&bc)[NB], half8_t (&an)[TMW], half8_t (&bn)[NB], int ks_next) {
            constexpr int base = decltype(base_tag)::value;
            slot(std::integral_constant<int, base + 0>{}, ac, bc, an, bn, ks_next);
            slot(std::integral_constant<int, base + 1>{}, ac, bc, an, bn, ks_next);
            if constexpr (NM >= 4) {
                slot(std::integral_constant<int, base + 2>{}, ac, bc, an, bn, ks_next);
                slot(std::integral_constant<int, base + 3>{}, ac, bc, an, bn, ks_next);
            }
            if constexpr (NM >= 8) {
                slot(std::integral_constant<int, base + 4>{}, ac, bc, an, bn, ks_next);
                slot(std::integral_constant<int, base + 5>{}, ac, bc, an, bn, ks_next);
                slot(std::integral_constant<int, base + 6>{}, ac, bc, an, bn, ks_next);
                slot(std::integral_constant<int, base + 7>{}, ac, bc, an, bn, ks_next);
            }
            if constexpr (NM >= 16) {
                slot(std::integral_constant<int, base + 8>{}, ac, bc, an, bn, ks_next);
                slot(std::integral_constant<int, base + 9>{}, ac, bc, an, bn, ks_next);
                slot(std::integral_constant<int, base + 10>{}, ac, bc, an, bn, ks_next);
                slot(std::integral_constant<int, base + 11>{}, ac, bc, an, bn, ks_next);
                slot(std::integral_constant<int, base + 12>{}, ac, bc, an, bn, ks_next);
                slot(std::integral_constant<int, base + 13>{}, ac, bc, an, bn, ks_next);
                slot(std::integral_constant<int, base + 14>{}, ac, bc, an, bn, ks_next);
                slot(std::integral_constant<int, base + 15>{}, ac, bc, an, bn, ks_next);
            }
        };
        __builtin_amdgcn_sched_barrier(0);
        kstep(std::integral_constant<int, 0>{}, a0, b0, a1, b1, 1);
        kstep(std::integral_constant<int, NM>{}, a1, b1, a0, b0, 2);
        kstep(std::integral_constant<int, 2 * NM>{}, a0, b0, a1, b1, 3);
        wait_copies_and_barrier<0>();
        // behind the barrier: copies ST k-tiles ahead, first operands and raw bytes of the next k-tile, k-step 3
        {
            const uint8_t* const xn = xbuf + ((kt + 1) & (ST - 1)) * kXTile;
            const uint8_t* const bnx = bex + ((kt + 1) & 1) * kBTile + b_rd;
            const uint8_t* const rawn = rraw + ((kt + 2) & (ST - 1)) * kRawTile + my_raw;
            __builtin_amdgcn_sched_barrier(0);
            constexpr int kTail = NM > TMW + NB ? (NM > XI + RI ? NM : XI + RI) : (TMW + NB > XI + RI ? TMW + NB : XI + RI);
#pragma unroll
            for (int i = 0; i < kTail; ++i) {
                if (i < NM) {
                    const int n = i / TMW, m = i % TMW;
                    acc[m][n] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a1[m], b1[n], acc[m][n], 0, 0, 0);
                }
                if (i < TMW) a0[i] = *reinterpret_cast<const half8_t*>(xn + i * 32 * kXRow + a_off[0]);
                else if (i < TMW + NB) b0[i - TMW] = *reinterpret_cast<const half8_t*>(bnx + (i - TMW) * 32 * 16);
                if (i < DUTY) P::fetch(rawn + i * 32 * P::kRowBytes, h, P::delta(my_d0[i < DUTY ? i : 0], kt + 2), r[i]);
                if (i < XI) issue_x1(kt + ST, i);
                else if (i < XI + RI) issue_raw1(kt + ST + 1, i - XI);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    }

    // columns with a scale outside the operand range: the unpacking lanes publish their flags, the owners store NaN
#pragma unroll
    for (int u = 0; u < DUTY; ++u) {
        const int mine = G::out_of_range(bad[u]) ? 1 : 0;
        const int both = mine | __shfl_xor(mine, 32);                             // the column's two k-halves
        if (h == 0) col_bad[32 * DUTY * wave + 32 * u + col] = (uint32_t)both;
    }
    __syncthreads();
#pragma unroll
    for (int n = 0; n < NB; ++n) {
        if (col_bad[32 * NB * wn + 32 * n + col]) {
#pragma unroll
            for (int m = 0; m < TMW; ++m)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[m][n][r] = __uint_as_float(kNaNBits);
        }
    }

    // epilogue: D[row = 32 m + 8 (r / 4) + 4 h + r % 4][column] times the row scale
    float* cdst = A.c;
    int64_t ldc = A.ldc;
    const int* c_rows = A.c_rows;
    int accumulate = A.accumulate;
    if (A.partial) {
        cdst = A.partial + (int64_t)kc * A.M * A.N;
        ldc = A.N;
        c_rows = nullptr;
        accumulate = 0;
    }
    if (!c_rows && !accumulate) {
        store_wave_tile<TMW, NB, false>(tile_scales, acc, cdst, ldc, A.N, m0, m_rows, wm * (BM / 2), n0 + 32 * NB * wn + col, h);
        return;
    }
#pragma unroll
    for (int m = 0; m < TMW; ++m) {
        float sc[16];
        int64_t off[16];
#pragma unroll
        for (int r2 = 0; r2 < 16; ++r2) {
            const int ml = wm * (BM / 2) + m * 32 + 8 * (r2 >> 2) + 4 * h + (r2 & 3);
            const int mr = m0 + min(ml, m_rows - 1);
            sc[r2] = A.xscale[mr];
            off[r2] = (int64_t)(c_rows ? c_rows[mr] : mr) * ldc;
        }
#pragma unroll
        for (int n = 0; n < NB; ++n) {
            const int my_n = n0 + 32 * NB * wn + 32 * n + col;
            if (my_n >= A.N) continue;
#pragma unroll
            for (int r2 = 0; r2 < 16; ++r2) {
                const int ml = wm * (BM / 2) + m * 32 + 8 * (r2 >> 2) + 4 * h + (r2 & 3);
                if (ml < m_rows) {
                    float* p = cdst + off[r2] + my_n;
                    *p = accumulate ? *p + acc[m][n][r2] * sc[r2] : acc[m][n][r2] * sc[r2];
                }
            }
        }
    }
}

// Number of K chunks for a plain launch: with few tiles and a long K, chunks of K fill the CUs that a whole-K launch
// leaves idle.  Model: rounds of workgroups x k-tiles per chunk, plus writing and re-reading the chunk sums.
inline int pick_k_chunks(int tiles, int nkt, int slots, int64_t out_elems, double us_per_ktile)
{
    int best = 1;
    double best_t = (double)((tiles + slots - 1) / slots) * nkt * us_per_ktile;
    for (int sc = 2; sc <= 4; ++sc) {
        const int chunk = ((nkt + sc - 1) / sc + 3) / 4 * 4;
        // chunks down to 12 k-tiles (a floor of 32 was slower on every launch of few tiles that was measured: Q4_K
        // 1024 x 4096 x 3072 62.7 -> 53.9 us, Q8_0 512 x 4096 x 2048 45.8 -> 35.8, Q6_K 1024 x 4096 x 3072 87.1 -> 65.6,
        // MXFP4 640 x 2880 x 2880 42.1 -> 32.6)
        if (chunk < 12) break;
        const double t = (double)((tiles * sc + slots - 1) / slots) * chunk * us_per_ktile + 2.0 * sc * out_elems * 4 / 4.5e6;
        if (t < 0.9 * best_t) {
            best = sc;
            best_t = t;
        }
    }
    return best;
}

template <typename G, int BM, int XST, int NW>
bool launch_tiles(GemmArgs a, int m_tiles, hipStream_t stream, const ChunkScratch& cs)
{
    constexpr int BN = NW * 32, RT = BN * G::kRawRow;
    auto kern = gemm_kernel<G, BM, XST, NW>;
    constexpr int RB = (XST > 2 && G::kSup == 2) ? 3 : 2;
    const size_t lds = (size_t)XST * BM * kXRow + (size_t)RB * RT + 1024 + BM * 4;
    if (!cs.need_out && !raise_lds_limit(reinterpret_cast<const void*>(kern), lds)) return false;
    a.m_tiles = m_tiles;
    a.n_tiles = (a.N + BN - 1) / BN;
    const int nkt = a.Kp / kBK;
    a.k_chunks = 1;
    a.chunk_kt = (nkt + 3) / 4 * 4;
    a.partial = nullptr;
    if (!a.tile_expert) {
        const int per_cu = std::max(1, (int)((160 * 1024) / (lds + 512)));
        // measured: about 1.7 us per k-tile of a 256 x 256 tile when all CUs are busy
        a.k_chunks = pick_k_chunks(a.m_tiles * a.n_tiles, nkt, device_info().num_cus * per_cu, (int64_t)a.M * a.N,
                                   1.7 * BM * BN / 65536.0 * per_cu);
        if (a.k_chunks > 1) {
            a.chunk_kt = ((nkt + a.k_chunks - 1) / a.k_chunks + 3) / 4 * 4;
            a.k_chunks = (nkt + a.chunk_kt - 1) / a.chunk_kt;
            const size_t need = (size_t)a.k_chunks * a.M * a.N * sizeof(float);
            if (cs.need_out) *cs.need_out = need;
            a.partial = chunk_scratch(cs, need);
            if (!a.partial) {
                // the caller's scratch is too small for the chunk sums: whole K per tile (slower, same result up to
                // fp32 summation order)
                a.k_chunks = 1;
                a.chunk_kt = (nkt + 3) / 4 * 4;
            }
        }
    }
    if (cs.need_out) return true;
    const int total = a.m_tiles * a.n_tiles * a.k_chunks;
    const int grid = ((total + 7) / 8) * 8;          // whole rounds over the 8 XCDs
    hipLaunchKernelGGL(kern, dim3(grid), dim3(NW * 64), lds, stream, a);
    if (!hip_ok(hipGetLastError(), "gemm launch")) return false;
    if (a.partial) {
        return launch_chunk_sum(a, stream);
    }
    return true;
}

template <typename P, int BM, int WN>
bool launch_xw(GemmArgs a, int m_tiles, hipStream_t stream, const ChunkScratch& cs)
{
    constexpr int BN = 256;
    auto kern = gemm_xw_kernel<P, BM, WN>;
    constexpr size_t kLds = (size_t)2 * BM * kXRow + (size_t)2 * BN * P::kRowBytes + (size_t)2 * 4 * 2 * BN * 16 + 1024 + BM * 4 + BN * 4;
    static_assert(kLds <= 160 * 1024, "LDS");
    const size_t lds = kLds;
    if (!cs.need_out && !raise_lds_limit(reinterpret_cast<const void*>(kern), lds)) return false;
    a.m_tiles = m_tiles;
    a.n_tiles = (a.N + BN - 1) / BN;
    const int nkt = a.Kp / kBK;
    a.k_chunks = 1;
    a.chunk_kt = (nkt + 3) / 4 * 4;
    a.partial = nullptr;
    if (!a.tile_expert) {
        a.k_chunks = pick_k_chunks(a.m_tiles * a.n_tiles, nkt, device_info().num_cus, (int64_t)a.M * a.N, 1.7 * BM * BN / 65536.0);
        if (a.k_chunks > 1) {
            a.chunk_kt = ((nkt + a.k_chunks - 1) / a.k_chunks + 3) / 4 * 4;
            a.k_chunks = (nkt + a.chunk_kt - 1) / a.chunk_kt;
            const size_t need = (size_t)a.k_chunks * a.M * a.N * sizeof(float);
            if (cs.need_out) *cs.need_out = need;
            a.partial = chunk_scratch(cs, need);
            if (!a.partial) {
                a.k_chunks = 1;
                a.chunk_kt = (nkt + 3) / 4 * 4;
            }
        }
    }
    if (cs.need_out) return true;
    const int total = a.m_tiles * a.n_tiles * a.k_chunks;
    const int grid = ((total + 7) / 8) * 8;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(128 * WN), lds, stream, a);
    if (!hip_ok(hipGetLastError(), "gemm launch")) return false;
    if (a.partial) {
        return launch_chunk_sum(a, stream);
    }
    return true;
}

// ------------------------------------------------------------------------------------------
// MXFP4 on the block-scaled matrix instruction (v_mfma_scale_f32_32x32x64_f8f6f4): the weight operand is the RAW block -
// 16 bytes of E2M1 pairs plus its E8M0 scale byte, exactly what the instruction's fp4 operand and block scale are -
// so nothing is unpacked at all.  The activations are two MX terms of fp6 (E2M3) per 32-element block, x = hi 2^Eh +
// lo 2^El (convert_x_mx_kernel), every product takes two instructions, and fp6 x fp4 runs at twice the rate of the
// fp16 instruction, so the pair costs half of what the fp16 k-tile costs.  Same tiles as gemm_xw_kernel (BM x 256 x 64,
// 2 x 4 wavefronts of BM / 2 x 64) and the same LDS-direct copies; no exchange area, so ST copy stages fit.  Operand
// layout of the instruction (probed on the device): output as the fp16 instructions; lane = column + 32 g holds block g
// of the k-tile's weights, 32 nibbles low nibble first, and lane = row + 32 g block g of the activations as a stream
// of 32 six-bit fields, field f pairing with nibble f; each lane's scale byte (selected by op_sel from its scale
// register) applies to its own block.
// A scale byte of 255 is NaN to the instruction (ggml's table gives 2^127 there; no quantizer writes it).
typedef int int8v_t __attribute__((ext_vector_type(8)));

template <int BM, int ST>
__global__ void __launch_bounds__(512) gemm_mx_kernel(const GemmArgs A)
{
    typedef PMXFP4 P;
    constexpr int BN = 256, WN = 4, NW = 8;
    constexpr int TMW = BM / 64;                          // 32-row blocks of a wavefront
    constexpr int NB = 2;                                 // 32-column blocks of a wavefront
    constexpr int kXTile = BM * kXRow;
    constexpr int XI = kXTile / 1024 / NW;
    constexpr int kRawTile = BN * P::kRowBytes;
    constexpr int kRawCopies = kRawTile / 1024;
    constexpr int RI = (kRawCopies + NW - 1) / NW;
    static_assert(TMW == 2 || TMW == 4, "128- or 256-row tiles");
    static_assert(kRawCopies * 1024 == kRawTile && XI >= 1 && XI * NW * 1024 == kXTile && ST >= 2, "tile pieces must be whole KiB");
    extern __shared__ uint8_t smem[];
    uint8_t* const xbuf = smem;                           // ST x kXTile
    uint8_t* const rraw = xbuf + ST * kXTile;             // ST x kRawTile
    uint8_t* const dump = rraw + ST * kRawTile;           // 1 KiB

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WN, wn = wave % WN;
    const int col = lane & 31, h = lane >> 5;

    const int tiles = A.m_tiles * A.n_tiles;
    const int total = tiles * A.k_chunks;
    int t = blockIdx.x;
    {
        const int per = (total + 7) >> 3;
        const int xcd = t & 7, slot = t >> 3;
        t = xcd * per + slot;
        if (slot >= per || t >= total) return;
    }
    const int kc = t / tiles;
    t -= kc * tiles;
    const int mt = t / A.n_tiles, nt = t - mt * A.n_tiles;
    const int m0 = mt * BM, m_rows = min(BM, A.M - m0), n0 = nt * BN;

    const uintptr_t wa = reinterpret_cast<uintptr_t>(A.w);
    const uint32_t base_delta = (uint32_t)(wa & 3);
    const __amdgpu_buffer_rsrc_t wrs = __builtin_amdgcn_make_buffer_rsrc(
        reinterpret_cast<void*>(wa - base_delta), 0, (int)(((uint32_t)A.w_bytes + base_delta + 3u) & ~3u), 0x00020000);
    const __amdgpu_buffer_rsrc_t xrs = __builtin_amdgcn_make_buffer_rsrc(const_cast<_Float16*>(A.x16), 0, (int)A.x16_bytes, 0x00020000);
    const uint32_t row_bytes = (uint32_t)((int64_t)A.w_bytes / A.N);
    const int kt_begin = kc * A.chunk_kt;
    const int nkt = min(A.Kp / kBK, kt_begin + A.chunk_kt);

    uint32_t x_off[XI], r_off[RI];
#pragma unroll
    for (int i = 0; i < XI; ++i) {
        const int q = (wave + NW * i) * 64 + lane;
        const int row = q >> 3, chunk = (q & 7) ^ ((row >> 1) & 7);
        x_off[i] = row < m_rows ? (uint32_t)(m0 + row) * (uint32_t)(A.xld * 2) + (uint32_t)chunk * 16u : kDeadOffset;
    }
#pragma unroll
    for (int i = 0; i < RI; ++i) {
        const int q = (wave + NW * i) * 64 + lane;                // 16-byte piece of the raw tile
        const int row = q / P::kParts, part = q - row * P::kParts;
        const bool ok = q < BN * P::kParts && n0 + row < A.N;
        r_off[i] = ok ? P::row_window(base_delta + (uint32_t)(n0 + row) * row_bytes) + P::part_base(part) : kDeadOffset;
    }
    // every wavefront issues XI + RI copies per k-tile (surplus raw copies go to the dump area, k-tiles past the end
    // read out of range), so the wait before a barrier is a count
    // copy c (0 .. RI + XI - 1) of k-tile kt into a stage
    auto issue_one = [&](int kt, int stage, int c) {
        const uint32_t past = kt < nkt ? 0u : kDeadOffset;
        if (c < RI) {
            const int id = wave + NW * c;
            copy16_to_lds(wrs, id < kRawCopies ? rraw + stage * kRawTile + id * 1024 : dump, r_off[c] | past, P::soffset(kt));
        } else {
            const int i = c - RI;
            copy16_to_lds(xrs, xbuf + stage * kXTile + (wave + NW * i) * 1024, x_off[i] | past, (uint32_t)kt * kXRow);
        }
    };
    auto issue = [&](int kt, int stage) {
#pragma unroll
        for (int c = 0; c < RI + XI; ++c) issue_one(kt, stage, c);
    };
    // The copies of a k-tile are spread over the TMW groups of matrix instructions that follow the barrier which freed
    // their stage (copy c goes behind group c % TMW): a copy occupies the wavefront and the CU's address path for tens
    // of cycles, and behind a group the matrix pipe has work queued for that long.
    auto issue_slot = [&](int kt, int stage, int slot) {
#pragma unroll
        for (int c = 0; c < RI + XI; ++c)
            if (c % TMW == slot) issue_one(kt, stage, c);
    };

    float16_t acc[TMW][NB];
#pragma unroll
    for (int m = 0; m < TMW; ++m)
#pragma unroll
        for (int n = 0; n < NB; ++n)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[m][n][r] = 0.f;

    // this lane's pieces of an activation row (block h of the k-tile): term p keeps the first 16 bytes of its stream in
    // piece 3 p + 2 h and the last 8 in half h of piece 3 p + 1; the two scale bytes are dword h of piece 6; pieces sit
    // where the copy's swizzle placed them
    const int sw = (col >> 1) & 7;
    const int a_row = (wm * (BM / 2) + col) * kXRow;
    int a_main[2], a_rest[2];
#pragma unroll
    for (int p = 0; p < 2; ++p) {
        a_main[p] = a_row + ((3 * p + 2 * h) ^ sw) * 16;
        a_rest[p] = a_row + ((3 * p + 1) ^ sw) * 16 + 8 * h;
    }
    const int a_scale = a_row + (6 ^ sw) * 16 + 4 * h;
    const int my_raw = (32 * NB * wn + col) * P::kRowBytes;
    uint32_t my_d0[NB];
#pragma unroll
    for (int n = 0; n < NB; ++n) my_d0[n] = P::row_delta(base_delta + (uint32_t)(n0 + 32 * NB * wn + 32 * n + col) * row_bytes);

    // B operands of k-tile kt from its stage: the lane's raw block (fetch_b), then re-aligned and with its scale byte
    // (finish_b) - two steps, so that the matrix instructions between them cover the LDS latency.  Block h of the
    // k-tile starts delta + 17 h bytes into the row's 48-byte window, i.e. delta + h (0 .. 6) bytes into the window's
    // 16-byte piece h: the 17 bytes lie in pieces h and h + 1, read as two aligned 16-byte pieces (at the 48-byte row
    // stride sixteen lanes cover all 64 banks once; dword reads at that stride collide four ways).
    auto fetch_b = [&](int /*kt*/, int st, uint4_t (&r)[NB][2]) {
        const uint8_t* const rws = rraw + st * kRawTile + my_raw + 16 * h;
#pragma unroll
        for (int n = 0; n < NB; ++n) {
            r[n][0] = *reinterpret_cast<const uint4_t*>(rws + n * 32 * P::kRowBytes);
            r[n][1] = *reinterpret_cast<const uint4_t*>(rws + n * 32 * P::kRowBytes + 16);
        }
    };
    auto finish_b = [&](int kt, const uint4_t (&r)[NB][2], int8v_t (&b)[NB], int (&sb)[NB]) {
        const bool live = (kt * 2 + h) * 32 < A.K;
#pragma unroll
        for (int n = 0; n < NB; ++n) {
            const uint32_t sh = P::delta(my_d0[n], kt) + (uint32_t)h;          // scale byte at sh, nibbles behind it
            const uint32_t e = ((sh >> 2 ? r[n][0].y : r[n][0].x) >> (8 * (sh & 3))) & 0xffu;
            const bool up = ((sh + 1) >> 2) != 0;                              // the nibbles start in dword 1
            const uint32_t shb = (sh + 1) & 3;
            const uint32_t v0 = up ? r[n][0].y : r[n][0].x, v1 = up ? r[n][0].z : r[n][0].y, v2 = up ? r[n][0].w : r[n][0].z;
            const uint32_t v3 = up ? r[n][1].x : r[n][0].w, v4 = up ? r[n][1].y : r[n][1].x;
            // a block past the end of K: zeros under a scale of one (its bytes belong to the next row)
            b[n][0] = live ? (int)__builtin_amdgcn_alignbyte(v1, v0, shb) : 0;
            b[n][1] = live ? (int)__builtin_amdgcn_alignbyte(v2, v1, shb) : 0;
            b[n][2] = live ? (int)__builtin_amdgcn_alignbyte(v3, v2, shb) : 0;
            b[n][3] = live ? (int)__builtin_amdgcn_alignbyte(v4, v3, shb) : 0;
            b[n][4] = b[n][5] = b[n][6] = b[n][7] = 0;
            sb[n] = live ? (int)e : 127;
        }
    };
    // A operands of 32-row block m: the two streams of the lane's block (24 bytes each) and its two scale bytes, kept in
    // plain registers (an aggregate would live in scratch memory, whose loads share the counter of the copies)
    typedef uint32_t uint2_t __attribute__((ext_vector_type(2)));
#define TSHIP_MX_AOP(V) uint4_t V##_h0, V##_l0; uint2_t V##_h1, V##_l1; uint32_t V##_sa
#define TSHIP_MX_LOAD_A(st, m, V)                                                              \
    do {                                                                                       \
        const uint8_t* const xr_ = xbuf + (st) * kXTile + (m) * 32 * kXRow;                     \
        V##_h0 = *reinterpret_cast<const uint4_t*>(xr_ + a_main[0]);                           \
        V##_h1 = *reinterpret_cast<const uint2_t*>(xr_ + a_rest[0]);                           \
        V##_l0 = *reinterpret_cast<const uint4_t*>(xr_ + a_main[1]);                           \
        V##_l1 = *reinterpret_cast<const uint2_t*>(xr_ + a_rest[1]);                           \
        V##_sa = *reinterpret_cast<const uint32_t*>(xr_ + a_scale); /* byte 0: scale of hi, byte 1: of lo */ \
    } while (0)
#define TSHIP_MX_MULTIPLY(V, m, B, SB)                                                                                   \
    do {                                                                                                                 \
        const int8v_t ahi_ = {(int)V##_h0.x, (int)V##_h0.y, (int)V##_h0.z, (int)V##_h0.w, (int)V##_h1.x, (int)V##_h1.y, 0, 0}; \
        const int8v_t alo_ = {(int)V##_l0.x, (int)V##_l0.y, (int)V##_l0.z, (int)V##_l0.w, (int)V##_l1.x, (int)V##_l1.y, 0, 0}; \
        _Pragma("unroll") for (int n = 0; n < NB; ++n) {                                                                 \
            acc[m][n] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(ahi_, B[n], acc[m][n], 2, 4, 0, (int)V##_sa, 0, SB[n]); \
            acc[m][n] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(alo_, B[n], acc[m][n], 2, 4, 1, (int)V##_sa, 0, SB[n]); \
        }                                                                                                                \
    } while (0)

    // The operands of a row block are read while the block before it is multiplied, and the k-tile's barrier sits in
    // front of its LAST row block: by then every operand of the k-tile is in registers, so behind the barrier the stage
    // takes the copy ST k-tiles on and the first operands of the next k-tile are read under that last block's matrix
    // instructions.  The LDS latency then never stands between two groups of matrix instructions.
    int stage = 0;                                         // stage of k-tile kt
#pragma unroll
    for (int j = 0; j < ST - 1; ++j) issue(kt_begin + j, j);
    wait_copies_and_barrier<(ST - 2) * (XI + RI)>();
    issue_slot(kt_begin + ST - 1, ST - 1, 0);              // its other copies follow in the first k-tile of the loop
    int8v_t b[NB];
    int sb[NB];
    uint4_t braw[NB][2];
    TSHIP_MX_AOP(a0);                                      // row blocks alternate between the two (TMW is even)
    TSHIP_MX_AOP(a1);
    fetch_b(kt_begin, 0, braw);
    TSHIP_MX_LOAD_A(0, 0, a0);
    finish_b(kt_begin, braw, b, sb);
#define TSHIP_MX_KTILE(KT, B, SB)                                                                                          \
    do {                                                                                                                 \
        const int prev_ = stage == 0 ? ST - 1 : stage - 1;     /* the stage freed by the barrier of k-tile KT - 1 */     \
        TSHIP_MX_LOAD_A(stage, 1, a1);                                                                                   \
        __builtin_amdgcn_sched_barrier(0);                                                                               \
        TSHIP_MX_MULTIPLY(a0, 0, B, SB);                                                                                 \
        issue_slot((KT) - 1 + ST, prev_, 1);                                                                             \
        __builtin_amdgcn_sched_barrier(0);                                                                               \
        if constexpr (TMW == 4) {                                                                                        \
            TSHIP_MX_LOAD_A(stage, 2, a0);                                                                               \
            __builtin_amdgcn_sched_barrier(0);                                                                           \
            TSHIP_MX_MULTIPLY(a1, 1, B, SB);                                                                             \
            issue_slot((KT) - 1 + ST, prev_, 2);                                                                         \
            __builtin_amdgcn_sched_barrier(0);                                                                           \
            TSHIP_MX_LOAD_A(stage, 3, a1);                                                                               \
            __builtin_amdgcn_sched_barrier(0);                                                                           \
            TSHIP_MX_MULTIPLY(a0, 2, B, SB);                                                                             \
            issue_slot((KT) - 1 + ST, prev_, 3);                                                                         \
            __builtin_amdgcn_sched_barrier(0);                                                                           \
        }                                                                                                                \
        const int next_ = stage == ST - 1 ? 0 : stage + 1;                                                               \
        /* k-tile KT + 1 has landed once at most the copies of the ST - 2 k-tiles after it are in flight */              \
        wait_copies_and_barrier<(ST - 2) * (XI + RI)>();                                                                 \
        fetch_b((KT) + 1, next_, braw);                                                                                  \
        TSHIP_MX_LOAD_A(next_, 0, a0);                                                                                   \
        __builtin_amdgcn_sched_barrier(0);                                                                               \
        TSHIP_MX_MULTIPLY(a1, TMW - 1, B, SB);                                                                           \
        issue_slot((KT) + ST, stage, 0);                                                                                 \
        __builtin_amdgcn_sched_barrier(0);                                                                               \
        finish_b((KT) + 1, braw, B, SB);      /* the last multiply has read B: the next k-tile's operands take its place */ \
        stage = next_;                                                                                                   \
    } while (0)
    for (int kt = kt_begin; kt < nkt; ++kt) TSHIP_MX_KTILE(kt, b, sb);
#undef TSHIP_MX_KTILE
#undef TSHIP_MX_AOP
#undef TSHIP_MX_LOAD_A
#undef TSHIP_MX_MULTIPLY

    // epilogue: D[row = 32 m + 8 (r / 4) + 4 h + r % 4][column] times the row scale
    float* cdst = A.c;
    int64_t ldc = A.ldc;
    const int* c_rows = A.c_rows;
    int accumulate = A.accumulate;
    if (A.partial) {
        cdst = A.partial + (int64_t)kc * A.M * A.N;
        ldc = A.N;
        c_rows = nullptr;
        accumulate = 0;
    }
    if (!c_rows && !accumulate) {
        store_wave_tile<TMW, NB, true>(nullptr, acc, cdst, ldc, A.N, m0, m_rows, wm * (BM / 2), n0 + 32 * NB * wn + col, h);
        return;
    }
#pragma unroll
    for (int m = 0; m < TMW; ++m) {
        float sc[16];
        int64_t off[16];
#pragma unroll
        for (int r2 = 0; r2 < 16; ++r2) {
            const int ml = wm * (BM / 2) + m * 32 + 8 * (r2 >> 2) + 4 * h + (r2 & 3);
            const int mr = m0 + min(ml, m_rows - 1);
            sc[r2] = A.xscale[mr];
            off[r2] = (int64_t)(c_rows ? c_rows[mr] : mr) * ldc;
        }
#pragma unroll
        for (int n = 0; n < NB; ++n) {
            const int my_n = n0 + 32 * NB * wn + 32 * n + col;
            if (my_n >= A.N) continue;
#pragma unroll
            for (int r2 = 0; r2 < 16; ++r2) {
                const int ml = wm * (BM / 2) + m * 32 + 8 * (r2 >> 2) + 4 * h + (r2 & 3);
                if (ml < m_rows) {
                    float* pc = cdst + off[r2] + my_n;
                    *pc = accumulate ? *pc + acc[m][n][r2] * sc[r2] : acc[m][n][r2] * sc[r2];
                }
            }
        }
    }
}

template <int BM>
bool launch_mx(GemmArgs a, int m_tiles, hipStream_t stream, const ChunkScratch& cs)
{
    constexpr int BN = 256, ST = BM == 128 ? 5 : 3;
    auto kern = gemm_mx_kernel<BM, ST>;
    constexpr size_t kLds = (size_t)ST * BM * kXRow + (size_t)ST * BN * PMXFP4::kRowBytes + 1024;
    static_assert(kLds <= 160 * 1024, "LDS");
    if (!cs.need_out && !raise_lds_limit(reinterpret_cast<const void*>(kern), kLds)) return false;
    a.m_tiles = m_tiles;
    a.n_tiles = (a.N + BN - 1) / BN;
    const int nkt = a.Kp / kBK;
    a.k_chunks = 1;
    a.chunk_kt = (nkt + 3) / 4 * 4;
    a.partial = nullptr;
    a.k_chunks = pick_k_chunks(a.m_tiles * a.n_tiles, nkt, device_info().num_cus, (int64_t)a.M * a.N, 1.7 * BM * BN / 65536.0);
    if (a.k_chunks > 1) {
        a.chunk_kt = ((nkt + a.k_chunks - 1) / a.k_chunks + 3) / 4 * 4;
        a.k_chunks = (nkt + a.chunk_kt - 1) / a.chunk_kt;
        const size_t need = (size_t)a.k_chunks * a.M * a.N * sizeof(float);
        if (cs.need_out) *cs.need_out = need;
        a.partial = chunk_scratch(cs, need);
        if (!a.partial) {
            a.k_chunks = 1;
            a.chunk_kt = (nkt + 3) / 4 * 4;
        }
    }
    if (cs.need_out) return true;
    const int total = a.m_tiles * a.n_tiles * a.k_chunks;
    const int grid = ((total + 7) / 8) * 8;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(512), kLds, stream, a);
    if (!hip_ok(hipGetLastError(), "gemm launch")) return false;
    if (a.partial) {
        return launch_chunk_sum(a, stream);
    }
    return true;
}

// ------------------------------------------------------------------------------------------
// At most 32 activation rows per tile (small batches, MoE experts with few tokens; also single rows of formats
// without a GEMV kernel).  The activations stay in REGISTERS: the eight wavefronts of a workgroup split K between
// them (KTW k-tiles each), every wavefront keeps the MFMA A operands of its K range for all 32 rows, and the
// workgroup walks over 32-column weight tiles.  Per tile a wavefront needs only its own K range of the 32 raw
// weight rows, which it copies itself (global -> LDS, a private ring of buffers, requested RING tiles ahead), so
// the main loop has no barrier and no activation traffic at all; the eight partial 32 x 32 sums meet in LDS (in
// the raw buffer the wavefront has just consumed), are added in a fixed order and stored.  A K longer than
// 8 * KTW k-tiles is cut into chunks whose sums a second kernel adds.
// ------------------------------------------------------------------------------------------
// an address that is the same in every lane, for the compiler to keep in scalar registers
__device__ __forceinline__ uintptr_t uniform_address(uintptr_t a)
{
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)a), hi = __builtin_amdgcn_readfirstlane((uint32_t)(a >> 32));
    return ((uintptr_t)hi << 32) | lo;
}
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// LDS layout of one wavefront of the register-resident kernel: RING raw buffers of 32 rows x CH 16-byte chunks
// (the bytes of KTW k-tiles plus the up to three bytes between the 4-byte aligned window start and the first
// block; the unpackers may read a few bytes further, into the next row, and ignore them)
template <typename G, int KTW>
struct SlimLayout {
    static constexpr int kNeed = (G::window_bytes(KTW) + 15) / 16;
    static constexpr int buf_of(int ch) { return 32 * ch * 16 > 4096 ? 32 * ch * 16 : 4096; }
    static constexpr int ring_of(int ch) { return 8 * 3 * buf_of(ch) + 1024 <= 160 * 1024 ? 3 : 2; }
    // an odd chunk count spreads the dword reads of the 32 rows over twice as many LDS banks; taken when it costs no
    // ring depth and still fits
    static constexpr bool kOdd = (kNeed & 1) == 0 && ring_of(kNeed + 1) == ring_of(kNeed) &&
                                 8 * ring_of(kNeed + 1) * buf_of(kNeed + 1) + 64 <= 160 * 1024;
    static constexpr int CH = kNeed + (kOdd ? 1 : 0);
    static constexpr int DI = (32 * CH + 63) / 64;                       // LDS-direct copies per buffer
    static constexpr int RAW = 32 * CH * 16;
    static constexpr int BUF = RAW > 4096 ? RAW : 4096;                  // raw rows, later the 32 x 32 fp32 partial sums
    static constexpr int RING = 8 * 3 * BUF + 1024 <= 160 * 1024 ? 3 : 2;
};

template <typename G, int KTW>
__global__ void __launch_bounds__(512) gemm_slim_kernel(const GemmArgs A)
{
    using L = SlimLayout<G, KTW>;
    constexpr int CH = L::CH, DI = L::DI, BUF = L::BUF, RING = L::RING;
    static_assert(KTW % G::kTileStep == 0, "a wavefront's K range must start at a block");
    extern __shared__ uint8_t smem[];                                   // 8 wavefronts x RING x BUF

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int col = lane & 31, h = lane >> 5;
    uint8_t* const my_buf = smem + wave * RING * BUF;

    const uint32_t row_bytes = (uint32_t)((int64_t)A.w_bytes / A.N);
    const int nkt = A.Kp / kBK;
    const int n32 = (A.N + 31) >> 5;
    const int per_tile = A.k_chunks * n32;                              // units of one row tile

    // grouped launches: the table may end in empty tiles
    int live_tiles = A.m_tiles;
    if (A.tile_expert) {
        int c = 0;
        for (int i = lane; i < A.m_tiles; i += 64) c += A.tile_rows[i] > 0 ? 1 : 0;
        for (int o = 32; o > 0; o >>= 1) c += __shfl_xor(c, o);
        live_tiles = __builtin_amdgcn_readfirstlane(c);
    }
    // units = (row tile, K chunk, 32-column tile), column tile fastest; every workgroup takes one contiguous run
    const int64_t units = (int64_t)live_tiles * per_tile;
    int u = (int)(units * blockIdx.x / gridDim.x);
    const int u_end = (int)(units * (blockIdx.x + 1) / gridDim.x);

    while (u < u_end) {
        const int mt = u / per_tile, rem = u - mt * per_tile;
        const int kc = rem / n32, nt0 = rem - kc * n32, cnt = min(n32 - nt0, u_end - u);
        u += cnt;
        const int kt0 = kc * A.chunk_kt + wave * KTW;
        const int kcnt = max(0, min(KTW, nkt - kt0));                  // k-tiles of this wavefront in this chunk
        int m0, m_rows;
        const uint8_t* wbase = A.w;
        if (A.tile_expert) {
            m0 = A.tile_row0[mt];
            m_rows = min(32, A.tile_rows[mt]);
            wbase += expert_offset(A, mt);
        } else {
            m0 = mt * 32;
            m_rows = min(32, A.M - m0);
        }
        // (the expert id comes from memory the kernel also writes to, so the compiler loads it per lane: without the
        // hint every copy would run in a loop over the distinct descriptors of the wavefront)
        const uintptr_t wa = uniform_address(reinterpret_cast<uintptr_t>(wbase));
        const uint32_t base_delta = (uint32_t)(wa & 3);
        const __amdgpu_buffer_rsrc_t wrs = __builtin_amdgcn_make_buffer_rsrc(
            reinterpret_cast<void*>(wa & ~(uintptr_t)3), 0, (int)(((uint32_t)A.w_bytes + base_delta + 3u) & ~3u), 0x00020000);

        // MFMA A operands of this wavefront's K range: row `col`, k-half h of every k-step
        half8_t a[KTW][4];
        {
            const _Float16* xr = A.x16 + (int64_t)(m0 + min(col, m_rows - 1)) * A.xld + h * 8;
            const half8_t zero = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
            for (int t = 0; t < KTW; ++t) {
                const int kt = min(kt0 + t, nkt - 1);
#pragma unroll
                for (int ks = 0; ks < 4; ++ks) {
                    const half8_t v = *reinterpret_cast<const half8_t*>(xr + kt * kBK + ks * 16);
                    a[t][ks] = (col < m_rows && t < kcnt) ? v : zero;
                }
            }
        }
        // Source offsets of the raw copies.  32 rows are a multiple of four bytes, so a row's alignment
        // inside its window is the same in every column tile.
        const uint32_t koff = G::tile_offset(kt0);
        uint32_t w_off[DI];
#pragma unroll
        for (int i = 0; i < DI; ++i) {
            const int q = i * 64 + lane;
            const int row = q / CH, chunk = q - row * CH;
            w_off[i] = (row < 32 && kcnt > 0) ? ((base_delta + (uint32_t)row * row_bytes + koff) & ~3u) + (uint32_t)chunk * 16u : kDeadOffset;
        }
        const uint32_t my_delta = (base_delta + (uint32_t)col * row_bytes + koff) & 3u;
        auto issue = [&](int i, int b) {                // column tile nt0 + i -> buffer b
            uint8_t* dst = my_buf + b * BUF;
            const bool any = i < cnt;
            const uint32_t so = any ? (uint32_t)(nt0 + i) * 32u * row_bytes : 0u;
#pragma unroll
            for (int q = 0; q < DI; ++q) {
                // an odd number of chunks per row leaves the last copy half full: its upper lanes stay out (they would
                // write into the next buffer)
                if (q * 64 + 32 < 32 * CH || lane < 32) copy16_to_lds(wrs, dst + q * 1024, any ? w_off[q] : kDeadOffset, so);
            }
        };
        // result rows of this thread in the reduction: accumulator registers `wave` and `wave + 8`
        float sc[2];
        int64_t coff[2];
        bool ok[2];
#pragma unroll
        for (int q = 0; q < 2; ++q) {
            const int r = wave + 8 * q;
            const int ml = 8 * (r >> 2) + 4 * h + (r & 3);
            const int m = m0 + min(ml, m_rows - 1);
            sc[q] = A.xscale[m];
            coff[q] = A.partial ? ((int64_t)kc * A.M + m) * A.N : (int64_t)(A.c_rows ? A.c_rows[m] : m) * A.ldc;
            ok[q] = ml < m_rows;
        }

#pragma unroll
        for (int b = 0; b < RING; ++b) issue(b, b);
        int b = 0;                                      // buffer of column tile i
        float pend[2] = {0.f, 0.f};
        int pend_n = -1;
        float* const dst = A.partial ? A.partial : A.c;
        auto flush = [&]() {
            if (pend_n >= 0 && pend_n < A.N) {
#pragma unroll
                for (int q = 0; q < 2; ++q)
                    if (ok[q]) dst[coff[q] + pend_n] = pend[q];
            }
        };
        for (int i = 0; i < cnt; ++i) {
            // the copies of tile i have landed; those of the RING - 1 tiles after it stay in flight
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"((RING - 1) * DI) : "memory");
            // the previous tile's results leave here, after the wait: a store in flight at the wait would be
            // counted against it
            flush();
            float16_t acc;
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[r] = 0.f;
            uint32_t bad = 0u;                          // a scale of this lane's column does not fit the fp16 operands
            const bool in_n = (nt0 + i) * 32 + col < A.N;
            const uint8_t* raw = my_buf + b * BUF + col * (CH * 16);
            // a wavefront with a full K range runs the k-tiles as one branch-free block, so the unpacking of one
            // k-tile is scheduled into the matrix instructions of the previous one
            auto k_tiles = [&](auto full_tag) {
                constexpr bool kFull = decltype(full_tag)::value;
#pragma unroll
                for (int t = 0; t < KTW; ++t) {
                    if (kFull || t < kcnt) {
                        uint32_t r[G::kRegs], o[16];
                        G::fetch(raw, t, h, my_delta, r);
                        G::dequant(r, t, h, my_delta, ((kt0 + t) * 2 + h) * 32 < A.K && in_n, o, bad);
#pragma unroll
                        for (int ks = 0; ks < 4; ++ks) {
                            const uint4_t bb = {o[4 * ks], o[4 * ks + 1], o[4 * ks + 2], o[4 * ks + 3]};
                            acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[t][ks], __builtin_bit_cast(half8_t, bb), acc, 0, 0, 0);
                        }
                    }
                }
            };
            if (kcnt == KTW) k_tiles(std::true_type{});
            else k_tiles(std::false_type{});
            {
                float16_t one[1] = {acc};
                poison_column<1>(one, G::out_of_range(bad));
                acc = one[0];
            }
            // partial sums of this wavefront's K range -> the buffer it has just consumed
            float* part = reinterpret_cast<float*>(my_buf + b * BUF);
#pragma unroll
            for (int r = 0; r < 16; ++r) part[r * 64 + lane] = acc[r];
            lds_barrier();
            float s0 = 0.f, s1 = 0.f;
#pragma unroll
            for (int v = 0; v < 8; ++v) {
                const float* pv = reinterpret_cast<const float*>(smem + (v * RING + b) * BUF);
                s0 += pv[wave * 64 + lane];
                s1 += pv[(wave + 8) * 64 + lane];
            }
            pend[0] = s0 * sc[0];
            pend[1] = s1 * sc[1];
            pend_n = (nt0 + i) * 32 + col;
            lds_barrier();                              // every partial sum has been read: the buffers may be refilled
            issue(i + RING, b);
            b = b + 1 == RING ? 0 : b + 1;
        }
        flush();
    }
}

// c[row][n] (+)= sum over the K chunks of partial[kc][m][n], chunks added in order
__global__ void __launch_bounds__(256) gemm_chunk_sum_kernel(const float* __restrict__ partial, int k_chunks, int M, int N,
                                                             const int* __restrict__ c_rows, float* __restrict__ c, int64_t ldc,
                                                             int accumulate)
{
    const int n = blockIdx.x * 256 + threadIdx.x;
    if (n >= N) return;
    for (int m = blockIdx.y; m < M; m += gridDim.y) {
        float* out = c + (int64_t)(c_rows ? c_rows[m] : m) * ldc + n;
        float s = accumulate ? *out : 0.f;
        for (int kc = 0; kc < k_chunks; ++kc) s += partial[((int64_t)kc * M + m) * N + n];
        *out = s;
    }
}

// the same, four columns per thread (N, ldc multiples of 4, c 16-byte aligned)
__global__ void __launch_bounds__(256) gemm_chunk_sum4_kernel(const float* __restrict__ partial, int k_chunks, int M, int N,
                                                              const int* __restrict__ c_rows, float* __restrict__ c, int64_t ldc,
                                                              int accumulate)
{
    const int n = (blockIdx.x * 256 + threadIdx.x) * 4;
    if (n >= N) return;
    for (int m = blockIdx.y; m < M; m += gridDim.y) {
        float4* out = reinterpret_cast<float4*>(c + (int64_t)(c_rows ? c_rows[m] : m) * ldc + n);
        float4 s = accumulate ? *out : float4{0.f, 0.f, 0.f, 0.f};
        for (int kc = 0; kc < k_chunks; ++kc) {
            const float4 v = *reinterpret_cast<const float4*>(partial + ((int64_t)kc * M + m) * N + n);
            s = float4{s.x + v.x, s.y + v.y, s.z + v.z, s.w + v.w};
        }
        *out = s;
    }
}

// c[row] (+)= the chunk sums of a launch whose K was cut into chunks
bool launch_chunk_sum(const GemmArgs& a, hipStream_t stream)
{
    const bool vec = (a.N & 3) == 0 && (a.ldc & 3) == 0 && (reinterpret_cast<uintptr_t>(a.c) & 15) == 0 &&
                     (reinterpret_cast<uintptr_t>(a.partial) & 15) == 0;
    if (vec)
        hipLaunchKernelGGL(gemm_chunk_sum4_kernel, dim3((a.N / 4 + 255) / 256, std::min(a.M, 65535)), dim3(256), 0, stream, a.partial,
                           a.k_chunks, a.M, a.N, a.c_rows, a.c, a.ldc, a.accumulate);
    else
        hipLaunchKernelGGL(gemm_chunk_sum_kernel, dim3((a.N + 255) / 256, std::min(a.M, 65535)), dim3(256), 0, stream, a.partial,
                           a.k_chunks, a.M, a.N, a.c_rows, a.c, a.ldc, a.accumulate);
    return hip_ok(hipGetLastError(), "gemm chunk sum launch");
}

template <typename G, int KTW>
bool launch_slim(GemmArgs a, int m_tiles, hipStream_t stream, const ChunkScratch& cs)
{
    using L = SlimLayout<G, KTW>;
    auto kern = gemm_slim_kernel<G, KTW>;
    const size_t lds = (size_t)8 * L::RING * L::BUF + 64;     // the unpackers may read a few bytes past the last row
    static_assert((size_t)8 * L::RING * L::BUF + 64 <= 160 * 1024, "raw buffers must fit LDS");
    if (!cs.need_out && !raise_lds_limit(reinterpret_cast<const void*>(kern), lds)) return false;
    a.m_tiles = m_tiles;
    a.n_tiles = (a.N + 31) / 32;
    a.chunk_kt = 8 * KTW;
    a.k_chunks = (a.Kp / kBK + a.chunk_kt - 1) / a.chunk_kt;
    a.partial = nullptr;
    const bool two_pass = a.k_chunks > 1 || a.accumulate;
    if (two_pass) {
        const size_t need = (size_t)a.k_chunks * a.M * a.N * sizeof(float);
        if (cs.need_out) *cs.need_out = need;
        a.partial = chunk_scratch(cs, need);
        if (!a.partial && !cs.need_out) {
            set_last_error("gemm: the K-chunk sums of this shape do not fit the scratch buffer.");
            return false;
        }
    }
    if (cs.need_out) return true;
    const int64_t units = (int64_t)m_tiles * a.k_chunks * a.n_tiles;
    const int grid = (int)std::min<int64_t>(units, device_info().num_cus);
    hipLaunchKernelGGL(kern, dim3(grid), dim3(512), lds, stream, a);
    if (!hip_ok(hipGetLastError(), "gemm launch")) return false;
    if (two_pass) {
        return launch_chunk_sum(a, stream);
    }
    return true;
}

// ------------------------------------------------------------------------------------------
// The register-resident kernel for MXFP4 on the block-scaled matrix instruction (see gemm_mx_kernel): the activations
// of the wavefront's K range stay in registers as MX fp6 pairs (12.5 registers per k-tile and 32-row block, where fp16
// operands take 16), the raw weight blocks of the ring buffers are the B operands as they are, and the pair of
// instructions per k-tile costs half of the four fp16 ones.  RB row blocks per unit: 1 is what the launcher uses.
// (RB = 2, 64-row units for the matrix time of one 32-row fp16 unit, so that an expert with 33 .. 64 tokens streams its
// weights once, is correct but no faster: its 8 KB of partial sums per wavefront leave room for a ring of two buffers
// only, and a unit's time is the wavefronts' LDS-direct copies and the two barriers, not the matrix instructions -
// 200.8 vs 200.6 us for the 256-token GPT-OSS expert stage.)
// ------------------------------------------------------------------------------------------
template <int KTW, int RB>
struct SlimMxLayout {
    static constexpr int kNeed = (GMXFP4::window_bytes(KTW) + 15) / 16;
    static constexpr int CH = kNeed | 1;                                 // odd: the 16-byte reads of 16 rows cover the banks once
    static constexpr int DI = (32 * CH + 63) / 64;
    static constexpr int RAW = 32 * CH * 16;
    static constexpr int BUF = RAW > RB * 4096 ? RAW : RB * 4096;        // raw rows, later RB x 32 x 32 fp32 partial sums
    static constexpr int RING = 8 * 3 * BUF + 1024 <= 160 * 1024 ? 3 : 2;
};

template <int KTW, int RB, int EPI>
__global__ void __launch_bounds__(512) gemm_slim_mx_kernel(const GemmArgs A)
{
    static_assert(EPI == 0 || RB == 1, "the fused epilogue takes 32-row units");
    typedef GMXFP4 G;
    using L = SlimMxLayout<KTW, RB>;
    constexpr int CH = L::CH, DI = L::DI, BUF = L::BUF, RING = L::RING;
    constexpr int DIE = DI + (EPI ? 1 : 0);                              // copies per tile: EPI adds the tile's 32 bias values
    constexpr int NQ = 2 * RB;                                          // results per thread in the reduction
    static_assert(KTW % G::kTileStep == 0, "a wavefront's K range must start at a block");
    typedef uint32_t uint2_t __attribute__((ext_vector_type(2)));
    extern __shared__ uint8_t smem[];                                   // 8 wavefronts x RING x BUF

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int col = lane & 31, h = lane >> 5;
    uint8_t* const my_buf = smem + wave * RING * BUF;
    float* const my_bias = reinterpret_cast<float*>(smem + 8 * RING * BUF) + wave * RING * 32;      // EPI: 32 floats per buffer

    const uint32_t row_bytes = (uint32_t)((int64_t)A.w_bytes / A.N);
    const int nkt = A.Kp / kBK;
    const int n32 = (A.N + 31) >> 5;
    const int per_tile = A.k_chunks * n32;                              // units of one row tile

    int live_tiles = A.m_tiles;
    if (A.tile_expert) {
        int c = 0;
        for (int i = lane; i < A.m_tiles; i += 64) c += A.tile_rows[i] > 0 ? 1 : 0;
        for (int o = 32; o > 0; o >>= 1) c += __shfl_xor(c, o);
        live_tiles = __builtin_amdgcn_readfirstlane(c);
    }
    const int64_t units = (int64_t)live_tiles * per_tile;
    int u = (int)(units * blockIdx.x / gridDim.x);
    int u_end = (int)(units * (blockIdx.x + 1) / gridDim.x);
    // EPI = 1, gate_up of the gpt-oss experts (N = 2 F, one K chunk, F / 32 whole column tiles): the units of a row tile
    // walk the column tiles as gate tile 0, up tile 0, gate tile 1, ... so that a workgroup holds both halves of a pair;
    // ranges start at pairs.  Unit j of the walk is column tile phys(j).
    if (EPI) {
        u &= ~1;
        u_end &= ~1;                                                   // units is even: every row tile has 2 x F / 32
    }
    auto phys = [&](int j) { return EPI ? (j >> 1) + (j & 1) * (n32 >> 1) : j; };

    while (u < u_end) {
        const int mt = u / per_tile, rem = u - mt * per_tile;
        const int kc = rem / n32, nt0 = rem - kc * n32, cnt = min(n32 - nt0, u_end - u);
        u += cnt;
        const int kt0 = kc * A.chunk_kt + wave * KTW;
        const int kcnt = max(0, min(KTW, nkt - kt0));                  // k-tiles of this wavefront in this chunk
        int m0, m_rows;
        const uint8_t* wbase = A.w;
        if (A.tile_expert) {
            m0 = A.tile_row0[mt];
            m_rows = min(32 * RB, A.tile_rows[mt]);
            wbase += expert_offset(A, mt);
        } else {
            m0 = mt * 32 * RB;
            m_rows = min(32 * RB, A.M - m0);
        }
        const int rbs = RB > 1 && m_rows > 32 ? RB : 1;                // row blocks with rows in them (uniform)
        // (the expert id comes from memory the kernel also writes to, so the compiler loads it per lane: without the
        // hint every copy would run in a loop over the distinct descriptors of the wavefront)
        const uintptr_t wa = uniform_address(reinterpret_cast<uintptr_t>(wbase));
        const uint32_t base_delta = (uint32_t)(wa & 3);
        const __amdgpu_buffer_rsrc_t wrs = __builtin_amdgcn_make_buffer_rsrc(
            reinterpret_cast<void*>(wa & ~(uintptr_t)3), 0, (int)(((uint32_t)A.w_bytes + base_delta + 3u) & ~3u), 0x00020000);

        // A operands of this wavefront's K range: row col + 32 rb, block h of every k-tile - the two 24-byte streams
        // and the scale dword (layout of convert_x_mx_kernel)
        uint4_t ah0[KTW][RB], al0[KTW][RB];
        uint2_t ah1[KTW][RB], al1[KTW][RB];
        uint32_t asa[KTW / 2][RB];                 // scale bytes (hi, lo) of k-tile 2 j in bytes 0, 1 and of 2 j + 1 in bytes 2, 3
        // (range-checked loads: rows past the tile and k-tiles past the wavefront's range read zeros - zero fields
        // under the smallest scale - without a select per register)
        const __amdgpu_buffer_rsrc_t xrs = __builtin_amdgcn_make_buffer_rsrc(const_cast<_Float16*>(A.x16), 0, (int)A.x16_bytes, 0x00020000);
        if (RB == 1 && m_rows > 16) {
            // (units of a few rows load them directly, further down: for them the pass through LDS is only a second latency)
            // Through the wavefront's (still empty) raw buffers: LDS-direct copies of whole row pieces (128 KTW contiguous
            // bytes per row, 16 rows per pass) and 16-byte LDS reads from there; loaded straight from memory, a lane per
            // row and K block, every 128-byte line was asked for in five separate pieces (see gemm_slim_mx48_kernel).
            constexpr int kRowPieces = KTW * 8 + 1;                     // one piece of padding spreads the rows over the banks
            constexpr int kPassCopies = (16 * kRowPieces + 63) / 64;
            static_assert(kPassCopies * 1024 <= RING * BUF, "a pass of 16 rows fits the ring");
            const uint32_t a_row = (uint32_t)(A.xld * 2);
#pragma unroll
            for (int pass = 0; pass < 2; ++pass) {
                // only the rows the unit has: an expert with two tokens copies two rows, and none in the second pass
                const int pass_rows = __builtin_amdgcn_readfirstlane(min(16, m_rows - 16 * pass));
                if (pass_rows <= 0) break;
                const int pass_copies = (pass_rows * kRowPieces + 63) >> 6;
#pragma unroll 1
                for (int c = 0; c < pass_copies; ++c) {
                    const int q = c * 64 + lane;
                    const int row = q / kRowPieces, piece = q - row * kRowPieces;
                    const int rl = 16 * pass + row;
                    const bool valid = row < pass_rows && piece < KTW * 8 && (piece >> 3) < kcnt;
                    copy16_to_lds(xrs, my_buf + c * 1024, valid ? (uint32_t)(m0 + rl) * a_row + (uint32_t)(kt0 * 128 + piece * 16) : kDeadOffset, 0u);
                }
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                // rows 0 .. 15 in the first pass (the upper lanes read along and are overwritten), 16 .. 31 in the second
                if (pass == 0 || col >= 16) {
#pragma unroll
                    for (int t = 0; t < KTW; ++t) {
                        const uint8_t* const kp = my_buf + (col & 15) * (kRowPieces * 16) + t * 128;
                        ah0[t][0] = *reinterpret_cast<const uint4_t*>(kp + (uint32_t)(2 * h) * 16u);
                        al0[t][0] = *reinterpret_cast<const uint4_t*>(kp + (uint32_t)(3 + 2 * h) * 16u);
                        ah1[t][0] = *reinterpret_cast<const uint2_t*>(kp + 16u + 8u * (uint32_t)h);
                        al1[t][0] = *reinterpret_cast<const uint2_t*>(kp + 64u + 8u * (uint32_t)h);
                        const uint32_t two = *reinterpret_cast<const uint32_t*>(kp + 96u + 4u * (uint32_t)h) & 0xffffu;
                        if (t & 1) asa[t >> 1][0] = (asa[t >> 1][0] & 0xffffu) | (two << 16);
                        else asa[t >> 1][0] = two;
                    }
                }
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");    // the reads are done: the buffers may be written again
            }
        } else {
    #pragma unroll
            for (int rb = 0; rb < RB; ++rb) {
                const int ml = col + 32 * rb;
                const uint32_t xrow = (uint32_t)(m0 + min(ml, m_rows - 1)) * (uint32_t)(A.xld * 2);
    #pragma unroll
                for (int t = 0; t < KTW; ++t) {
                    const bool on = ml < m_rows && t < kcnt;
                    const uint32_t xt = on ? xrow + (uint32_t)(kt0 + t) * 128u : kDeadOffset;
                    const uint4_t vh0 = __builtin_amdgcn_raw_buffer_load_b128(xrs, (int)(xt + (uint32_t)(2 * h) * 16u), 0, 0);
                    const uint4_t vl0 = __builtin_amdgcn_raw_buffer_load_b128(xrs, (int)(xt + (uint32_t)(3 + 2 * h) * 16u), 0, 0);
                    ah0[t][rb] = vh0;
                    al0[t][rb] = vl0;
                    ah1[t][rb] = __builtin_amdgcn_raw_buffer_load_b64(xrs, (int)(xt + 16u + 8u * (uint32_t)h), 0, 0);
                    al1[t][rb] = __builtin_amdgcn_raw_buffer_load_b64(xrs, (int)(xt + 64u + 8u * (uint32_t)h), 0, 0);
                    const uint32_t two = __builtin_amdgcn_raw_buffer_load_b32(xrs, (int)(xt + 96u + 4u * (uint32_t)h), 0, 0) & 0xffffu;
                    if (t & 1) asa[t >> 1][rb] |= two << 16;
                    else asa[t >> 1][rb] = two;
                }
            }
        }
        const uint32_t koff = G::tile_offset(kt0);
        uint32_t w_off[DI];
#pragma unroll
        for (int i = 0; i < DI; ++i) {
            const int q = i * 64 + lane;
            const int row = q / CH, chunk = q - row * CH;
            w_off[i] = (row < 32 && kcnt > 0) ? ((base_delta + (uint32_t)row * row_bytes + koff) & ~3u) + (uint32_t)chunk * 16u : kDeadOffset;
        }
        const uint32_t my_delta = (base_delta + (uint32_t)col * row_bytes + koff) & 3u;
        // EPI: the expert's [2 F] bias row (an empty range without a bias: the copies deliver zeros)
        const float* const eb = EPI && A.epi_bias ? A.epi_bias + (int64_t)(A.tile_expert ? A.tile_expert[mt] : 0) * A.N : nullptr;
        const uintptr_t ba = uniform_address(reinterpret_cast<uintptr_t>(eb));
        const __amdgpu_buffer_rsrc_t brs = __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>(ba & ~(uintptr_t)3), 0, ba ? A.N * 4 : 0, 0x00020000);
        const uint32_t bias_off = (uint32_t)lane * 16u;
        // copy q of column tile nt0 + i -> buffer b
        auto issue_one = [&](int i, int b, int q) {
            const bool any = i < cnt;
            const uint32_t so = any ? (uint32_t)phys(nt0 + i) * 32u * row_bytes : 0u;
            if (EPI && q == DI) {
                // the bias of the tile's 32 columns (zeros without one) comes the same way: a plain load would make the
                // compiler wait for every copy in flight before its value is used
                if (lane < 8) copy16_to_lds(brs, reinterpret_cast<uint8_t*>(my_bias + b * 32), any ? bias_off + (uint32_t)phys(nt0 + i) * 128u : kDeadOffset, 0u);
                return;
            }
            if (q * 64 + 32 < 32 * CH || lane < 32) copy16_to_lds(wrs, my_buf + b * BUF + q * 1024, any ? w_off[q] : kDeadOffset, so);
        };
        auto issue = [&](int i, int b) {
#pragma unroll
            for (int q = 0; q < DIE; ++q) issue_one(i, b, q);
        };
        // With three buffers the refill of a buffer waits for the NEXT unit and goes out copy by copy behind the matrix
        // instructions of its k-tiles (copy q behind k-tile q % KTW): a copy keeps the wavefront busy for tens of
        // cycles, and there the matrix pipe has work queued for that long.
        constexpr bool kDefer = RING >= 3;
        static_assert(EPI == 0 || (kDefer && BUF >= 32 * 144), "the fused epilogue stages a 32 x 32 tile in a buffer that is refilled a unit later");
        // results of this thread in the reduction: accumulator registers wave + 8 q of the RB x 16
        int64_t coff[NQ];
        bool ok[NQ];
#pragma unroll
        for (int q = 0; q < NQ; ++q) {
            const int rr = wave + 8 * q, r = rr & 15;
            const int ml = 32 * (rr >> 4) + 8 * (r >> 2) + 4 * h + (r & 3);
            const int m = m0 + min(ml, m_rows - 1);
            coff[q] = A.partial ? ((int64_t)kc * A.M + m) * A.N : (int64_t)(A.c_rows ? A.c_rows[m] : m) * A.ldc;
            ok[q] = ml < m_rows;
        }

#pragma unroll
        for (int b = 0; b < RING; ++b) issue(b, b);
        int b = 0;                                      // buffer of column tile i
        float pend[NQ];
#pragma unroll
        for (int q = 0; q < NQ; ++q) pend[q] = 0.f;
        int pend_n = -1;
        float* const dst = A.partial ? A.partial : A.c;
        float gate[NQ];                                 // EPI: the gate sums of the pair whose up tile is next
        int epi_blk = -1, epi_buf = 0;                  // EPI: the staged activation block that waits for its conversion
        auto flush = [&]() {
            if constexpr (EPI == 0) {
                if (pend_n >= 0 && pend_n < A.N) {
#pragma unroll
                    for (int q = 0; q < NQ; ++q)
                        if (ok[q]) dst[coff[q] + pend_n] = pend[q];
                }
            } else {
                // lane r of the last wavefront (whose K range is the one that may be short) converts row r of the staged
                // 32 x 32 activations into block epi_blk of the down projection's activation rows
                if (epi_blk >= 0 && wave == 7 && lane < m_rows && lane < 32) {
                    const float* const stage = reinterpret_cast<const float*>(smem + (7 * RING + epi_buf) * BUF) + lane * 36;
                    float16v_t va, vb;
#pragma unroll
                    for (int t = 0; t < 4; ++t) {
                        // (vector-typed reads: for reads through a struct type the compiler waits for every copy in flight)
                        const uint4_t fa = reinterpret_cast<const uint4_t*>(stage)[t], fb = reinterpret_cast<const uint4_t*>(stage)[4 + t];
                        va[4 * t] = __uint_as_float(fa.x), va[4 * t + 1] = __uint_as_float(fa.y), va[4 * t + 2] = __uint_as_float(fa.z), va[4 * t + 3] = __uint_as_float(fa.w);
                        vb[4 * t] = __uint_as_float(fb.x), vb[4 * t + 1] = __uint_as_float(fb.y), vb[4 * t + 2] = __uint_as_float(fb.z), vb[4 * t + 3] = __uint_as_float(fb.w);
                    }
                    uint8_t* const tile = A.epi_out + (int64_t)(m0 + lane) * A.epi_ld + (epi_blk >> 1) * 128;
                    mx_store_block(tile, epi_blk & 1, mx_encode_block(va, vb, true));
                    // the last block of an odd count: the other half of its k-tile lies past F
                    if (epi_blk + 1 == (n32 >> 1) && !(epi_blk & 1)) mx_store_block(tile, 1, mx_encode_block(va, vb, false));
                }
                epi_blk = -1;
            }
        };
        for (int i = 0; i < cnt; ++i) {
            // the copies of tile i have landed; those of the tiles after it stay in flight (deferred refills: the tile
            // RING - 1 on is only issued during this unit)
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"((kDefer ? RING - 2 : RING - 1) * DIE) : "memory");
            flush();
            const int b_prev = b == 0 ? RING - 1 : b - 1;      // the buffer of tile i - 1
            float16_t acc[RB];
#pragma unroll
            for (int rb = 0; rb < RB; ++rb)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[rb][r] = 0.f;
            const uint8_t* raw = my_buf + b * BUF + col * (CH * 16);
            // the raw block of k-tile t + 1 is fetched from LDS while k-tile t is multiplied; the fences keep the compiler
            // from fetching every k-tile up front (the A operands leave few registers)
            auto k_tiles = [&](auto full_tag) {
                constexpr bool kFull = decltype(full_tag)::value;
                // Block h of k-tile t starts my_delta + 17 (2 t + h) bytes into the row, i.e. s = my_delta + h + 2 t (< 16)
                // bytes into its 16-byte piece h + 2 t: two aligned 16-byte reads hold it (at the odd row stride sixteen
                // lanes cover all 64 banks once, where dword reads collide four ways).
                uint4_t r[KTW + 1][2];
                const uint8_t* const rawh = raw + 16 * h;
                auto fetch = [&](int t) {
                    r[t][0] = *reinterpret_cast<const uint4_t*>(rawh + 32 * t);
                    r[t][1] = *reinterpret_cast<const uint4_t*>(rawh + 32 * t + 16);
                };
                fetch(0);
#pragma unroll
                for (int t = 0; t < KTW; ++t) {
                    if (t + 1 < KTW) fetch(t + 1);
                    __builtin_amdgcn_sched_barrier(0);
                    if (kFull || t < kcnt) {
                        // the lane's raw block of k-tile t: sixteen bytes of nibbles re-aligned, and its scale byte
                        const uint32_t v[8] = {r[t][0].x, r[t][0].y, r[t][0].z, r[t][0].w, r[t][1].x, r[t][1].y, r[t][1].z, r[t][1].w};
                        const uint32_t sft = my_delta + (uint32_t)h + 2u * t;          // scale byte at sft, nibbles behind it
                        const int e0 = (2 * t) >> 2, d0 = (2 * t + 1) >> 2;            // the dwords they start in at the least
                        const uint32_t e = (((int)(sft >> 2) != e0 ? v[e0 + 1] : v[e0]) >> (8 * (sft & 3))) & 0xffu;
                        const bool up = (int)((sft + 1) >> 2) != d0;
                        const uint32_t b0 = up ? v[d0 + 1] : v[d0], b1 = up ? v[d0 + 2] : v[d0 + 1], b2 = up ? v[d0 + 3] : v[d0 + 2];
                        const uint32_t b3 = up ? v[d0 + 4] : v[d0 + 3], b4 = up ? v[d0 + 5 < 8 ? d0 + 5 : 7] : v[d0 + 4];
                        const uint32_t shb = (sft + 1) & 3;
                        const bool live = ((kt0 + t) * 2 + h) * 32 < A.K;
                        const int8v_t bq = {live ? (int)__builtin_amdgcn_alignbyte(b1, b0, shb) : 0, live ? (int)__builtin_amdgcn_alignbyte(b2, b1, shb) : 0,
                                            live ? (int)__builtin_amdgcn_alignbyte(b3, b2, shb) : 0, live ? (int)__builtin_amdgcn_alignbyte(b4, b3, shb) : 0,
                                            0, 0, 0, 0};
                        const int sbq = live ? (int)e : 127;
#pragma unroll
                        for (int rb = 0; rb < RB; ++rb) {
                            if (rb < rbs) {
                                const int8v_t ahi = {(int)ah0[t][rb].x, (int)ah0[t][rb].y, (int)ah0[t][rb].z, (int)ah0[t][rb].w,
                                                     (int)ah1[t][rb].x, (int)ah1[t][rb].y, 0, 0};
                                const int8v_t alo = {(int)al0[t][rb].x, (int)al0[t][rb].y, (int)al0[t][rb].z, (int)al0[t][rb].w,
                                                     (int)al1[t][rb].x, (int)al1[t][rb].y, 0, 0};
                                const int sa2 = (int)asa[t >> 1][rb];
                                if (t & 1) {
                                    acc[rb] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(ahi, bq, acc[rb], 2, 4, 2, sa2, 0, sbq);
                                    acc[rb] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(alo, bq, acc[rb], 2, 4, 3, sa2, 0, sbq);
                                } else {
                                    acc[rb] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(ahi, bq, acc[rb], 2, 4, 0, sa2, 0, sbq);
                                    acc[rb] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(alo, bq, acc[rb], 2, 4, 1, sa2, 0, sbq);
                                }
                            }
                        }
                    }
                    if (kDefer && i > 0) {
#pragma unroll
                        for (int q = t; q < DIE; q += KTW) issue_one(i - 1 + RING, b_prev, q);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            };
            if (kcnt == KTW) k_tiles(std::true_type{});
            else k_tiles(std::false_type{});
            // partial sums of this wavefront's K range -> the buffer it has just consumed
            float* part = reinterpret_cast<float*>(my_buf + b * BUF);
#pragma unroll
            for (int rb = 0; rb < RB; ++rb)
#pragma unroll
                for (int r = 0; r < 16; ++r) part[(rb * 16 + r) * 64 + lane] = acc[rb][r];
            lds_barrier();
            float s[NQ];
#pragma unroll
            for (int q = 0; q < NQ; ++q) s[q] = 0.f;
#pragma unroll
            for (int v = 0; v < 8; ++v) {
                const float* pv = reinterpret_cast<const float*>(smem + (v * RING + b) * BUF);
#pragma unroll
                for (int q = 0; q < NQ; ++q) s[q] += pv[(wave + 8 * q) * 64 + lane];
            }
#pragma unroll
            for (int q = 0; q < NQ; ++q) pend[q] = s[q];      // the row scale of this activation layout is one
            pend_n = (nt0 + i) * 32 + col;
            if constexpr (EPI == 1) {
                const int j = nt0 + i;
                if (j & 1) {
                    // bias + SwiGLU-OAI of this thread's (gate, up) sums: columns (j / 2) 32 + col of the F activations
                    const float bu = my_bias[b * 32 + col];
#pragma unroll
                    for (int q = 0; q < NQ; ++q) pend[q] = ok[q] ? swiglu_oai(gate[q], s[q] + bu, A.epi_alpha, A.epi_limit) : 0.f;
                } else {
                    const float bg = my_bias[b * 32 + col];
#pragma unroll
                    for (int q = 0; q < NQ; ++q) gate[q] = s[q] + bg;
                }
            }
            lds_barrier();                              // every partial sum has been read: the buffers may be refilled
            if constexpr (EPI == 1) {
                const int j = nt0 + i;
                if (j & 1) {
                    // The 32 x 32 activations are one MX block per row: they meet in the last wavefront's buffer of this
                    // tile (free until that wavefront refills it during the next unit), 144 bytes per row; flush() converts
                    // them at the top of the next unit, where its stores lie behind the wait for the copies.
                    float* const stage = reinterpret_cast<float*>(smem + (7 * RING + b) * BUF);
#pragma unroll
                    for (int q = 0; q < NQ; ++q) {
                        const int rr = wave + 8 * q, r = rr & 15;
                        stage[(8 * (r >> 2) + 4 * h + (r & 3)) * 36 + col] = pend[q];
                    }
                    lds_barrier();
                    epi_blk = j >> 1;
                    epi_buf = b;
                }
            }
            if (!kDefer) issue(i + RING, b);
            b = b + 1 == RING ? 0 : b + 1;
        }
        flush();
    }
}

// ------------------------------------------------------------------------------------------
// 48-row units of the register-resident MX kernel, on v_mfma_scale_f32_16x16x128_f8f6f4 (lane = index + 16 g holds the
// 32 values of K block g of the 128; results: column = lane & 15, rows 4 (lane >> 4) + 0 .. 3 - probed on the device
// like the 32 x 32 x 64 form).  Three row blocks and two column blocks of 16 per unit: the A operands of 48 rows over a
// wavefront's six k-tiles take 114 registers where 64 rows of the 32 x 32 form would take 150, and 24 accumulators
// make 6 KB of partial sums per wavefront, which fit the raw buffer they replace.  With 32 experts and four of them
// per token, 256 tokens give an expert 32 rows on average and more than 48 almost never: nearly every expert streams
// its weights once, where 32-row units stream those of every second expert twice.
// One K chunk (K <= 3072); tiles, copies, ring and reduction as in gemm_slim_mx_kernel.  EPI = 1 (gate_up of the
// gpt-oss experts, column tiles walked in (gate, up) pairs): the result is bias + SwiGLU-OAI of each pair, an
// [M x F] fp32 matrix - half the bytes of the [M x 2 F] sums - which convert_x_mx_kernel then turns into the down
// projection's activations (the conversion inside the epilogue, as the 32-row kernel has it, does not fit the
// registers beside the A operands of 48 rows).
// ------------------------------------------------------------------------------------------
template <int EPI>
__global__ void __launch_bounds__(512) gemm_slim_mx48_kernel(const GemmArgs A)
{
    typedef GMXFP4 G;
    constexpr int KTW = 6, KG = 3;                                      // k-tiles and 128-wide K groups per wavefront
    using L = SlimMxLayout<KTW, 1>;
    constexpr int CH = L::CH, DI = L::DI, BUF = L::BUF, RING = L::RING;
    constexpr int DIE = DI + (EPI ? 1 : 0);
    constexpr int NQ = 3;                                               // results per thread in the reduction
    static_assert(RING == 3 && BUF >= 24 * 256, "the partial sums replace a raw buffer");
    typedef uint32_t uint2_t __attribute__((ext_vector_type(2)));
    typedef float float4v_t __attribute__((ext_vector_type(4)));
    extern __shared__ uint8_t smem[];                                   // 8 wavefronts x RING x BUF (+ EPI: bias values)

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int idx = lane & 15, g = lane >> 4;
    uint8_t* const my_buf = smem + wave * RING * BUF;
    float* const my_bias = reinterpret_cast<float*>(smem + 8 * RING * BUF) + wave * RING * 32;

    const uint32_t row_bytes = (uint32_t)((int64_t)A.w_bytes / A.N);
    const int nkt = A.Kp / kBK;
    const int n32 = (A.N + 31) >> 5;

    int live_tiles = A.m_tiles;
    if (A.tile_expert) {
        int c = 0;
        for (int i = lane; i < A.m_tiles; i += 64) c += A.tile_rows[i] > 0 ? 1 : 0;
        for (int o = 32; o > 0; o >>= 1) c += __shfl_xor(c, o);
        live_tiles = __builtin_amdgcn_readfirstlane(c);
    }
    const int64_t units = (int64_t)live_tiles * n32;
    int u = (int)(units * blockIdx.x / gridDim.x);
    int u_end = (int)(units * (blockIdx.x + 1) / gridDim.x);
    if (EPI) {                                                          // pairs of (gate, up) column tiles, see gemm_slim_mx_kernel
        u &= ~1;
        u_end &= ~1;
    }
    auto phys = [&](int j) { return EPI ? (j >> 1) + (j & 1) * (n32 >> 1) : j; };

    while (u < u_end) {
        const int mt = u / n32, nt0 = u - mt * n32, cnt = min(n32 - nt0, u_end - u);
        u += cnt;
        const int kt0 = wave * KTW;
        const int kcnt = max(0, min(KTW, nkt - kt0));                  // k-tiles of this wavefront
        int m0, m_rows;
        const uint8_t* wbase = A.w;
        if (A.tile_expert) {
            m0 = A.tile_row0[mt];
            m_rows = min(48, A.tile_rows[mt]);
            wbase += expert_offset(A, mt);
        } else {
            m0 = mt * 48;
            m_rows = min(48, A.M - m0);
        }
        const uintptr_t wa = uniform_address(reinterpret_cast<uintptr_t>(wbase));
        const uint32_t base_delta = (uint32_t)(wa & 3);
        const __amdgpu_buffer_rsrc_t wrs = __builtin_amdgcn_make_buffer_rsrc(
            reinterpret_cast<void*>(wa & ~(uintptr_t)3), 0, (int)(((uint32_t)A.w_bytes + base_delta + 3u) & ~3u), 0x00020000);

        // A operands: row idx + 16 rb, K block 4 T + g of the wavefront's range = half g & 1 of its k-tile 2 T + g / 2
        uint4_t ah0[KG][3], al0[KG][3];
        uint2_t ah1[KG][3], al1[KG][3];
        uint32_t asa[2][3];                        // scale bytes (hi, lo): group 0 in bytes 0, 1 and group 1 in bytes 2, 3 of [0], group 2 in [1]
        const __amdgpu_buffer_rsrc_t xrs = __builtin_amdgcn_make_buffer_rsrc(const_cast<_Float16*>(A.x16), 0, (int)A.x16_bytes, 0x00020000);
        const uint32_t hh = (uint32_t)(g & 1);
        // They reach the registers through the wavefront's (still empty) raw buffers: LDS-direct copies of whole row
        // pieces - 768 contiguous bytes per row, one row block of 16 rows per pass - and 16-byte LDS reads from there.
        // Loading them straight from memory (a lane per row and K block, 45 instructions of scattered 16-byte pieces
        // per wavefront) took 10 us of a launch: every CU asked the L2 for five pieces of each 128-byte line separately.
        {
            constexpr int kRowPieces = KTW * 8 + 1;                     // 49: one piece of padding spreads the rows over the banks
            constexpr int kPassCopies = (16 * kRowPieces + 63) / 64;    // 13
            static_assert(kPassCopies * 1024 <= RING * BUF, "a pass of 16 rows fits the ring");
            const uint32_t a_row = (uint32_t)(A.xld * 2);
#pragma unroll
            for (int rb = 0; rb < 3; ++rb) {
#pragma unroll 1
                for (int c = 0; c < kPassCopies; ++c) {             // a loop: unrolled, its 39 offsets would all be live at once
                    const int q = c * 64 + lane;
                    const int row = q / kRowPieces, piece = q - row * kRowPieces;
                    const int rl = 16 * rb + row;
                    const bool valid = row < 16 && piece < KTW * 8 && rl < m_rows && (piece >> 3) < kcnt;
                    copy16_to_lds(xrs, my_buf + c * 1024, valid ? (uint32_t)(m0 + rl) * a_row + (uint32_t)(kt0 * 128 + piece * 16) : kDeadOffset, 0u);
                }
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
                for (int T = 0; T < KG; ++T) {
                    const uint8_t* const kp = my_buf + idx * (kRowPieces * 16) + (2 * T + (g >> 1)) * 128;
                    ah0[T][rb] = *reinterpret_cast<const uint4_t*>(kp + 2u * hh * 16u);
                    al0[T][rb] = *reinterpret_cast<const uint4_t*>(kp + (3u + 2u * hh) * 16u);
                    ah1[T][rb] = *reinterpret_cast<const uint2_t*>(kp + 16u + 8u * hh);
                    al1[T][rb] = *reinterpret_cast<const uint2_t*>(kp + 64u + 8u * hh);
                    const uint32_t two = *reinterpret_cast<const uint32_t*>(kp + 96u + 4u * hh) & 0xffffu;
                    if (T == 0) asa[0][rb] = two;
                    else if (T == 1) asa[0][rb] |= two << 16;
                    else asa[1][rb] = two;
                }
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");    // the reads are done: the buffers may be written again
            }
        }
        const uint32_t koff = G::tile_offset(kt0);
        uint32_t w_off[DI];
#pragma unroll
        for (int i = 0; i < DI; ++i) {
            const int q = i * 64 + lane;
            const int row = q / CH, chunk = q - row * CH;
            w_off[i] = (row < 32 && kcnt > 0) ? ((base_delta + (uint32_t)row * row_bytes + koff) & ~3u) + (uint32_t)chunk * 16u : kDeadOffset;
        }
        // where the raw rows of this lane's two columns (idx, 16 + idx) start inside their windows
        uint32_t my_delta[2];
#pragma unroll
        for (int cb = 0; cb < 2; ++cb) my_delta[cb] = (base_delta + (uint32_t)(16 * cb + idx) * row_bytes + koff) & 3u;
        const float* const eb = EPI && A.epi_bias ? A.epi_bias + (int64_t)(A.tile_expert ? A.tile_expert[mt] : 0) * A.N : nullptr;
        const uintptr_t ba = uniform_address(reinterpret_cast<uintptr_t>(eb));
        const __amdgpu_buffer_rsrc_t brs = __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>(ba & ~(uintptr_t)3), 0, ba ? A.N * 4 : 0, 0x00020000);
        const uint32_t bias_off = (uint32_t)lane * 16u;
        auto issue_one = [&](int i, int b, int q) {
            const bool any = i < cnt;
            const uint32_t so = any ? (uint32_t)phys(nt0 + i) * 32u * row_bytes : 0u;
            if (EPI && q == DI) {
                if (lane < 8) copy16_to_lds(brs, reinterpret_cast<uint8_t*>(my_bias + b * 32), any ? bias_off + (uint32_t)phys(nt0 + i) * 128u : kDeadOffset, 0u);
                return;
            }
            if (q * 64 + 32 < 32 * CH || lane < 32) copy16_to_lds(wrs, my_buf + b * BUF + q * 1024, any ? w_off[q] : kDeadOffset, so);
        };
        auto issue = [&](int i, int b) {
#pragma unroll
            for (int q = 0; q < DIE; ++q) issue_one(i, b, q);
        };
        // results of this thread in the reduction: accumulator registers a = wave + 8 q of the 24 -
        // a = (4 (2 rb + cb) + r): row 16 rb + 4 g + r, column 16 cb + idx
        int64_t coff[NQ];
        int ncol[NQ], mloc[NQ];
        bool ok[NQ];
#pragma unroll
        for (int q = 0; q < NQ; ++q) {
            const int a = wave + 8 * q;
            mloc[q] = 16 * (a >> 3) + 4 * g + (a & 3);
            ncol[q] = 16 * ((a >> 2) & 1) + idx;
            const int m = m0 + min(mloc[q], m_rows - 1);
            coff[q] = (int64_t)(A.c_rows ? A.c_rows[m] : m) * A.ldc;
            ok[q] = mloc[q] < m_rows;
        }

#pragma unroll
        for (int b = 0; b < RING; ++b) issue(b, b);
        int b = 0;                                      // buffer of column tile i
        float pend[NQ], gate[NQ];
#pragma unroll
        for (int q = 0; q < NQ; ++q) pend[q] = gate[q] = 0.f;
        int pend_n0 = -1;
        const int width = EPI ? A.N >> 1 : A.N;         // columns of the result
        auto flush = [&]() {
            if (pend_n0 >= 0) {
#pragma unroll
                for (int q = 0; q < NQ; ++q)
                    if (ok[q] && pend_n0 + ncol[q] < width) A.c[coff[q] + pend_n0 + ncol[q]] = pend[q];
            }
        };
        for (int i = 0; i < cnt; ++i) {
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"((RING - 2) * DIE) : "memory");
            flush();
            const int b_prev = b == 0 ? RING - 1 : b - 1;      // the buffer of tile i - 1
            float4v_t acc[3][2];
#pragma unroll
            for (int rb = 0; rb < 3; ++rb)
#pragma unroll
                for (int cb = 0; cb < 2; ++cb) acc[rb][cb] = float4v_t{0.f, 0.f, 0.f, 0.f};
            const uint8_t* const raw = my_buf + b * BUF + idx * (CH * 16) + 16 * g;
#pragma unroll
            for (int T = 0; T < KG; ++T) {
                if (2 * T < kcnt) {
                    // Block 4 T + g of raw row 16 cb + idx starts s = my_delta + 4 T + g (< 16) bytes into its 16-byte
                    // piece 4 T + g: two aligned 16-byte reads hold it.
                    int8v_t bq[2];
                    int sbq[2];
#pragma unroll
                    for (int cb = 0; cb < 2; ++cb) {
                        const uint8_t* const rp = raw + cb * 16 * (CH * 16) + 64 * T;
                        const uint4_t r0 = *reinterpret_cast<const uint4_t*>(rp), r1 = *reinterpret_cast<const uint4_t*>(rp + 16);
                        const uint32_t v[8] = {r0.x, r0.y, r0.z, r0.w, r1.x, r1.y, r1.z, r1.w};
                        const uint32_t sft = my_delta[cb] + (uint32_t)g + 4u * T;       // scale byte at sft, nibbles behind it
                        const uint32_t e = (((int)(sft >> 2) != T ? v[T + 1] : v[T]) >> (8 * (sft & 3))) & 0xffu;
                        const bool up = (int)((sft + 1) >> 2) != T;
                        const uint32_t b0 = up ? v[T + 1] : v[T], b1 = up ? v[T + 2] : v[T + 1], b2 = up ? v[T + 3] : v[T + 2];
                        const uint32_t b3 = up ? v[T + 4] : v[T + 3], b4 = up ? v[T + 5] : v[T + 4];
                        const uint32_t shb = (sft + 1) & 3;
                        // a block of a k-tile past the wavefront's range or past K: zeros under a scale of one
                        const bool live = 2 * T + (g >> 1) < kcnt && ((kt0 * 2 + 4 * T + g) * 32 < A.K);
                        bq[cb] = int8v_t{live ? (int)__builtin_amdgcn_alignbyte(b1, b0, shb) : 0, live ? (int)__builtin_amdgcn_alignbyte(b2, b1, shb) : 0,
                                         live ? (int)__builtin_amdgcn_alignbyte(b3, b2, shb) : 0, live ? (int)__builtin_amdgcn_alignbyte(b4, b3, shb) : 0,
                                         0, 0, 0, 0};
                        sbq[cb] = live ? (int)e : 127;
                    }
#pragma unroll
                    for (int rb = 0; rb < 3; ++rb) {
                        if (16 * rb >= m_rows) continue;              // a row block without rows (uniform)
                        const int8v_t ahi = {(int)ah0[T][rb].x, (int)ah0[T][rb].y, (int)ah0[T][rb].z, (int)ah0[T][rb].w,
                                             (int)ah1[T][rb].x, (int)ah1[T][rb].y, 0, 0};
                        const int8v_t alo = {(int)al0[T][rb].x, (int)al0[T][rb].y, (int)al0[T][rb].z, (int)al0[T][rb].w,
                                             (int)al1[T][rb].x, (int)al1[T][rb].y, 0, 0};
                        const int sa2 = (int)asa[T >> 1][rb];
#pragma unroll
                        for (int cb = 0; cb < 2; ++cb) {
                            if (T == 1) {
                                acc[rb][cb] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(ahi, bq[cb], acc[rb][cb], 2, 4, 2, sa2, 0, sbq[cb]);
                                acc[rb][cb] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(alo, bq[cb], acc[rb][cb], 2, 4, 3, sa2, 0, sbq[cb]);
                            } else {
                                acc[rb][cb] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(ahi, bq[cb], acc[rb][cb], 2, 4, 0, sa2, 0, sbq[cb]);
                                acc[rb][cb] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(alo, bq[cb], acc[rb][cb], 2, 4, 1, sa2, 0, sbq[cb]);
                            }
                        }
                    }
                }
                // the refill of the buffer of tile i - 1, copy by copy behind the groups (see gemm_slim_mx_kernel)
                if (i > 0) {
#pragma unroll
                    for (int q = T; q < DIE; q += KG) issue_one(i - 1 + RING, b_prev, q);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            // partial sums of this wavefront's K range -> the buffer it has just consumed
            float* part = reinterpret_cast<float*>(my_buf + b * BUF);
#pragma unroll
            for (int rb = 0; rb < 3; ++rb)
#pragma unroll
                for (int cb = 0; cb < 2; ++cb)
#pragma unroll
                    for (int r = 0; r < 4; ++r) part[(4 * (2 * rb + cb) + r) * 64 + lane] = acc[rb][cb][r];
            lds_barrier();
            float s[NQ];
#pragma unroll
            for (int q = 0; q < NQ; ++q) s[q] = 0.f;
#pragma unroll
            for (int v = 0; v < 8; ++v) {
                const float* pv = reinterpret_cast<const float*>(smem + (v * RING + b) * BUF);
#pragma unroll
                for (int q = 0; q < NQ; ++q) s[q] += pv[(wave + 8 * q) * 64 + lane];
            }
#pragma unroll
            for (int q = 0; q < NQ; ++q) pend[q] = s[q];      // the row scale of this activation layout is one
            pend_n0 = EPI ? ((nt0 + i) & 1 ? ((nt0 + i) >> 1) * 32 : -1) : (nt0 + i) * 32;      // EPI: a pair's activations after its up tile
            if constexpr (EPI == 1) {
                const int j = nt0 + i;
                if (j & 1) {
#pragma unroll
                    for (int q = 0; q < NQ; ++q)
                        pend[q] = ok[q] ? swiglu_oai(gate[q], s[q] + my_bias[b * 32 + ncol[q]], A.epi_alpha, A.epi_limit) : 0.f;
                } else {
#pragma unroll
                    for (int q = 0; q < NQ; ++q) gate[q] = s[q] + my_bias[b * 32 + ncol[q]];
                }
            }
            lds_barrier();                              // every partial sum has been read: the buffers may be refilled
            b = b + 1 == RING ? 0 : b + 1;
        }
        flush();
    }
}

template <int KTW, int RB, int EPI = 0>
bool launch_slim_mx(GemmArgs a, int m_tiles, hipStream_t stream, const ChunkScratch& cs)
{
    using L = SlimMxLayout<KTW, RB>;
    auto kern = gemm_slim_mx_kernel<KTW, RB, EPI>;
    constexpr size_t lds = (size_t)8 * L::RING * L::BUF + (EPI ? 8 * L::RING * 128 : 64);      // EPI: 32 bias values per buffer
    static_assert(lds <= 160 * 1024, "raw buffers must fit LDS");
    if (!cs.need_out && !raise_lds_limit(reinterpret_cast<const void*>(kern), lds)) return false;
    a.m_tiles = m_tiles;
    a.n_tiles = (a.N + 31) / 32;
    a.chunk_kt = 8 * KTW;
    a.k_chunks = (a.Kp / kBK + a.chunk_kt - 1) / a.chunk_kt;
    a.partial = nullptr;
    const bool two_pass = a.k_chunks > 1 || a.accumulate;
    if (EPI && (two_pass || (a.N & 63) || a.M <= 0)) {
        set_last_error("gemm: the fused SwiGLU epilogue takes one K chunk and whole 32-column tiles of gate and of up.");
        return false;
    }
    if (two_pass) {
        const size_t need = (size_t)a.k_chunks * a.M * a.N * sizeof(float);
        if (cs.need_out) *cs.need_out = need;
        a.partial = chunk_scratch(cs, need);
        if (!a.partial && !cs.need_out) {
            set_last_error("gemm: the K-chunk sums of this shape do not fit the scratch buffer.");
            return false;
        }
    }
    if (cs.need_out) return true;
    const int64_t units = (int64_t)m_tiles * a.k_chunks * a.n_tiles;
    const int grid = (int)std::min<int64_t>(units, device_info().num_cus);
    hipLaunchKernelGGL(kern, dim3(grid), dim3(512), lds, stream, a);
    if (!hip_ok(hipGetLastError(), "gemm launch")) return false;
    if (two_pass) {
        return launch_chunk_sum(a, stream);
    }
    return true;
}

// k-tiles per wavefront of the MX register-resident kernel: 2, 4 or 6 (75 registers of A operands at 6), a longer K in
// chunks
template <int RB>
bool launch_slim_mx_for(const GemmArgs& a, int m_tiles, hipStream_t stream, const ChunkScratch& cs)
{
    const int need = (a.Kp / kBK + 7) / 8;
    if (need <= 2) return launch_slim_mx<2, RB>(a, m_tiles, stream, cs);
    if (need <= 4) return launch_slim_mx<4, RB>(a, m_tiles, stream, cs);
    return launch_slim_mx<6, RB>(a, m_tiles, stream, cs);
}

// k-tiles per wavefront of the register-resident kernel: a multiple of the format's block step, at most what two
// raw buffers per wavefront fit into LDS; a longer K is cut into chunks of 8 x that many k-tiles
template <typename G, int KTW>
constexpr bool slim_fits()
{
    return (size_t)8 * SlimLayout<G, KTW>::RING * SlimLayout<G, KTW>::BUF + 64 <= 160 * 1024;
}

template <typename G>
int slim_ktw(int nkt)
{
    const int need = (nkt + 7) / 8;
    const int ktw = (need + G::kTileStep - 1) / G::kTileStep * G::kTileStep;
    const int limit = slim_fits<G, 8>() ? 8 : slim_fits<G, 6>() && G::kTileStep == 2 ? 6 : 4;
    return ktw <= limit ? ktw : limit;       // longer K: chunks of 8 * limit k-tiles
}

template <typename G>
bool launch_slim_for(const GemmArgs& a, int ktw, int m_tiles, hipStream_t stream, const ChunkScratch& cs)
{
    if constexpr (G::kTileStep == 2) {
        if (ktw == 2) return launch_slim<G, 2>(a, m_tiles, stream, cs);
        if constexpr (slim_fits<G, 6>())
            if (ktw == 6) return launch_slim<G, 6>(a, m_tiles, stream, cs);
    }
    if (ktw == 4) return launch_slim<G, 4>(a, m_tiles, stream, cs);
    if constexpr (slim_fits<G, 8>())
        if (ktw == 8) return launch_slim<G, 8>(a, m_tiles, stream, cs);
    set_last_error("gemm: no register-resident kernel for this K.");
    return false;
}

// 128-row tiles are 128 x 256 (one workgroup per CU) for these formats, 128 x 128 (two per CU) for the others
template <typename G>
constexpr bool kWide128 = G::kSup == 2 || G::kRawRow > 144 || std::is_same<G, GQ4K>::value;

// 48-row units (gemm_slim_mx48_kernel): one K chunk
template <int EPI>
bool launch_slim_mx48(GemmArgs a, int m_tiles, hipStream_t stream, const ChunkScratch& cs)
{
    using L = SlimMxLayout<6, 1>;
    auto kern = gemm_slim_mx48_kernel<EPI>;
    constexpr size_t lds = (size_t)8 * L::RING * L::BUF + (EPI ? 8 * L::RING * 128 : 64);
    static_assert(lds <= 160 * 1024, "raw buffers must fit LDS");
    if (a.Kp / kBK > 48 || a.accumulate || (EPI && (a.N & 63))) {
        set_last_error("gemm: 48-row units take K <= 3072, no accumulation and, with the fused epilogue, whole column tiles.");
        return false;
    }
    if (cs.need_out) {
        *cs.need_out = 0;
        return true;
    }
    if (!raise_lds_limit(reinterpret_cast<const void*>(kern), lds)) return false;
    a.m_tiles = m_tiles;
    a.n_tiles = (a.N + 31) / 32;
    a.chunk_kt = 48;
    a.k_chunks = 1;
    a.partial = nullptr;
    const int64_t units = (int64_t)m_tiles * a.n_tiles;
    const int grid = (int)std::min<int64_t>(units, device_info().num_cus);
    hipLaunchKernelGGL(kern, dim3(grid), dim3(512), lds, stream, a);
    return hip_ok(hipGetLastError(), "gemm launch");
}

template <typename G>
bool launch_for_type(const GemmArgs& a, int bm, int m_tiles, hipStream_t stream, const ChunkScratch& cs)
{
    if (bm == 32 && !a.x_mx) return launch_slim_for<G>(a, slim_ktw<G>(a.Kp / kBK), m_tiles, stream, cs);
    // Q4_K and MXFP4: the 2 x 4 wavefront layout with the operand exchange through LDS (gemm_xw_kernel); 128-row tiles are
    // 128 x 256.  Q4_K takes it for every launch, MXFP4 for plain ones: the MXFP4 expert tiles of a MoE prefill (128
    // rows) stay on two 128 x 128 workgroups per CU (926 vs 968 us at 2048 tokens).
    if constexpr (std::is_same<G, GQ4K>::value) {
        if (bm == 256) return launch_xw<PQ4K, 256, 4>(a, m_tiles, stream, cs);
        if (bm == 128) return launch_xw<PQ4K, 128, 4>(a, m_tiles, stream, cs);
    } else if constexpr (std::is_same<G, GMXFP4>::value) {
        if (a.x_mx) {
            if (bm == 256 && !a.tile_expert) return launch_mx<256>(a, m_tiles, stream, cs);
            if (bm == 128 && !a.tile_expert) return launch_mx<128>(a, m_tiles, stream, cs);
            // a plain small batch whose K fits one chunk, in 48-row units where those are at most two thirds as many as
            // 32-row units (33 .. 48, 65 .. 96, 129 .. 144 rows): a unit less is a pass less over the weights, and a 48-row
            // pass costs a little more than a 32-row one (32 x 184320 x 2880 65 us; 48 rows 77 instead of 97, 96 rows 132
            // instead of 164, but 128 rows 208 instead of 186)
            if (bm == 32 && !a.tile_expert && !a.accumulate && a.Kp / kBK <= 48 && 3 * ((a.M + 47) / 48) <= 2 * ((a.M + 31) / 32))
                return launch_slim_mx48<0>(a, (a.M + 47) / 48, stream, cs);
            if (bm == 32) return launch_slim_mx_for<1>(a, m_tiles, stream, cs);
            if (bm == 48) return launch_slim_mx48<0>(a, m_tiles, stream, cs);
            set_last_error("gemm: the MX activation layout serves 32- and 48-row units and plain launches of 128- and 256-row tiles.");
            return false;
        }
        if (bm == 256 && !a.tile_expert) return launch_xw<PMXFP4, 256, 4>(a, m_tiles, stream, cs);
        if (bm == 128 && !a.tile_expert) return launch_xw<PMXFP4, 128, 4>(a, m_tiles, stream, cs);
        if (bm == 128) return launch_tiles<G, 128, 2, 4>(a, m_tiles, stream, cs);
    } else {
        if constexpr (2 * 256 * kXRow + 2 * 256 * G::kRawRow + 1024 <= 160 * 1024) {
            if (bm == 256) return launch_tiles<G, 256, 2, 8>(a, m_tiles, stream, cs);
        }
        // 128-row tiles: for the 4-bit formats two independent 128 x 128 workgroups per CU (their copy, LDS and
        // matrix phases overlap) measured faster than one 128 x 256 workgroup; Q8_0 and Q6_K the other way round
        if (bm == 128)
            return kWide128<G> ? launch_tiles<G, 128, 2, 8>(a, m_tiles, stream, cs)
                               : launch_tiles<G, 128, 2, 4>(a, m_tiles, stream, cs);
    }
    set_last_error("gemm: unsupported tile height.");
    return false;
}

}  // namespace

namespace {
// Halfs between two rows of converted activations: the row length padded to whole k-tiles.  (Padding the stride by a
// cache line or more, so that rows at an even number of 128-byte lines apart would not share L2 channels, changed no
// GEMM time: 0, 128, 256, 384 and 2176 bytes measured alike.)
int x_row_halfs(int K) { return (K + kBK - 1) / kBK * kBK; }
}  // namespace

size_t gemm_workspace_bytes(int M, int K)
{
    return (size_t)M * x_row_halfs(K) * sizeof(_Float16) + (((size_t)M * sizeof(float) + 255) & ~(size_t)255) + 256;
}

// Rows of activations per tile for a plain (ungrouped) launch.  The 32-row register-resident kernel streams the
// weights once per 32 rows, but at a much higher rate than the LDS-tiled kernels and mostly out of the memory-side
// cache, so it wins well past 32 rows (measured crossovers: 4-bit formats about 128 rows, or up to 512 when the
// big tiles would leave CUs idle; Q8_0 about 64; Q6_K, whose big tiles are limited to 128 rows, about 256).
namespace {
bool wide_128_row_tiles(int type)
{
    switch (type) {
    case kTypeQ4_K: return kWide128<GQ4K>;
    case kTypeMXFP4: return true;      // plain launches: gemm_xw_kernel's 128 x 256 tiles
    case kTypeQ8_0: return kWide128<GQ80>;
    case kTypeQ6_K: return kWide128<GQ6K>;
    case kTypeQ5_K: return kWide128<GQ5K>;
    case kTypeQ4_0: return kWide128<GLegacy<kTypeQ4_0>>;
    case kTypeQ4_1: return kWide128<GLegacy<kTypeQ4_1>>;
    case kTypeQ5_0: return kWide128<GLegacy<kTypeQ5_0>>;
    case kTypeQ5_1: return kWide128<GLegacy<kTypeQ5_1>>;
    default: return kWide128<GLegacy<kTypeIQ4_NL>>;
    }
}
}  // namespace

int gemm_tile_m(int type, int M, int N)
{
    const int slim_rows = type == kTypeQ8_0 ? 64 : type == kTypeQ6_K ? 256 : 128;
    if (M <= slim_rows) return 32;
    if ((type == kTypeQ4_K || type == kTypeMXFP4) && M <= 512 && ((M + 127) / 128) * ((N + 127) / 128) <= 128) return 32;
    // the 128 x 256 tiles of the other formats: up to 128 rows when they would be very few (Q8_0 128 x 4096 x 4096: 48 -> 27 us)
    if (wide_128_row_tiles(type) && M <= 128 && ((M + 127) / 128) * ((N + 255) / 256) <= 32) return 32;
    // 128- or 256-row tiles by rounds of workgroups x time per k-tile of a round (measured per k-tile: a 256 x 256 tile
    // 2.0 us; two co-resident 128 x 128 tiles of the 4-bit formats 1.37 us; one 128 x 256 tile of the other formats
    // 1.4 us).  The model reproduces the measured crossovers (Q4_K, us, 128 / 256 rows): 1024 x 14336 x 4096 196 / 160,
    // 512 x 28672 x 4096 191 / 158, 600 x 21504 x 5376 221 / 198, 512 x 14336 x 4096 94 / 105, MXFP4 512 x 5760 x 2880
    // 52 / 88.
    const int cus = device_info().num_cus;
    const bool two_per_cu = !wide_128_row_tiles(type);                    // 128 x 128 tiles, two workgroups per CU
    const int64_t tiles256 = (int64_t)((M + 255) / 256) * ((N + 255) / 256);
    const int64_t tiles128 = (int64_t)((M + 127) / 128) * ((N + (two_per_cu ? 127 : 255)) / (two_per_cu ? 128 : 256));
    const double t256 = (double)((tiles256 + cus - 1) / cus) * 2.0;
    const double t128 = (double)((tiles128 + (two_per_cu ? 2 : 1) * cus - 1) / ((two_per_cu ? 2 : 1) * cus)) * (two_per_cu ? 1.37 : 1.4);
    return t256 < t128 ? 256 : 128;
}

namespace {

template <int TYPE, int SRC>
void launch_convert_typed(const ConvertSrc& src, int M, int K, int kp, _Float16* x16, float* scales, hipStream_t stream)
{
    const int ldo = x_row_halfs(K);
    // short rows: 256 threads hold the whole row and eight workgroups share a CU
    if (K <= 256 * kCvtHold * 4)
        hipLaunchKernelGGL((convert_x_kernel<TYPE, 256, SRC>), dim3(M), dim3(256), 0, stream, src, K, kp, ldo, x16, scales);
    else
        hipLaunchKernelGGL((convert_x_kernel<TYPE, 1024, SRC>), dim3(M), dim3(1024), 0, stream, src, K, kp, ldo, x16, scales);
}

template <int SRC>
bool launch_convert(int type, const ConvertSrc& src, int M, int K, void* workspace, hipStream_t stream, int layout = 0)
{
    const int kp = (K + kBK - 1) / kBK * kBK;
    float* scales = static_cast<float*>(workspace);
    _Float16* x16 = reinterpret_cast<_Float16*>(static_cast<char*>(workspace) + (((size_t)M * sizeof(float) + 255) & ~(size_t)255));
    if (layout == 1) {
        if (type != kTypeMXFP4) {
            set_last_error("gemm: the MX activation layout is for MXFP4 weights.");
            return false;
        }
        const int chunks = (kp / 32 + kMxCvtBlocks - 1) / kMxCvtBlocks;
        hipLaunchKernelGGL((convert_x_mx_kernel<SRC>), dim3((unsigned)((int64_t)M * chunks)), dim3(kMxCvtBlocks), 0, stream, src, K, kp,
                           x_row_halfs(K), chunks, x16, scales);
        return hip_ok(hipGetLastError(), "activation convert launch");
    }
    // three activation orders: the K-quant nibble order, the split-nibble order of the 32-weight blocks, natural
    switch (type) {
    case kTypeQ4_K: case kTypeQ5_K: launch_convert_typed<kTypeQ4_K, SRC>(src, M, K, kp, x16, scales, stream); break;
    case kTypeMXFP4: case kTypeQ4_0: case kTypeQ4_1: case kTypeQ5_0: case kTypeQ5_1: case kTypeIQ4_NL:
        launch_convert_typed<kTypeMXFP4, SRC>(src, M, K, kp, x16, scales, stream);
        break;
    case kTypeQ8_0: case kTypeQ6_K: launch_convert_typed<kTypeQ8_0, SRC>(src, M, K, kp, x16, scales, stream); break;
    default: set_last_error("gemm: unsupported type."); return false;
    }
    return hip_ok(hipGetLastError(), "activation convert launch");
}

}  // namespace

// Which activation layout the GEMM of this shape reads: 0 fp16 in the format's unpack order; 1 two MX fp6 terms for
// gemm_mx_kernel (plain MXFP4 launches on 128- or 256-row tiles).
// (rows longer than 32768 stay on the fp16 path, whose tile kernels cut such a K into chunks, and so do small batches
// over small weights, which gain nothing: 64 x 5760 x 2880 18.2 vs 17.7 us, 16 x 4096 x 14336 26.9 vs 23.0 us, but
// 32 x 184320 x 2880 61-67 vs 74-84 us)
int gemm_x_layout(int type, int M, int N, int K)
{
    if (type != kTypeMXFP4 || K > 1024 * kCvtHold * 4) return 0;
    return gemm_tile_m(type, M, N) >= 128 || (int64_t)N * K >= ((int64_t)64 << 20) ? 1 : 0;
}

bool launch_convert_x(int type, const float* x, int64_t ldx, const int* row_map, int M, int K, void* workspace,
                      hipStream_t stream, const float* norm_w, float eps, int layout)
{
    ConvertSrc src{};
    src.x = x;
    src.ldx = ldx;
    src.row_map = row_map;
    src.norm_w = norm_w;
    src.eps = eps;
    return launch_convert<kSrcPlain>(type, src, M, K, workspace, stream, layout);
}

bool launch_convert_x_swiglu(int type, const float* gate_up, const float* bias, const int* expert_of, float alpha, float limit,
                             int M, int F, void* workspace, hipStream_t stream, int layout)
{
    ConvertSrc src{};
    src.x = gate_up;
    src.ldx = 2 * (int64_t)F;
    src.bias = bias;
    src.expert_of = expert_of;
    src.alpha = alpha;
    src.limit = limit;
    return launch_convert<kSrcSwiglu>(type, src, M, F, workspace, stream, layout);
}

namespace {
bool gemm_dispatch(int type, const void* w, int64_t w_bytes, const void* workspace, float* c, int64_t ldc, const int* c_rows,
                   int M, int N, int K, const GemmTiles* tiles, hipStream_t stream, bool accumulate, const ChunkScratch& cs,
                   int x_layout)
{
    if (w_bytes >= kMaxOperandBytes && !tiles) {
        set_last_error("gemm: a single weight of 2 GiB or more must be split by rows.");
        return false;
    }
    GemmArgs a{};
    a.w = static_cast<const uint8_t*>(w);
    a.w_bytes = w_bytes;
    a.xscale = static_cast<const float*>(workspace);
    a.x16 = reinterpret_cast<const _Float16*>(static_cast<const char*>(workspace) + (((size_t)M * sizeof(float) + 255) & ~(size_t)255));
    a.c = c;
    a.ldc = ldc;
    a.c_rows = c_rows;
    a.accumulate = accumulate ? 1 : 0;
    a.x_mx = x_layout == 1 ? 1 : 0;
    a.M = M;
    a.N = N;
    a.K = K;
    a.Kp = (K + kBK - 1) / kBK * kBK;
    a.xld = x_row_halfs(K);
    a.x16_bytes = (int64_t)M * a.xld * (int64_t)sizeof(_Float16);
    if (a.x16_bytes >= kMaxOperandBytes) {
        set_last_error("gemm: the converted activations of one call must stay below 2 GiB; split the rows.");
        return false;
    }
    int bm, m_tiles;
    if (tiles) {
        a.tile_expert = tiles->expert;
        a.tile_row0 = tiles->row0;
        a.tile_rows = tiles->rows;
        a.expert_stride = tiles->expert_stride;
        a.expert_off = tiles->expert_off;
        bm = tiles->bm;
        m_tiles = tiles->count;
    } else {
        bm = gemm_tile_m(type, M, N);
        if (type == kTypeQ6_K && bm == 256) bm = 128;     // two raw Q6_K super-tiles of 256 columns do not fit LDS
        m_tiles = (M + bm - 1) / bm;
    }
    if (m_tiles == 0) return true;
    switch (type) {
    case kTypeQ4_K: return launch_for_type<GQ4K>(a, bm, m_tiles, stream, cs);
    case kTypeMXFP4: return launch_for_type<GMXFP4>(a, bm, m_tiles, stream, cs);
    case kTypeQ8_0: return launch_for_type<GQ80>(a, bm, m_tiles, stream, cs);
    case kTypeQ6_K: return launch_for_type<GQ6K>(a, bm, m_tiles, stream, cs);
    case kTypeQ5_K: return launch_for_type<GQ5K>(a, bm, m_tiles, stream, cs);
    case kTypeQ4_0: return launch_for_type<GLegacy<kTypeQ4_0>>(a, bm, m_tiles, stream, cs);
    case kTypeQ4_1: return launch_for_type<GLegacy<kTypeQ4_1>>(a, bm, m_tiles, stream, cs);
    case kTypeQ5_0: return launch_for_type<GLegacy<kTypeQ5_0>>(a, bm, m_tiles, stream, cs);
    case kTypeQ5_1: return launch_for_type<GLegacy<kTypeQ5_1>>(a, bm, m_tiles, stream, cs);
    case kTypeIQ4_NL: return launch_for_type<GLegacy<kTypeIQ4_NL>>(a, bm, m_tiles, stream, cs);
    default: set_last_error("gemm: unsupported type."); return false;
    }
}
}  // namespace

bool launch_gemm(int type, const void* w, int64_t w_bytes, const void* workspace, float* c, int64_t ldc, const int* c_rows,
                 int M, int N, int K, const GemmTiles* tiles, hipStream_t stream, bool accumulate, void* chunk_ws,
                 size_t chunk_ws_bytes, int x_layout)
{
    const ChunkScratch cs{static_cast<float*>(chunk_ws), chunk_ws ? chunk_ws_bytes : 0, nullptr};
    return gemm_dispatch(type, w, w_bytes, workspace, c, ldc, c_rows, M, N, K, tiles, stream, accumulate, cs, x_layout);
}

bool gemm_swiglu_mx_fits(int F, int K)
{
    const int kt = (K + kBK - 1) / kBK;
    return F > 0 && F % 32 == 0 && kt > 16 && kt <= 48 && F <= 32768;
}

bool launch_gemm_swiglu_mx(const void* w, const void* workspace, void* workspace_out, float* act, const float* bias, float alpha,
                           float limit, int M, int F, int K, const GemmTiles* tiles, hipStream_t stream)
{
    if (!tiles || (tiles->bm != 32 && tiles->bm != 48) || !gemm_swiglu_mx_fits(F, K)) {
        set_last_error("gemm: the fused SwiGLU epilogue takes 32- or 48-row expert tiles, F a multiple of 32 and 1025 .. 3072 columns of K.");
        return false;
    }
    GemmArgs a{};
    a.w = static_cast<const uint8_t*>(w);
    a.w_bytes = tiles->expert_stride;
    a.xscale = static_cast<const float*>(workspace);
    a.x16 = reinterpret_cast<const _Float16*>(static_cast<const char*>(workspace) + (((size_t)M * sizeof(float) + 255) & ~(size_t)255));
    a.x_mx = 1;
    a.M = M;
    a.N = 2 * F;
    a.K = K;
    a.Kp = (K + kBK - 1) / kBK * kBK;
    a.xld = x_row_halfs(K);
    a.x16_bytes = (int64_t)M * a.xld * (int64_t)sizeof(_Float16);
    a.epi_bias = bias;
    a.epi_alpha = alpha;
    a.epi_limit = limit;
    a.epi_out = reinterpret_cast<uint8_t*>(static_cast<char*>(workspace_out) + (((size_t)M * sizeof(float) + 255) & ~(size_t)255));
    a.epi_ld = (int64_t)x_row_halfs(F) * (int64_t)sizeof(_Float16);
    if (a.x16_bytes >= kMaxOperandBytes || (int64_t)M * a.epi_ld >= kMaxOperandBytes) {
        set_last_error("gemm: the converted activations of one call must stay below 2 GiB; split the rows.");
        return false;
    }
    a.tile_expert = tiles->expert;
    a.tile_row0 = tiles->row0;
    a.tile_rows = tiles->rows;
    a.expert_stride = tiles->expert_stride;
    a.expert_off = tiles->expert_off;
    if (tiles->count == 0) return true;
    const ChunkScratch cs{nullptr, 0, nullptr};
    if (tiles->bm == 48) {
        // 48-row units leave the activations as fp32 [M x F] in act; the conversion is a launch of its own
        a.c = act;
        a.ldc = F;
        return launch_slim_mx48<1>(a, tiles->count, stream, cs) &&
               launch_convert_x(kTypeMXFP4, act, F, nullptr, M, F, workspace_out, stream, nullptr, 0.f, 1);
    }
    return a.Kp / kBK <= 32 ? launch_slim_mx<4, 1, 1>(a, tiles->count, stream, cs) : launch_slim_mx<6, 1, 1>(a, tiles->count, stream, cs);
}

size_t gemm_chunk_ws_bytes(int type, int M, int N, int K, const GemmTiles* tiles, bool accumulate, int x_layout)
{
    size_t need = 0;
    // a buffer "large enough" so that the launchers make the choices they would make with the reported bytes at hand
    const ChunkScratch cs{nullptr, ~(size_t)0, &need};
    const int64_t w_bytes = tiles ? 0 : (int64_t)(block_bytes(type) * (K / block_elems(type))) * N;
    if (!gemm_dispatch(type, nullptr, w_bytes, nullptr, nullptr, N, nullptr, M, N, K, tiles, nullptr, accumulate, cs,
                       x_layout >= 0 ? x_layout : tiles ? 0 : gemm_x_layout(type, M, N, K)))
        return 0;
    return need;
}

}  // namespace tship
