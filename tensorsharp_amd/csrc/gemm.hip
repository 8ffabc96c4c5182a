// Prefill GEMM  C[M x N] = X[M x K] * W[N x K]^T  over raw GGUF blocks (Q8_0 / Q4_K / MXFP4) on
// the gfx950 matrix cores.
//
//   1. convert_x_kernel: fp32 activations -> fp16, one power-of-two scale per row (so no input
//      magnitude overflows or underflows fp16), written in the k-order in which the weight
//      format unpacks (so the dequantizer never has to shuffle lanes), zero-padded to a
//      multiple of the k-tile.  Optionally gathers rows through an index (MoE).
//   2. gemm_kernel: BM x BN x 64 tiles (256 x 256 with 8 wavefronts for large M).  Per k-tile the raw
//      quantized bytes of BN weight rows are loaded (Q4_K: 32 quant bytes + the super-block header per
//      row, Q8_0 / MXFP4: two blocks per row through a range-checked buffer resource), dequantized
//      ONCE to fp16 with packed-fp16 VALU and written to LDS next to the activation tile; the
//      wavefronts then run v_mfma_f32_32x32x16_f16 out of LDS with fp32 accumulation.  LDS is
//      double-buffered, the global loads run two tiles ahead, and the tile order is XCD-aware.
//   3. epilogue: fp32 accumulators times the row scale -> C (optionally scattered through a row
//      index).
//
// Arithmetic: dequantised values follow ManagedQuantizedOps.cs:411-427 / :447-479 / :579-598 and
// are then rounded to fp16 operands (Q4_K: d*sc and dmin*m rounded to fp16 first); the contraction
// is TensorSharp.Models/ModelBase.cs:924-991 with fp32 accumulation on the matrix cores.
#include "tship_internal.h"

#include <algorithm>

namespace tship {
namespace {

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef uint32_t uint4_t __attribute__((ext_vector_type(4)));

constexpr int kBK = 64;                 // k-tile
constexpr int kLdsRow = kBK + 8;        // fp16 per LDS row: 144 B keeps ds_read_b128 conflict-free
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

// position inside a k-tile at which activation k (0..63) is stored, per weight format
template <int TYPE>
__device__ __forceinline__ int k_slot(int k)
{
    if (TYPE == kTypeQ4_K) {
        // quant dword -> (e0,e2),(e1,e3): order [0,2,1,3] inside every 4
        const int q = k & 3;
        return (k & ~3) | ((q & 1) << 1) | (q >> 1);
    }
    if (TYPE == kTypeMXFP4) {
        // quant byte j -> (e_j, e_{j+16}) inside every 32
        const int j = k & 15, hi = (k >> 4) & 1;
        return (k & ~31) | (j << 1) | hi;
    }
    return k;
}

// ------------------------------------------------------------------------------------------
// activations: fp32 [M x K] (row stride ldx) -> fp16 [M x Kp] in unpack order, per-row scale
// ------------------------------------------------------------------------------------------
template <int TYPE>
__global__ void __launch_bounds__(256) convert_x_kernel(const float* __restrict__ x, int64_t ldx, const int* __restrict__ row_map,
                                                        int K, int Kp, _Float16* __restrict__ out, float* __restrict__ scales)
{
    const int m = blockIdx.x;
    const float* src = x + (int64_t)(row_map ? row_map[m] : m) * ldx;
    __shared__ float red[4];
    float amax = 0.f;
    for (int k = threadIdx.x * 4; k < K; k += 1024) {
        const float4 v = *reinterpret_cast<const float4*>(src + k);
        amax = fmaxf(amax, fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w))));
    }
    for (int o = 32; o > 0; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o));
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    // power-of-two scale bringing amax into [2^13, 2^14)
    int e = (int)((__float_as_uint(amax) >> 23) & 0xffu);
    if (e == 255) e = 127;
    if (e < 14) e = 14;
    const int se = e - 13;
    const float inv = __uint_as_float((uint32_t)(254 - se) << 23);
    if (threadIdx.x == 0) scales[m] = __uint_as_float((uint32_t)se << 23);
    _Float16* dst = out + (int64_t)m * Kp;
    for (int k = threadIdx.x; k < Kp; k += 256) {
        const float v = k < K ? src[k] * inv : 0.f;
        dst[(k & ~(kBK - 1)) | k_slot<TYPE>(k & (kBK - 1))] = (_Float16)v;
    }
}

// ------------------------------------------------------------------------------------------
// weight tile loaders: ITEMS work items per row and k-tile, each yielding 32 fp16 for LDS
// ------------------------------------------------------------------------------------------
struct WTensor {
    __amdgpu_buffer_rsrc_t rs;   // range-checked view of the weight bytes
    uint32_t base_delta;         // (weight address) & 3
    uint32_t row_bytes;
    int K;
};

// Q4_K: item (row, h) = quant bytes [16h, 16h+16) of the k-tile's 64-group
struct GQ4K {
    static constexpr int kRegs = 8;
    static constexpr bool kWholeTile = true;    // K is a multiple of 256: every k-tile is complete
    static __device__ __forceinline__ void load(const WTensor& W, uint32_t row_off, int kt, int h, uint32_t (&r)[kRegs])
    {
        const uint32_t blk = row_off + (uint32_t)(kt >> 2) * 144u;
        const uint4_t hdr = __builtin_amdgcn_raw_buffer_load_b128(W.rs, (int)blk, 0, 0);
        const uint4_t q = __builtin_amdgcn_raw_buffer_load_b128(W.rs, (int)(blk + 16u + (uint32_t)(kt & 3) * 32u + (uint32_t)h * 16u), 0, 0);
        r[0] = hdr.x; r[1] = hdr.y; r[2] = hdr.z; r[3] = hdr.w;
        r[4] = q.x; r[5] = q.y; r[6] = q.z; r[7] = q.w;
    }
    // writes k' [16h, 16h+16) (low nibbles) and [32+16h, ...) (high nibbles) of LDS row `dst`
    static __device__ __forceinline__ void store(const uint32_t (&r)[kRegs], uint32_t /*row_off*/, int kt, int h, bool live, _Float16* dst)
    {
        const int g4 = kt & 3;
        const int sh = (g4 & 1) * 16;
        const uint32_t a = r[1] >> sh, b = r[2] >> sh, c = r[3] >> sh;
        const uint32_t sc_lo = a & 0x3f3fu, m_lo = b & 0x3f3fu;
        const uint32_t sc_hi = (c & 0x0f0fu) | ((a >> 2) & 0x3030u);
        const uint32_t m_hi = ((c >> 4) & 0x0f0fu) | ((b >> 2) & 0x3030u);
        const uint32_t sc = (g4 & 2) ? sc_hi : sc_lo, mn = (g4 & 2) ? m_hi : m_lo;
        H2U dm;
        dm.u = r[0];
        const float d = live ? (float)dm.h.x : 0.f, dmin = live ? (float)dm.h.y : 0.f;
        const uint32_t s1 = splat(d * (float)(sc & 0xffu)), o1 = splat(-(dmin * (float)(mn & 0xffu)));
        const uint32_t s2 = splat(d * (float)(sc >> 8) * 0.0625f), o2 = splat(-(dmin * (float)(mn >> 8)));
        const uint32_t magic = 0x64006400u, neg1024 = 0xe400e400u;   // 1024.0, -1024.0
        uint32_t lo[8], hi[8];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t q = r[4 + j], q8 = q >> 8;
            // 0x6400 | nibble = 1024 + q (low) or 1024 + 16 q (high): exact after subtracting 1024
            lo[2 * j] = pk_fma(pk_add((q & 0x000f000fu) | magic, neg1024), s1, o1);
            lo[2 * j + 1] = pk_fma(pk_add((q8 & 0x000f000fu) | magic, neg1024), s1, o1);
            hi[2 * j] = pk_fma(pk_add((q & 0x00f000f0u) | magic, neg1024), s2, o2);
            hi[2 * j + 1] = pk_fma(pk_add((q8 & 0x00f000f0u) | magic, neg1024), s2, o2);
        }
        uint4* p = reinterpret_cast<uint4*>(dst + 16 * h);
        p[0] = uint4{lo[0], lo[1], lo[2], lo[3]};
        p[1] = uint4{lo[4], lo[5], lo[6], lo[7]};
        p[4] = uint4{hi[0], hi[1], hi[2], hi[3]};
        p[5] = uint4{hi[4], hi[5], hi[6], hi[7]};
    }
};

// MXFP4: item (row, b) = block b (0/1) of the k-tile, 17 bytes inside a 20-byte aligned window
struct GMXFP4 {
    static constexpr int kRegs = 5;
    static constexpr bool kWholeTile = false;   // K % 64 may be 32: the last tile's second block is absent
    static __device__ __forceinline__ void load(const WTensor& W, uint32_t row_off, int kt, int b, uint32_t (&r)[kRegs])
    {
        const int blk = kt * 2 + b;
        const uint32_t p = row_off + (uint32_t)blk * 17u;
        const uint32_t al = (blk * 32 < W.K) ? (p & ~3u) : kDeadOffset;
        const uint4_t v = __builtin_amdgcn_raw_buffer_load_b128(W.rs, (int)al, 0, 0);
        r[0] = v.x; r[1] = v.y; r[2] = v.z; r[3] = v.w;
        r[4] = __builtin_amdgcn_raw_buffer_load_b32(W.rs, (int)(al + 16u), 0, 0);
    }
    template <int SEL>
    static __device__ __forceinline__ uint32_t cvt(uint32_t q, float scale)
    {
        H2U c;
        c.h = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(q, scale, SEL);
        return c.u;
    }
    static __device__ __forceinline__ void store(const uint32_t (&r)[kRegs], uint32_t row_off, int kt, int b, bool live, _Float16* dst)
    {
        const uint32_t o = (row_off + (uint32_t)(kt * 2 + b) * 17u) & 3u;
        const uint32_t e = (r[0] >> (8 * o)) & 0xffu;
        const bool wrap = o == 3;
        const uint32_t b0 = wrap ? r[1] : r[0], b1 = wrap ? r[2] : r[1], b2 = wrap ? r[3] : r[2];
        const uint32_t b3 = wrap ? r[4] : r[3], b4 = r[4];
        const uint32_t shb = (o + 1) & 3;
        const uint32_t q0 = __builtin_amdgcn_alignbyte(b1, b0, shb), q1 = __builtin_amdgcn_alignbyte(b2, b1, shb);
        const uint32_t q2 = __builtin_amdgcn_alignbyte(b3, b2, shb), q3 = __builtin_amdgcn_alignbyte(b4, b3, shb);
        // doubled E2M1 * 2^(e-128) = E2M1 * 2^(e-127); an absent block (K tail) stores zeros
        const float scale = live ? __uint_as_float(e == 0 ? 0x00400000u : (e << 23)) : 0.f;
        uint4* p = reinterpret_cast<uint4*>(dst + 32 * b);
        p[0] = uint4{cvt<0>(q0, scale), cvt<1>(q0, scale), cvt<2>(q0, scale), cvt<3>(q0, scale)};
        p[1] = uint4{cvt<0>(q1, scale), cvt<1>(q1, scale), cvt<2>(q1, scale), cvt<3>(q1, scale)};
        p[2] = uint4{cvt<0>(q2, scale), cvt<1>(q2, scale), cvt<2>(q2, scale), cvt<3>(q2, scale)};
        p[3] = uint4{cvt<0>(q3, scale), cvt<1>(q3, scale), cvt<2>(q3, scale), cvt<3>(q3, scale)};
    }
};

// Q8_0: item (row, b) = block b (0/1) of the k-tile, 34 bytes inside a 36-byte aligned window
struct GQ80 {
    static constexpr int kRegs = 9;
    static constexpr bool kWholeTile = false;
    static __device__ __forceinline__ void load(const WTensor& W, uint32_t row_off, int kt, int b, uint32_t (&r)[kRegs])
    {
        const int blk = kt * 2 + b;
        const uint32_t p = row_off + (uint32_t)blk * 34u;
        const uint32_t al = (blk * 32 < W.K) ? (p & ~3u) : kDeadOffset;
        const uint4_t v0 = __builtin_amdgcn_raw_buffer_load_b128(W.rs, (int)al, 0, 0);
        const uint4_t v1 = __builtin_amdgcn_raw_buffer_load_b128(W.rs, (int)(al + 16u), 0, 0);
        r[0] = v0.x; r[1] = v0.y; r[2] = v0.z; r[3] = v0.w;
        r[4] = v1.x; r[5] = v1.y; r[6] = v1.z; r[7] = v1.w;
        r[8] = __builtin_amdgcn_raw_buffer_load_b32(W.rs, (int)(al + 32u), 0, 0);
    }
    static __device__ __forceinline__ void store(const uint32_t (&r)[kRegs], uint32_t row_off, int kt, int b, bool live, _Float16* dst)
    {
        const bool odd = ((row_off + (uint32_t)(kt * 2 + b) * 34u) & 2u) != 0;
        const uint32_t dbits = odd ? (r[0] >> 16) : (r[0] & 0xffffu);
        const uint32_t d2 = live ? (dbits | (dbits << 16)) : 0u;      // fp16 d in both halves
        const uint32_t bias = 0xe480e480u;                              // -1152.0 = -(1024 + 128)
        uint32_t o[16];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint32_t q = (odd ? r[i + 1] : __builtin_amdgcn_alignbyte(r[i + 1], r[i], 2)) ^ 0x80808080u;
            // bytes u = q + 128 become fp16 1024 + u: (0x64, u) pairs picked with v_perm
            const uint32_t p0 = __builtin_amdgcn_perm(0x64646464u, q, 0x04010400u);   // (u0, u1)
            const uint32_t p1 = __builtin_amdgcn_perm(0x64646464u, q, 0x04030402u);   // (u2, u3)
            o[2 * i] = pk_mul(pk_add(p0, bias), d2);
            o[2 * i + 1] = pk_mul(pk_add(p1, bias), d2);
        }
        uint4* p = reinterpret_cast<uint4*>(dst + 32 * b);
        p[0] = uint4{o[0], o[1], o[2], o[3]};
        p[1] = uint4{o[4], o[5], o[6], o[7]};
        p[2] = uint4{o[8], o[9], o[10], o[11]};
        p[3] = uint4{o[12], o[13], o[14], o[15]};
    }
};

struct GemmArgs {
    const uint8_t* w;        // weight bytes (of expert 0 for grouped launches)
    int64_t w_bytes;         // bytes of one weight matrix (per expert for grouped launches)
    const _Float16* x16;     // [rows x Kp] converted activations
    const float* xscale;     // [rows]
    float* c;                // result
    int64_t ldc;
    const int* c_rows;       // optional: result row index per activation row (scatter)
    int M, N, K, Kp;
    int m_tiles, n_tiles;
    // grouped (MoE) launches: m-tiles enumerated through this table
    const int* tile_expert;  // [m_tiles] expert id
    const int* tile_row0;    // [m_tiles] first activation row
    const int* tile_rows;    // [m_tiles] rows in the tile (<= BM)
    int64_t expert_stride;   // bytes between experts
};

// One k-tile of MFMA work for a wavefront: TM x TN tiles of 32x32, four k-steps of 16.  The LDS
// fragments of k-step s+1 are requested before the MFMAs of k-step s are issued, so the matrix
// pipe covers the LDS latency.
template <int TM, int TN>
__device__ __forceinline__ void mma_tile(const _Float16* xs, const _Float16* ws, float16_t (&acc)[TM][TN])
{
    half8_t a[2][TM], b[2][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i) a[0][i] = *reinterpret_cast<const half8_t*>(xs + i * 32 * kLdsRow);
#pragma unroll
    for (int j = 0; j < TN; ++j) b[0][j] = *reinterpret_cast<const half8_t*>(ws + j * 32 * kLdsRow);
#pragma unroll
    for (int ks = 0; ks < kBK / 16; ++ks) {
        const int c = ks & 1, n = c ^ 1;
        if (ks + 1 < kBK / 16) {
#pragma unroll
            for (int i = 0; i < TM; ++i) a[n][i] = *reinterpret_cast<const half8_t*>(xs + i * 32 * kLdsRow + (ks + 1) * 16);
#pragma unroll
            for (int j = 0; j < TN; ++j) b[n][j] = *reinterpret_cast<const half8_t*>(ws + j * 32 * kLdsRow + (ks + 1) * 16);
        }
        __builtin_amdgcn_sched_barrier(0);   // keep the requests above the MFMAs they are meant to overlap
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[c][i], b[c][j], acc[i][j], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
    }
}

// BM x BN x 64 tiles, WM x WN wavefronts.  LDS holds two k-tiles (activations + dequantized weights);
// per iteration every wavefront (a) dequantizes the raw bytes it fetched for tile kt+1 into the idle
// buffer, (b) requests the raw bytes of tile kt+2, (c) multiplies tile kt.  Wavefronts that share a
// SIMD run (a)(b) and (c) in opposite order so that the VALU dequantization of one overlaps the MFMA
// phase of the other.  One barrier per k-tile.
template <typename G, int BM, int BN, int WM, int WN>
__global__ void __launch_bounds__(WM * WN * 64) gemm_kernel(const GemmArgs A)
{
    constexpr int NT = WM * WN * 64;
    constexpr int TM = BM / WM / 32, TN = BN / WN / 32;
    constexpr int XCH = BM * 8 / NT;                 // 16-byte activation chunks per thread per k-tile
    constexpr int WIT = BN * 2 / NT;                 // weight items per thread per k-tile
    constexpr int kBufElems = (BM + BN) * kLdsRow;
    static_assert(XCH >= 1 && WIT >= 1, "tile too small for the workgroup");
    extern __shared__ _Float16 smem[];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WN, wn = wave % WN;

    // XCD-aware tile order: workgroup ids go round-robin over the 8 XCDs, so each XCD gets a contiguous
    // run of tiles; consecutive tiles share the activation rows (same m-tile), which then stay in that
    // XCD's L2 while its CUs walk over the weight columns.
    const int total = A.m_tiles * A.n_tiles;
    int t = blockIdx.x;
    {
        const int per = (total + 7) >> 3;
        const int xcd = t & 7, slot = t >> 3;
        t = xcd * per + slot;
        if (slot >= per || t >= total) return;
    }
    const int mt = t / A.n_tiles, nt = t - mt * A.n_tiles;
    int m0, m_rows;
    const uint8_t* wbase = A.w;
    if (A.tile_expert) {
        m0 = A.tile_row0[mt];
        m_rows = A.tile_rows[mt];
        if (m_rows <= 0) return;          // table entries past the last tile
        wbase += (int64_t)A.tile_expert[mt] * A.expert_stride;
    } else {
        m0 = mt * BM;
        m_rows = min(BM, A.M - m0);
    }
    const int n0 = nt * BN;

    WTensor W;
    const uintptr_t wa = reinterpret_cast<uintptr_t>(wbase);
    W.base_delta = (uint32_t)(wa & 3);
    W.rs = __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>(wa & ~(uintptr_t)3), 0,
                                             (int)(((uint32_t)A.w_bytes + W.base_delta + 3u) & ~3u), 0x00020000);
    W.K = A.K;
    W.row_bytes = (uint32_t)((int64_t)A.w_bytes / A.N);

    // per-thread sources / destinations (constant over the k loop)
    const _Float16* x_src[XCH];
    int x_dst[XCH];
#pragma unroll
    for (int i = 0; i < XCH; ++i) {
        const int c = tid + i * NT;
        const int row = c >> 3, chunk = c & 7;
        x_src[i] = A.x16 + (int64_t)(m0 + min(row, m_rows - 1)) * A.Kp + chunk * 8;
        x_dst[i] = row * kLdsRow + chunk * 8;
    }
    uint32_t w_off[WIT];
    int w_part[WIT], w_dst[WIT];
#pragma unroll
    for (int i = 0; i < WIT; ++i) {
        const int it = tid + i * NT;
        const int row = it >> 1;
        w_part[i] = it & 1;
        w_off[i] = W.base_delta + (uint32_t)min(n0 + row, A.N - 1) * W.row_bytes;
        w_dst[i] = (BM + row) * kLdsRow;
    }

    uint4_t xr[XCH];
    uint32_t wr[WIT][G::kRegs];
#define TSHIP_GEMM_LOAD(kt)                                                                        \
    do {                                                                                           \
        _Pragma("unroll") for (int i = 0; i < XCH; ++i) xr[i] = *reinterpret_cast<const uint4_t*>(x_src[i] + (kt) * kBK); \
        _Pragma("unroll") for (int i = 0; i < WIT; ++i) G::load(W, w_off[i], (kt), w_part[i], wr[i]);  \
    } while (0)
#define TSHIP_GEMM_STORE(kt, buf)                                                                  \
    do {                                                                                           \
        _Float16* dstb = smem + (buf) * kBufElems;                                                 \
        _Pragma("unroll") for (int i = 0; i < XCH; ++i) *reinterpret_cast<uint4_t*>(dstb + x_dst[i]) = xr[i]; \
        _Pragma("unroll") for (int i = 0; i < WIT; ++i) {                                          \
            const bool live = G::kWholeTile || ((kt) * 2 + w_part[i]) * 32 < A.K;                  \
            G::store(wr[i], w_off[i], (kt), w_part[i], live, dstb + w_dst[i]);                     \
        }                                                                                          \
    } while (0)

    float16_t acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    const int nkt = A.Kp / kBK;
    const int frag = (lane & 31) * kLdsRow + (lane >> 5) * 8;
    const int xs_off = wm * (BM / WM) * kLdsRow + frag;
    const int ws_off = (BM + wn * (BN / WN)) * kLdsRow + frag;
    // wavefronts w and w + 4 share a SIMD: one of them multiplies first, the other dequantizes first
    const bool mma_first = (wave & 4) != 0 && NT > 256;

    TSHIP_GEMM_LOAD(0);
    TSHIP_GEMM_STORE(0, 0);
    if (nkt > 1) TSHIP_GEMM_LOAD(1);
    __syncthreads();
    for (int kt = 0; kt < nkt; ++kt) {
        const int cur = kt & 1;
        const _Float16* bufc = smem + cur * kBufElems;
        if (mma_first) mma_tile<TM, TN>(bufc + xs_off, bufc + ws_off, acc);
        if (kt + 1 < nkt) TSHIP_GEMM_STORE(kt + 1, cur ^ 1);
        // past the last tile the loads wrap to tile 0: harmless, and the loop body stays branch-free
        TSHIP_GEMM_LOAD(kt + 2 < nkt ? kt + 2 : 0);
        if (!mma_first) mma_tile<TM, TN>(bufc + xs_off, bufc + ws_off, acc);
        __syncthreads();
    }
#undef TSHIP_GEMM_LOAD
#undef TSHIP_GEMM_STORE

    // epilogue: D[row = 8*(r/4) + 4*(lane/32) + r%4][col = lane%32]
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int ml = wm * (BM / WM) + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
            if (ml < m_rows) {
                const int m = m0 + ml;
                const float s = A.xscale[m];
                float* crow = A.c + (int64_t)(A.c_rows ? A.c_rows[m] : m) * A.ldc;
#pragma unroll
                for (int j = 0; j < TN; ++j) {
                    const int n = n0 + wn * (BN / WN) + j * 32 + (lane & 31);
                    if (n < A.N) crow[n] = acc[i][j][r] * s;
                }
            }
        }
    }
}

template <typename G, int BM, int BN, int WM, int WN>
bool launch_tiles(GemmArgs a, int m_tiles, hipStream_t stream)
{
    auto kern = gemm_kernel<G, BM, BN, WM, WN>;
    const size_t lds = (size_t)2 * (BM + BN) * kLdsRow * sizeof(_Float16);
    if (lds > 64 * 1024 &&
        !hip_ok(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds),
                "gemm: raising the dynamic LDS limit"))
        return false;
    a.m_tiles = m_tiles;
    a.n_tiles = (a.N + BN - 1) / BN;
    const int total = a.m_tiles * a.n_tiles;
    const int grid = ((total + 7) / 8) * 8;          // whole rounds over the 8 XCDs
    hipLaunchKernelGGL(kern, dim3(grid), dim3(WM * WN * 64), lds, stream, a);
    return hip_ok(hipGetLastError(), "gemm launch");
}

template <typename G>
bool launch_for_type(const GemmArgs& a, int bm, int m_tiles, hipStream_t stream)
{
#ifdef TSHIP_GEMM_VARIANT
    if (bm == 256) return launch_tiles<G, TSHIP_GEMM_VARIANT>(a, m_tiles, stream);
#endif
    if (bm == 256) return launch_tiles<G, 256, 256, 4, 2>(a, m_tiles, stream);
    if (bm == 128) return launch_tiles<G, 128, 256, 2, 4>(a, m_tiles, stream);
    return launch_tiles<G, 64, 128, 1, 4>(a, m_tiles, stream);
}

}  // namespace

size_t gemm_workspace_bytes(int M, int K)
{
    const size_t kp = (size_t)((K + kBK - 1) / kBK) * kBK;
    return (size_t)M * kp * sizeof(_Float16) + (((size_t)M * sizeof(float) + 255) & ~(size_t)255) + 256;
}

int gemm_tile_m(int M) { return M > 1024 ? 256 : M > 64 ? 128 : 64; }

bool launch_convert_x(int type, const float* x, int64_t ldx, const int* row_map, int M, int K, void* workspace,
                      hipStream_t stream)
{
    const int kp = (K + kBK - 1) / kBK * kBK;
    float* scales = static_cast<float*>(workspace);
    _Float16* x16 = reinterpret_cast<_Float16*>(static_cast<char*>(workspace) + (((size_t)M * sizeof(float) + 255) & ~(size_t)255));
    switch (type) {
    case kTypeQ4_K: hipLaunchKernelGGL(convert_x_kernel<kTypeQ4_K>, dim3(M), dim3(256), 0, stream, x, ldx, row_map, K, kp, x16, scales); break;
    case kTypeMXFP4: hipLaunchKernelGGL(convert_x_kernel<kTypeMXFP4>, dim3(M), dim3(256), 0, stream, x, ldx, row_map, K, kp, x16, scales); break;
    case kTypeQ8_0: hipLaunchKernelGGL(convert_x_kernel<kTypeQ8_0>, dim3(M), dim3(256), 0, stream, x, ldx, row_map, K, kp, x16, scales); break;
    default: set_last_error("gemm: unsupported type."); return false;
    }
    return hip_ok(hipGetLastError(), "activation convert launch");
}

bool launch_gemm(int type, const void* w, int64_t w_bytes, const void* workspace, float* c, int64_t ldc, const int* c_rows,
                 int M, int N, int K, const GemmTiles* tiles, hipStream_t stream)
{
    if (w_bytes >= ((int64_t)1 << 31) - 64 && !tiles) {
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
    a.M = M;
    a.N = N;
    a.K = K;
    a.Kp = (K + kBK - 1) / kBK * kBK;
    int bm, m_tiles;
    if (tiles) {
        a.tile_expert = tiles->expert;
        a.tile_row0 = tiles->row0;
        a.tile_rows = tiles->rows;
        a.expert_stride = tiles->expert_stride;
        bm = tiles->bm;
        m_tiles = tiles->count;
    } else {
        bm = gemm_tile_m(M);
        m_tiles = (M + bm - 1) / bm;
    }
    if (m_tiles == 0) return true;
    switch (type) {
    case kTypeQ4_K: return launch_for_type<GQ4K>(a, bm, m_tiles, stream);
    case kTypeMXFP4: return launch_for_type<GMXFP4>(a, bm, m_tiles, stream);
    case kTypeQ8_0: return launch_for_type<GQ80>(a, bm, m_tiles, stream);
    default: set_last_error("gemm: unsupported type."); return false;
    }
}

}  // namespace tship
