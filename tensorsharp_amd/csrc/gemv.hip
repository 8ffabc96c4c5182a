// Decode GEMV  y[N] = W[N x K] * x[K]  over raw GGUF blocks (Q8_0 / Q4_K / Q5_K / Q6_K / MXFP4) for gfx950.
//
// Shape of the kernel (all formats):
//   * persistent workgroups of 8 wavefronts (two per CU); each workgroup stages x once into LDS in the layout its
//     format's unpack order wants (fp16 pairs for the K-quants and MXFP4, fp32 for Q8_0), padded so that a
//     ds_read_b128 per lane is bank-conflict free;
//   * a wavefront owns a group of consecutive weight rows at a time, one row per LPR lanes (Q8_0 / MXFP4: 4 rows x 16
//     lanes, the K-quants: 2 rows x 32 lanes).  A row is cut into "units" (Q8_0: one 34-byte block, MXFP4: one 17-byte
//     block, K-quants: one 64-weight group of a 256-weight block); lane l of a row takes units l, l + LPR, ... so
//     consecutive lanes read consecutive bytes of the raw blocks with 128-bit loads, everything that depends only on
//     the lane (block offset, scale bit positions, LDS address of its activations) is computed once, and the row /
//     step part of every address is a scalar.  Unaligned units (34 B / 17 B blocks, pieces of the 210-byte Q6_K
//     block) are fetched as aligned dwords through a range-checked buffer resource and re-aligned in registers with
//     v_alignbyte;
//   * the loads of the next step are issued before the current step is consumed (two register sets that swap roles),
//     and the very first step is issued before x is staged, so that weight latency overlaps the prologue;
//   * dequantization happens in registers: Q8_0 int8 -> fp32 (sign-extending byte select); 4-, 5- and 6-bit values
//     assembled in the low bits of an fp16 are subnormals (v * 2^-24), exact operands of v_dot2_f32_f16; MXFP4 E2M1
//     pairs -> fp16 with v_cvt_scalef32_pk_f16_fp4 feeding v_dot2_f32_f16; block scales (fp16 d, 6-bit K-quant
//     scales / mins, int8 Q6_K scales, E8M0) are applied once per unit in fp32;
//   * the per-lane sums of a row are reduced with four DPP adds inside 16 lanes (and a lane-swap add for 32-lane
//     rows); the results of a group leave as one store instruction;
//   * the fused decode paths hang on the two ends of the same kernel.  Staging modes: x * norm_weight with the RMSNorm
//     scale applied to the row sums at the store (a scalar commutes with the product, so no reduction precedes the
//     staging), silu(gate) * up of a [gate | up] row, and the GPT-OSS clamped SwiGLU with per-expert bias.  Store modes:
//     y = add + W x (residual), and the paired mode in which a wavefront computes gate row j and up row j of a stacked
//     [gate; up] weight side by side and stores silu(gate_j) * up_j.
//
// Arithmetic restated from TensorSharp.Models/ManagedQuantizedOps.cs:156-200 (dot of a dequantised row with the
// activation row); except for Q8_0 the activations of each unit are rounded to fp16 after a power-of-two scale of
// their own, so no input magnitude overflows or underflows fp16.
#include "tship_internal.h"

#include <algorithm>
#include <cstdlib>
#include <cstring>

namespace tship {
namespace {

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));

constexpr int kWaves = 8;          // wavefronts per workgroup
constexpr int kWgPerCu = 2;        // persistent workgroups per CU
constexpr int kThreads = kWaves * 64;
constexpr int kMaxGroup = 8;

// one GEMV
// activation modes: what the workgroup stages as x
constexpr int kActPlain = 0;      // x[k]
constexpr int kActRmsNorm = 1;    // (x[k] / sqrt(mean(x^2) + eps)) * norm_w[k]        (ggml_rms_norm, ggml_mul)
constexpr int kActSiluMul = 2;    // silu(x[k]) * x[K + k]: x is a [2K] gate|up row    (ggml_silu, ggml_mul)

struct GemvProblem {
    const uint8_t* w;
    int64_t w_bytes;
    const float* x;
    float* y;
    const float* add;         // optional: y = add + W x (may be y itself: residual accumulation)
    const float* norm_w;      // activation mode kActRmsNorm: the norm weight [K]
    float eps;
    float limit;
    int act;                  // how x is formed while it is staged (kAct*)
    const int* expert_id;     // optional (MoE): the weight is w + expert_id[0] * expert_stride
    int64_t expert_stride;
    int n_experts;            // ids outside [0, n_experts) select no weight: the problem reads zeros
    int pair_rows;            // F > 0: the weight holds F gate rows then F up rows and y[j] = glu(gate_j, up_j), j < F
    int pair_kind;            // glu of the paired mode: 0 silu(g) * u; 1 GPT-OSS (norm_w: optional [E][2F] bias indexed by
                              // expert_id, eps: alpha, limit: clamp), with plain activation staging only
    // routed sum (MoE down projection of one token): the rows of a group are row h of the 64 / LPR experts slot_ids[0..],
    // each with its own activation vector x + slot * K, and y[h] = sum_slot slot_w[slot] * (W[slot_ids[slot]][h] . x[slot] +
    // slot_bias[slot_ids[slot]][h]) added in slot order (GptOssModel.cs:718-735); slots whose id lies outside the table add nothing
    const int* slot_ids;      // null: off
    const float* slot_w;
    const float* slot_bias;   // optional [n_experts][N]
    int N;
    int K;
};

// up to kMaxGroup independent GEMVs served by one launch; workgroups [wg_begin[i], wg_begin[i+1])
// work on problem i.  Passed by value as the kernel argument (no device-side descriptor memory).
struct GemvGroup {
    GemvProblem p[kMaxGroup];
    int wg_begin[kMaxGroup + 1];
    int count;
    int strict;     // at most one step in flight per wavefront (launches long enough to saturate HBM)
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

#define TSHIP_DPP_F(v, ctrl) __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), ctrl, 0xf, 0xf, true))
constexpr int kDppXor1 = 0xb1;         // quad_perm [1,0,3,2]
constexpr int kDppXor2 = 0x4e;         // quad_perm [2,3,0,1]
constexpr int kDppHalfMirror = 0x141;  // lane i <-> 7-i inside each 8
constexpr int kDppMirror = 0x140;      // lane i <-> 15-i inside each 16

// Power-of-two pair (inverse, scale) that brings amax into [2^13, 2^14): fp16 keeps 11 bits for
// everything down to 2^-27 of the unit's largest magnitude and nothing overflows.
__device__ __forceinline__ void pow2_scale(float amax, float* inv, float* scale)
{
    int e = (int)((__float_as_uint(amax) >> 23) & 0xffu);
    if (e == 255) e = 127;  // inf / NaN activations: leave unscaled, they propagate
    if (e < 14) e = 14;
    const int se = e - 13;  // biased exponent of the scale, 1..241
    *scale = __uint_as_float((uint32_t)se << 23);
    *inv = __uint_as_float((uint32_t)(254 - se) << 23);
}

typedef uint32_t uint4_t __attribute__((ext_vector_type(4)));

// Range-checked loads through a buffer resource whose extent is the weight tensor: dwords past
// the end (and every dword of a deliberately out-of-range offset) read as zero instead of
// faulting, so the fetch code has no branches and the loads of two batches can stay in flight.
__device__ __forceinline__ void buf_load4(__amdgpu_buffer_rsrc_t rs, uint32_t voff, uint32_t soff, uint32_t* w)
{
    const uint4_t v = __builtin_amdgcn_raw_buffer_load_b128(rs, (int)voff, (int)soff, 0);
    w[0] = v.x; w[1] = v.y; w[2] = v.z; w[3] = v.w;
}
__device__ __forceinline__ uint32_t buf_load1(__amdgpu_buffer_rsrc_t rs, uint32_t voff, uint32_t soff)
{
    return __builtin_amdgcn_raw_buffer_load_b32(rs, (int)voff, (int)soff, 0);
}
constexpr uint32_t kDeadOffset = 0x80000000u;   // beyond any resource extent used here (< 2 GiB)

// ==========================================================================================
// Per-format pieces: LDS layout of x, staging, raw-unit load, unit dot product.
// ==========================================================================================

// ---- Q4_K ----------------------------------------------------------------------------------
// LDS unit (one 64-weight group, 144 B): 32 dwords of fp16 pairs in unpack order, then the fp32
// sums of the scaled fp16 activations of its two 32-weight sub-blocks, then the unit's scale.
// Unpack order of quant dword j (bytes 4j..4j+3 of the group's 32 quant bytes):
//   dword 4j+0 = (x[4j], x[4j+2])          low nibbles of bytes 0 and 2
//   dword 4j+1 = (x[4j+1], x[4j+3])        low nibbles of bytes 1 and 3
//   dword 4j+2 = (x[32+4j], x[32+4j+2])    high nibbles
//   dword 4j+3 = (x[32+4j+1], x[32+4j+3])
struct FmtQ4K {
    static constexpr int kLPR = 32;   // lanes per row: a step covers kLPR consecutive units of 64 / kLPR rows
    static constexpr int kUnitElems = 64;
    static constexpr int kLdsDwords = 36;
    static constexpr int kRegs = 12;

    static __device__ __forceinline__ int64_t row_bytes(int K) { return (int64_t)(K >> 8) * 144; }

    static constexpr int kStageF4 = 1;   // float4 loads per work item

    // work item `it` = activations [4*it, 4*it+4): byte offset of its float4
    static __device__ __forceinline__ void stage_offsets(int it, uint32_t (&off)[kStageF4]) { off[0] = (uint32_t)it * 16u; }

    // one work item = one float4; the 16 lanes of a DPP row share a unit.  Every workgroup converts the whole vector, so
    // the instruction count of this routine is launch time (K = 14336: 7 items per thread, 16 wavefronts per CU): the
    // largest magnitude is an integer maximum of the bit patterns (one DPP instruction per level, NaN / inf on top), the
    // sub-block sums come from two dot products with (1, 1).
    static __device__ __forceinline__ void stage_store(const float4 (&vv)[kStageF4], int it, bool live, uint32_t* lds)
    {
        const float4 v = vv[0];
        constexpr uint32_t kAbs = 0x7fffffffu;
        uint32_t m = max(max(__float_as_uint(v.x) & kAbs, __float_as_uint(v.y) & kAbs),
                         max(__float_as_uint(v.z) & kAbs, __float_as_uint(v.w) & kAbs));
        m = max(m, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)m, kDppXor1, 0xf, 0xf, true));
        m = max(m, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)m, kDppXor2, 0xf, 0xf, true));
        m = max(m, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)m, kDppHalfMirror, 0xf, 0xf, true));
        m = max(m, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)m, kDppMirror, 0xf, 0xf, true));
        float inv, scale;
        pow2_scale(__uint_as_float(m), &inv, &scale);
        const _Float16 h0 = (_Float16)(v.x * inv), h1 = (_Float16)(v.y * inv);
        const _Float16 h2 = (_Float16)(v.z * inv), h3 = (_Float16)(v.w * inv);
        H2U a, b;
        a.h = half2_t{h0, h2};
        b.h = half2_t{h1, h3};
        // sum of the four fp16 values in fp32
        float s = dot2(b.u, 0x3c003c00u, dot2(a.u, 0x3c003c00u, 0.f));
        // sum over the 8 lanes of one 32-weight sub-block
        s += TSHIP_DPP_F(s, kDppXor1);
        s += TSHIP_DPP_F(s, kDppXor2);
        s += TSHIP_DPP_F(s, kDppHalfMirror);
        if (live) {
            // item it = floats [4 it, 4 it + 4): unit it / 16, sub-block (it / 8) % 2, quant dword it % 8
            const int g = it >> 4, sub = (it >> 3) & 1, j = it & 7;
            uint32_t* unit = lds + g * kLdsDwords;
            uint2 w2;
            w2.x = a.u;
            w2.y = b.u;
            *reinterpret_cast<uint2*>(unit + 4 * j + 2 * sub) = w2;
            if ((it & 7) == 0) reinterpret_cast<float*>(unit)[32 + sub] = s;
            if ((it & 15) == 0) reinterpret_cast<float*>(unit)[34] = scale;
        }
    }
    static __device__ __forceinline__ int stage_items(int K) { return K >> 2; }

    static constexpr int kSlotBytes = kLPR / 4 * 144;   // kLPR consecutive units of a row

    // Lane-invariant part of the addressing: unit g = l16 + 16*step lives in super-block g/4 at
    // quant bytes (g & 3)*32; only the step / row-group part (a scalar) changes from step to step.
    struct Lane {
        uint32_t voff;    // byte offset of the lane's super-block: its row inside the group + inside the step
        uint32_t qoff;    // byte offset of the lane's 32 quant bytes inside the super-block
        int sh;           // bit position of the lane's scale pair inside the packed scale dwords
        bool upper;       // sub-blocks 4..7 use the split 4+2 bit encoding
    };
    static __device__ __forceinline__ Lane lane_setup(int sub, int l16, uint32_t row_bytes)
    {
        Lane L;
        L.voff = (uint32_t)sub * row_bytes + (uint32_t)(l16 >> 2) * 144u;
        L.qoff = 16u + (uint32_t)(l16 & 3) * 32u;
        L.sh = (l16 & 1) * 16;
        L.upper = (l16 & 2) != 0;
        return L;
    }

    // row_delta: (row start address) & 3, always 0 for Q4_K
    static __device__ __forceinline__ uint32_t load(__amdgpu_buffer_rsrc_t rs, const Lane& L, uint32_t soff,
                                                    uint32_t /*row_delta*/, int /*slot*/, bool live, uint32_t (&w)[kRegs])
    {
        const uint32_t hdr = live ? L.voff : kDeadOffset;
        const uint32_t q = hdr + L.qoff;
        buf_load4(rs, hdr, soff, &w[0]);
        buf_load4(rs, q, soff, &w[4]);
        buf_load4(rs, q + 16, soff, &w[8]);
        return 0;
    }

    static __device__ __forceinline__ float dot(const uint32_t (&w)[kRegs], const Lane& L, uint32_t /*aux*/,
                                                const uint32_t* xu_dw)
    {
        const uint4* xu = reinterpret_cast<const uint4*>(xu_dw);
        float lo = 0.f, hi = 0.f;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const uint4 xv = xu[j];
            const uint32_t q = w[4 + j];
            const uint32_t q8 = q >> 8;
            // a nibble left in place is an fp16 subnormal: q * 2^-24 (low) or 16q * 2^-24 (high);
            // v_dot2_f32_f16 honours fp16 denormals, so the integer values enter the dot exactly
            lo = dot2(q & 0x000f000fu, xv.x, lo);
            lo = dot2(q8 & 0x000f000fu, xv.y, lo);
            hi = dot2(q & 0x00f000f0u, xv.z, hi);
            hi = dot2(q8 & 0x00f000f0u, xv.w, hi);
        }
        const uint4 tail = xu[8];
        const float s1 = __uint_as_float(tail.x), s2 = __uint_as_float(tail.y), xscale = __uint_as_float(tail.z);
        // 6-bit scales / mins of the lane's two sub-blocks (ggml-quants.c:703-710), branch-free:
        // sub-blocks 0..3 keep 6 bits in place, 4..7 keep 4 bits in bytes 8..11 and 2 bits on top of bytes 0..7
        const uint32_t a = w[1] >> L.sh, b = w[2] >> L.sh, c = w[3] >> L.sh;
        const uint32_t sc_lo = a & 0x3f3fu, m_lo = b & 0x3f3fu;
        const uint32_t sc_hi = (c & 0x0f0fu) | ((a >> 2) & 0x3030u);
        const uint32_t m_hi = ((c >> 4) & 0x0f0fu) | ((b >> 2) & 0x3030u);
        const uint32_t sc = L.upper ? sc_hi : sc_lo, mn = L.upper ? m_hi : m_lo;
        const float sc1 = (float)(sc & 0xffu), sc2 = (float)(sc >> 8);
        const float m1 = (float)(mn & 0xffu), m2 = (float)(mn >> 8);
        const half2_t dm = as_half2(w[0]);
        const float d = (float)dm.x, dmin = (float)dm.y;
        // lo carries q * 2^-24, hi carries 16q * 2^-24
        const float dl = lo * 16777216.f, dh = hi * 1048576.f;
        return (d * (sc1 * dl + sc2 * dh) - dmin * (m1 * s1 + m2 * s2)) * xscale;
    }
};

// ---- Q5_K ------------------------------------------------------------------------------------
// Q4_K with a fifth bit: block of 176 bytes = d, dmin, 12 scale bytes, qh[32], qs[128] (ggml-quants.c
// dequantize_row_q5_K; ManagedQuantizedOps.cs:521-577).  Unit u = 64-weight group: its 32 quant bytes, and of every
// qh byte l the bits 2u (weight 64u + l) and 2u + 1 (weight 64u + 32 + l).  x in LDS, scales and mins: as FmtQ4K.
struct FmtQ5K : FmtQ4K {
    static constexpr int kRegs = 20;

    static __device__ __forceinline__ int64_t row_bytes(int K) { return (int64_t)(K >> 8) * 176; }
    static constexpr int kSlotBytes = kLPR / 4 * 176;

    struct Lane {
        uint32_t voff;    // the lane's super-block
        uint32_t qoff;    // its 32 quant bytes inside the super-block
        int sh;           // bit position of the lane's scale pair inside the packed scale dwords
        bool upper;       // sub-blocks 4..7 use the split 4+2 bit encoding
        int hsh;          // bit position of the group's pair of fifth bits inside a qh byte
    };
    static __device__ __forceinline__ Lane lane_setup(int sub, int l16, uint32_t row_bytes)
    {
        Lane L;
        L.voff = (uint32_t)sub * row_bytes + (uint32_t)(l16 >> 2) * 176u;
        L.qoff = 48u + (uint32_t)(l16 & 3) * 32u;
        L.sh = (l16 & 1) * 16;
        L.upper = (l16 & 2) != 0;
        L.hsh = (l16 & 3) * 2;
        return L;
    }

    static __device__ __forceinline__ uint32_t load(__amdgpu_buffer_rsrc_t rs, const Lane& L, uint32_t soff,
                                                    uint32_t /*row_delta*/, int /*slot*/, bool live, uint32_t (&w)[kRegs])
    {
        const uint32_t hdr = live ? L.voff : kDeadOffset;
        const uint32_t q = hdr + L.qoff;
        buf_load4(rs, hdr, soff, &w[0]);
        buf_load4(rs, hdr + 16, soff, &w[4]);      // qh, shared by the four groups of the super-block
        buf_load4(rs, hdr + 32, soff, &w[8]);
        buf_load4(rs, q, soff, &w[12]);
        buf_load4(rs, q + 16, soff, &w[16]);
        return 0;
    }

    static __device__ __forceinline__ float dot(const uint32_t (&w)[kRegs], const Lane& L, uint32_t /*aux*/,
                                                const uint32_t* xu_dw)
    {
        const uint4* xu = reinterpret_cast<const uint4*>(xu_dw);
        float lo = 0.f, hi = 0.f;
        constexpr uint32_t kNib = 0x000f000fu, kFifth = 0x00100010u;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const uint4 xv = xu[j];
            const uint32_t q = w[12 + j];
            const uint32_t h = w[4 + j] >> L.hsh;      // bit 0 of every byte: low-nibble weight, bit 1: high-nibble weight
            // a 5-bit value left in the low bits of an fp16 is the subnormal v * 2^-24
            lo = dot2((q & kNib) | ((h << 4) & kFifth), xv.x, lo);
            lo = dot2(((q >> 8) & kNib) | ((h >> 4) & kFifth), xv.y, lo);
            hi = dot2(((q >> 4) & kNib) | ((h << 3) & kFifth), xv.z, hi);
            hi = dot2(((q >> 12) & kNib) | ((h >> 5) & kFifth), xv.w, hi);
        }
        const uint4 tail = xu[8];
        const float s1 = __uint_as_float(tail.x), s2 = __uint_as_float(tail.y), xscale = __uint_as_float(tail.z);
        const uint32_t a = w[1] >> L.sh, b = w[2] >> L.sh, c = w[3] >> L.sh;
        const uint32_t sc_lo = a & 0x3f3fu, m_lo = b & 0x3f3fu;
        const uint32_t sc_hi = (c & 0x0f0fu) | ((a >> 2) & 0x3030u);
        const uint32_t m_hi = ((c >> 4) & 0x0f0fu) | ((b >> 2) & 0x3030u);
        const uint32_t sc = L.upper ? sc_hi : sc_lo, mn = L.upper ? m_hi : m_lo;
        const float sc1 = (float)(sc & 0xffu), sc2 = (float)(sc >> 8);
        const float m1 = (float)(mn & 0xffu), m2 = (float)(mn >> 8);
        const half2_t dm = as_half2(w[0]);
        const float d = (float)dm.x, dmin = (float)dm.y;
        return (d * ((sc1 * lo + sc2 * hi) * 16777216.f) - dmin * (m1 * s1 + m2 * s2)) * xscale;
    }
};

// ---- MXFP4 -----------------------------------------------------------------------------------
// LDS unit (one 32-weight block, 80 B): 16 dwords (x[j], x[j+16]) as fp16 pairs, then the unit's
// scale, then 12 B pad.
struct FmtMXFP4 {
    static constexpr int kLPR = 16;
    static constexpr int kUnitElems = 32;
    static constexpr int kLdsDwords = 20;
    static constexpr int kRegs = 5;

    static __device__ __forceinline__ int64_t row_bytes(int K) { return (int64_t)(K >> 5) * 17; }

    static constexpr int kStageF4 = 2;

    // one work item = x[b*32 + 4i .. +3] and x[b*32 + 16 + 4i .. +3]; the 4 lanes of a quad share a unit
    static __device__ __forceinline__ void stage_offsets(int it, uint32_t (&off)[kStageF4])
    {
        const uint32_t b = (uint32_t)it >> 2, i = (uint32_t)it & 3u;
        off[0] = (b * 32u + 4u * i) * 4u;
        off[1] = off[0] + 64u;
    }

    static __device__ __forceinline__ void stage_store(const float4 (&vv)[kStageF4], int it, bool live, uint32_t* lds)
    {
        const float4 lo = vv[0], hi = vv[1];
        float amax = fmaxf(fmaxf(fmaxf(fabsf(lo.x), fabsf(lo.y)), fmaxf(fabsf(lo.z), fabsf(lo.w))),
                           fmaxf(fmaxf(fabsf(hi.x), fabsf(hi.y)), fmaxf(fabsf(hi.z), fabsf(hi.w))));
        amax = fmaxf(amax, TSHIP_DPP_F(amax, kDppXor1));
        amax = fmaxf(amax, TSHIP_DPP_F(amax, kDppXor2));
        float inv, scale;
        pow2_scale(amax, &inv, &scale);
        if (live) {
            const int b = it >> 2, i = it & 3;
            uint4 o;
            o.x = pack_half2(lo.x * inv, hi.x * inv);
            o.y = pack_half2(lo.y * inv, hi.y * inv);
            o.z = pack_half2(lo.z * inv, hi.z * inv);
            o.w = pack_half2(lo.w * inv, hi.w * inv);
            uint32_t* unit = lds + b * kLdsDwords;
            *reinterpret_cast<uint4*>(unit + 4 * i) = o;
            if (i == 0) reinterpret_cast<float*>(unit)[16] = scale;
        }
    }
    static __device__ __forceinline__ int stage_items(int K) { return K >> 3; }

    static constexpr int kSlotBytes = kLPR * 17;

    struct Lane {
        uint32_t voff;   // byte offset of the lane's block: row inside the group + inside the step (before alignment)
    };
    static __device__ __forceinline__ Lane lane_setup(int sub, int l16, uint32_t row_bytes)
    {
        Lane L;
        L.voff = (uint32_t)sub * row_bytes + (uint32_t)l16 * 17u;
        return L;
    }

    // the 17 bytes of the block sit at byte (p & 3) of a 20-byte dword-aligned window;
    // row_delta = (row start address) & 3, slot*kSlotBytes keeps the same alignment as slot 0
    // only modulo 4, so the byte position is recomputed per step.  Returns p & 3.
    static __device__ __forceinline__ uint32_t load(__amdgpu_buffer_rsrc_t rs, const Lane& L, uint32_t soff,
                                                    uint32_t row_delta, int /*slot*/, bool live, uint32_t (&w)[kRegs])
    {
        const uint32_t p = L.voff + row_delta;          // relative to the 4-byte aligned row base + slot
        const uint32_t al = live ? (p & ~3u) : kDeadOffset;
        buf_load4(rs, al, soff, &w[0]);
        w[4] = buf_load1(rs, al + 16, soff);
        return p & 3u;
    }

    template <int SEL>
    static __device__ __forceinline__ uint32_t fp4_pair(uint32_t q)
    {
        H2U c;
        c.h = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(q, 1.0f, SEL);  // (low nibble, high nibble) as E2M1
        return c.u;
    }

    static __device__ __forceinline__ float dot(const uint32_t (&w)[kRegs], const Lane& /*L*/, uint32_t o,
                                                const uint32_t* xu_dw)
    {
        const uint32_t e = (w[0] >> (8 * o)) & 0xffu;
        // quant bytes start at byte o+1 of the aligned window
        const bool wrap = o == 3;
        const uint32_t b0 = wrap ? w[1] : w[0], b1 = wrap ? w[2] : w[1], b2 = wrap ? w[3] : w[2];
        const uint32_t b3 = wrap ? w[4] : w[3], b4 = w[4];
        const uint32_t shb = (o + 1) & 3;
        const uint32_t q0 = __builtin_amdgcn_alignbyte(b1, b0, shb);
        const uint32_t q1 = __builtin_amdgcn_alignbyte(b2, b1, shb);
        const uint32_t q2 = __builtin_amdgcn_alignbyte(b3, b2, shb);
        const uint32_t q3 = __builtin_amdgcn_alignbyte(b4, b3, shb);
        const uint4* xu = reinterpret_cast<const uint4*>(xu_dw);
        const uint4 x0 = xu[0], x1 = xu[1], x2 = xu[2], x3 = xu[3];
        const float xscale = __uint_as_float(xu[4].x);
        float s = 0.f, t = 0.f;
        s = dot2(fp4_pair<0>(q0), x0.x, s); t = dot2(fp4_pair<1>(q0), x0.y, t);
        s = dot2(fp4_pair<2>(q0), x0.z, s); t = dot2(fp4_pair<3>(q0), x0.w, t);
        s = dot2(fp4_pair<0>(q1), x1.x, s); t = dot2(fp4_pair<1>(q1), x1.y, t);
        s = dot2(fp4_pair<2>(q1), x1.z, s); t = dot2(fp4_pair<3>(q1), x1.w, t);
        s = dot2(fp4_pair<0>(q2), x2.x, s); t = dot2(fp4_pair<1>(q2), x2.y, t);
        s = dot2(fp4_pair<2>(q2), x2.z, s); t = dot2(fp4_pair<3>(q2), x2.w, t);
        s = dot2(fp4_pair<0>(q3), x3.x, s); t = dot2(fp4_pair<1>(q3), x3.y, t);
        s = dot2(fp4_pair<2>(q3), x3.z, s); t = dot2(fp4_pair<3>(q3), x3.w, t);
        // table value = 2 * E2M1, block scale = 2^(e-128) with the subnormal patterns of ggml_e8m0_to_fp32_half
        // (ggml-impl.h:471-489) for e < 2: exact for every code, 255 included
        const float bscale = __uint_as_float(e < 2 ? (0x00200000u << e) : ((e - 1u) << 23));
        // the activations' own scale first: the sums are of staged magnitude (up to 2^19), the block scale may be 2^127
        return ((s + t) * xscale) * 2.0f * bscale;
    }
};

// ---- Q4_0 / Q4_1 -----------------------------------------------------------------------------
// Blocks of 32 weights behind a small header: fp16 d (Q4_1 / Q5_1: also fp16 m; Q5_0 / Q5_1: also 32 fifth bits), then 16
// bytes whose low nibble is weight j and high nibble weight j + 16.  Values d * (q - 8), d * q + m, d * (q5 - 16),
// d * q5 + m, d * table[q] (ggml-quants.c dequantize_row_q4_0 / q4_1 / q5_0 / q5_1 / iq4_nl; ManagedQuantizedOps.cs:268-409,
// :559-577).
// LDS unit (80 B): for quant dword i, dwords 4i .. 4i+3 = (x[4i], x[4i+2]), (x[4i+1], x[4i+3]), then the same of
// x[16 + ..]; then the sum of the scaled fp16 activations and the unit's power-of-two scale.  Nibbles masked in place
// are fp16 subnormals (q * 2^-24, high nibbles 16 q * 2^-24) for v_dot2_f32_f16, a fifth bit joins them one bit above
// (bit 4 / bit 8), IQ4_NL's table values enter as bytes value + 128; the -8 / -16 / -128 / + m term leaves through the sum.
template <int TYPE>
struct FmtLegacy {
    static constexpr bool kMin = TYPE == kTypeQ4_1 || TYPE == kTypeQ5_1;
    static constexpr bool kFive = TYPE == kTypeQ5_0 || TYPE == kTypeQ5_1;
    static constexpr bool kTable = TYPE == kTypeIQ4_NL;
    static constexpr int kHdr = 2 + (kMin ? 2 : 0) + (kFive ? 4 : 0);      // bytes before the 16 quant bytes
    static constexpr int kLPR = 16;
    static constexpr int kUnitElems = 32;
    static constexpr int kLdsDwords = 20;
    static constexpr int kBlock = kHdr + 16;
    static constexpr int kRegs = (kBlock + 2 + 3) / 4;     // dwords of the window: the block at byte 0 or 2 of it

    static __device__ __forceinline__ int64_t row_bytes(int K) { return (int64_t)(K >> 5) * kBlock; }

    static constexpr int kStageF4 = 2;
    // one work item = x[b*32 + 4i .. +3] and x[b*32 + 16 + 4i .. +3]; the 4 lanes of a quad share a unit
    static __device__ __forceinline__ void stage_offsets(int it, uint32_t (&off)[kStageF4])
    {
        const uint32_t b = (uint32_t)it >> 2, i = (uint32_t)it & 3u;
        off[0] = (b * 32u + 4u * i) * 4u;
        off[1] = off[0] + 64u;
    }
    static __device__ __forceinline__ void stage_store(const float4 (&vv)[kStageF4], int it, bool live, uint32_t* lds)
    {
        const float4 lo = vv[0], hi = vv[1];
        float amax = fmaxf(fmaxf(fmaxf(fabsf(lo.x), fabsf(lo.y)), fmaxf(fabsf(lo.z), fabsf(lo.w))),
                           fmaxf(fmaxf(fabsf(hi.x), fabsf(hi.y)), fmaxf(fabsf(hi.z), fabsf(hi.w))));
        amax = fmaxf(amax, TSHIP_DPP_F(amax, kDppXor1));
        amax = fmaxf(amax, TSHIP_DPP_F(amax, kDppXor2));
        float inv, scale;
        pow2_scale(amax, &inv, &scale);
        const _Float16 a0 = (_Float16)(lo.x * inv), a1 = (_Float16)(lo.y * inv), a2 = (_Float16)(lo.z * inv), a3 = (_Float16)(lo.w * inv);
        const _Float16 b0 = (_Float16)(hi.x * inv), b1 = (_Float16)(hi.y * inv), b2 = (_Float16)(hi.z * inv), b3 = (_Float16)(hi.w * inv);
        float s = (((float)a0 + (float)a1) + ((float)a2 + (float)a3)) + (((float)b0 + (float)b1) + ((float)b2 + (float)b3));
        s += TSHIP_DPP_F(s, kDppXor1);
        s += TSHIP_DPP_F(s, kDppXor2);
        if (live) {
            const int b = it >> 2, i = it & 3;
            H2U p0, p1, p2, p3;
            p0.h = half2_t{a0, a2};
            p1.h = half2_t{a1, a3};
            p2.h = half2_t{b0, b2};
            p3.h = half2_t{b1, b3};
            uint4 o;
            o.x = p0.u;
            o.y = p1.u;
            o.z = p2.u;
            o.w = p3.u;
            uint32_t* unit = lds + b * kLdsDwords;
            *reinterpret_cast<uint4*>(unit + 4 * i) = o;
            if (i == 0) {
                reinterpret_cast<float*>(unit)[16] = s;
                reinterpret_cast<float*>(unit)[17] = scale;
            }
        }
    }
    static __device__ __forceinline__ int stage_items(int K) { return K >> 3; }

    static constexpr int kSlotBytes = kLPR * kBlock;

    struct Lane {
        uint32_t voff;
    };
    static __device__ __forceinline__ Lane lane_setup(int sub, int l16, uint32_t row_bytes)
    {
        Lane L;
        L.voff = (uint32_t)sub * row_bytes + (uint32_t)l16 * (uint32_t)kBlock;
        return L;
    }

    // the block sits at byte 0 or 2 of a dword-aligned window of kRegs dwords.  Returns p & 3.
    static __device__ __forceinline__ uint32_t load(__amdgpu_buffer_rsrc_t rs, const Lane& L, uint32_t soff,
                                                    uint32_t row_delta, int /*slot*/, bool live, uint32_t (&w)[kRegs])
    {
        const uint32_t p = L.voff + row_delta;
        const uint32_t al = live ? (p & ~3u) : kDeadOffset;
        buf_load4(rs, al, soff, &w[0]);
#pragma unroll
        for (int i = 4; i < kRegs; ++i) w[i] = buf_load1(rs, al + 4u * i, soff);
        return p & 3u;
    }

    // the aligned dword at byte `off` (a multiple of 2) of the block, which starts 0 (odd == false) or 2 bytes into w
    static __device__ __forceinline__ uint32_t at(const uint32_t (&w)[kRegs], bool odd, int off)
    {
        // even block: byte off of w; odd block: byte off + 2 of w
        const int e = off, o = off + 2;
        const uint32_t ve = (e & 3) ? __builtin_amdgcn_alignbyte(w[(e >> 2) + 1 < kRegs ? (e >> 2) + 1 : kRegs - 1], w[e >> 2], 2) : w[e >> 2];
        const uint32_t vo = (o & 3) ? __builtin_amdgcn_alignbyte(w[(o >> 2) + 1 < kRegs ? (o >> 2) + 1 : kRegs - 1], w[o >> 2], 2) : w[o >> 2];
        return odd ? vo : ve;
    }

    static __device__ __forceinline__ float dot(const uint32_t (&w)[kRegs], const Lane& /*L*/, uint32_t o, const uint32_t* xu_dw)
    {
        const bool odd = (o & 2u) != 0;
        const uint32_t hdr = at(w, odd, 0);                   // d | (m or the next two bytes) << 16
        H2U dh, mh;
        dh.u = hdr & 0xffffu;
        mh.u = kMin ? hdr >> 16 : 0u;
        const float d = (float)dh.h.x, m = (float)mh.h.x;
        const uint32_t qh = kFive ? at(w, odd, kMin ? 4 : 2) : 0u;
        const uint4* xu = reinterpret_cast<const uint4*>(xu_dw);
        float lo = 0.f, hi = 0.f;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t q = at(w, odd, kHdr + 4 * i);      // quant bytes 4i .. 4i + 3
            const uint4 xv = xu[i];
            if constexpr (kTable) {
                // {-127,-104,-83,-65,-49,-35,-22,-10, 1,13,25,38,53,69,89,113} + 128 as bytes, looked up with v_perm
                const uint32_t t0 = 0x3f2d1801u, t1 = 0x766a5d4fu, t2 = 0xa6998d81u, t3 = 0xf1d9c5b5u;
                uint32_t nl = q & 0x0f0f0f0fu, nh = (q >> 4) & 0x0f0f0f0fu;
                const uint32_t ml = ((nl >> 3) & 0x01010101u) * 0xffu, mh2 = ((nh >> 3) & 0x01010101u) * 0xffu;
                const uint32_t sl = nl & 0x07070707u, sh = nh & 0x07070707u;
                nl = (__builtin_amdgcn_perm(t3, t2, sl) & ml) | (__builtin_amdgcn_perm(t1, t0, sl) & ~ml);
                nh = (__builtin_amdgcn_perm(t3, t2, sh) & mh2) | (__builtin_amdgcn_perm(t1, t0, sh) & ~mh2);
                // bytes (0, 2) and (1, 3) into the low bytes of the two halves: subnormals (value + 128) * 2^-24
                lo = dot2(__builtin_amdgcn_perm(0u, nl, 0x0c020c00u), xv.x, lo);
                lo = dot2(__builtin_amdgcn_perm(0u, nl, 0x0c030c01u), xv.y, lo);
                hi = dot2(__builtin_amdgcn_perm(0u, nh, 0x0c020c00u), xv.z, hi);
                hi = dot2(__builtin_amdgcn_perm(0u, nh, 0x0c030c01u), xv.w, hi);
            } else {
                const uint32_t q8 = q >> 8;
                uint32_t a = q & 0x000f000fu, b = q8 & 0x000f000fu, c = q & 0x00f000f0u, e = q8 & 0x00f000f0u;
                if constexpr (kFive) {
                    // fifth bits of elements 4i .. 4i + 3 (bit 4 above a low nibble) and 16 + 4i .. (bit 8 above a high nibble)
                    const uint32_t t = qh >> (4 * i), u = qh >> (16 + 4 * i);
                    a |= ((t & 1u) << 4) | ((t & 4u) << 18);
                    b |= ((t & 2u) << 3) | ((t & 8u) << 17);
                    c |= ((u & 1u) << 8) | ((u & 4u) << 22);
                    e |= ((u & 2u) << 7) | ((u & 8u) << 21);
                }
                lo = dot2(a, xv.x, lo);
                lo = dot2(b, xv.y, lo);
                hi = dot2(c, xv.z, hi);
                hi = dot2(e, xv.w, hi);
            }
        }
        const uint4 tail = xu[4];
        const float sum = __uint_as_float(tail.x), xscale = __uint_as_float(tail.y);
        if constexpr (kTable) return d * ((lo + hi) * 16777216.f - 128.f * sum) * xscale;
        const float qx = lo * 16777216.f + hi * 1048576.f;
        return (kMin ? d * qx + m * sum : d * (qx - (kFive ? 16.f : 8.f) * sum)) * xscale;
    }
};

// ---- Q8_0 ------------------------------------------------------------------------------------
// LDS unit (one 32-weight block, 144 B): 32 fp32 activations, 16 B pad.  fp32 throughout.
struct FmtQ80 {
    static constexpr int kLPR = 16;
    static constexpr int kUnitElems = 32;
    static constexpr int kLdsDwords = 36;
    static constexpr int kRegs = 9;

    static __device__ __forceinline__ int64_t row_bytes(int K) { return (int64_t)(K >> 5) * 34; }

    static constexpr int kStageF4 = 1;

    static __device__ __forceinline__ void stage_offsets(int it, uint32_t (&off)[kStageF4]) { off[0] = (uint32_t)it * 16u; }

    static __device__ __forceinline__ void stage_store(const float4 (&vv)[kStageF4], int it, bool live, uint32_t* lds)
    {
        if (live) *reinterpret_cast<float4*>(lds + (it >> 3) * kLdsDwords + (it & 7) * 4) = vv[0];
    }
    static __device__ __forceinline__ int stage_items(int K) { return K >> 2; }

    static constexpr int kSlotBytes = kLPR * 34;

    struct Lane {
        uint32_t voff;
    };
    static __device__ __forceinline__ Lane lane_setup(int sub, int l16, uint32_t row_bytes)
    {
        Lane L;
        L.voff = (uint32_t)sub * row_bytes + (uint32_t)l16 * 34u;
        return L;
    }

    // the 34 bytes of the block sit at byte 0 or 2 of a 36-byte dword-aligned window. Returns p & 3.
    static __device__ __forceinline__ uint32_t load(__amdgpu_buffer_rsrc_t rs, const Lane& L, uint32_t soff,
                                                    uint32_t row_delta, int /*slot*/, bool live, uint32_t (&w)[kRegs])
    {
        const uint32_t p = L.voff + row_delta;
        const uint32_t al = live ? (p & ~3u) : kDeadOffset;
        buf_load4(rs, al, soff, &w[0]);
        buf_load4(rs, al + 16, soff, &w[4]);
        w[8] = buf_load1(rs, al + 32, soff);
        return p & 3u;
    }

    static __device__ __forceinline__ float dot4_i8(uint32_t q, float4 xv, float acc)
    {
        acc += (float)(int8_t)(q & 0xffu) * xv.x;
        acc += (float)(int8_t)((q >> 8) & 0xffu) * xv.y;
        acc += (float)(int8_t)((q >> 16) & 0xffu) * xv.z;
        acc += (float)(int8_t)(q >> 24) * xv.w;
        return acc;
    }

    static __device__ __forceinline__ float dot(const uint32_t (&w)[kRegs], const Lane& /*L*/, uint32_t o,
                                                const uint32_t* xu_dw)
    {
        // blocks are 2-byte aligned: the block starts at byte 0 or 2 of the aligned window
        const bool odd = (o & 2u) != 0;
        H2U dh;
        dh.u = odd ? (w[0] >> 16) : (w[0] & 0xffffu);
        const float d = (float)dh.h.x;
        const float4* xu = reinterpret_cast<const float4*>(xu_dw);
        float s0 = 0.f, s1 = 0.f;
#pragma unroll
        for (int i = 0; i < 8; i += 2) {
            const uint32_t qa = odd ? w[i + 1] : __builtin_amdgcn_alignbyte(w[i + 1], w[i], 2);
            const uint32_t qb = odd ? w[i + 2] : __builtin_amdgcn_alignbyte(w[i + 2], w[i + 1], 2);
            s0 = dot4_i8(qa, xu[i], s0);
            s1 = dot4_i8(qb, xu[i + 1], s1);
        }
        return (s0 + s1) * d;
    }
};

// ---- Q6_K ------------------------------------------------------------------------------------
// Block of 256 weights, 210 bytes: ql[128] low nibbles, qh[64] 2-bit tops, 16 int8 scales (one per 16 weights), fp16 d
// (ggml-quants.c dequantize_row_q6_K; ManagedQuantizedOps.cs:481-520).  Unit = 64 weights (n = half of the block,
// j = which 16 of its 32 columns): weights 128 n + 16 j + t + 32 r for t = 0..15 and run r = 0..3, held in
//   piece A = ql[64 n + 16 j + t]        low nibble -> run 0, high nibble -> run 2
//   piece B = ql[64 n + 32 + 16 j + t]   low nibble -> run 1, high nibble -> run 3
//   piece H = qh[32 n + 16 j + t]        bits 2r .. 2r+1 -> run r
// and scale[8 n + j + 2 r] for run r.  Blocks are 2-byte aligned, so each 16-byte piece is fetched as a 20-byte
// dword-aligned window and re-aligned in registers.
// LDS unit (176 B): for quant dword i of piece A, dwords 4i .. 4i+3 = (x[t], x[t+2]), (x[t+1], x[t+3]) of run 0, then
// the same of run 2 (t = 4 i); piece B (runs 1, 3) in dwords 16 .. 31; then the four runs' sums of the scaled fp16
// activations, then the four runs' power-of-two scales, 16 B pad (a 44-dword stride keeps ds_read_b128 conflict-free).
// A 6-bit value left in the low bits of an fp16 is the subnormal v * 2^-24, exact in v_dot2_f32_f16.
struct FmtQ6K {
    static constexpr int kLPR = 32;
    static constexpr int kUnitElems = 64;
    static constexpr int kLdsDwords = 44;
    static constexpr int kRegs = 19;

    static __device__ __forceinline__ int64_t row_bytes(int K) { return (int64_t)(K >> 8) * 210; }

    static constexpr int kStageF4 = 1;
    static __device__ __forceinline__ void stage_offsets(int it, uint32_t (&off)[kStageF4]) { off[0] = (uint32_t)it * 16u; }

    // one work item = 4 consecutive activations of one run; the 4 lanes of a quad share the run
    static __device__ __forceinline__ void stage_store(const float4 (&vv)[kStageF4], int it, bool live, uint32_t* lds)
    {
        const float4 v = vv[0];
        float amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
        amax = fmaxf(amax, TSHIP_DPP_F(amax, kDppXor1));
        amax = fmaxf(amax, TSHIP_DPP_F(amax, kDppXor2));
        float inv, scale;
        pow2_scale(amax, &inv, &scale);
        const _Float16 h0 = (_Float16)(v.x * inv), h1 = (_Float16)(v.y * inv);
        const _Float16 h2 = (_Float16)(v.z * inv), h3 = (_Float16)(v.w * inv);
        float s = ((float)h0 + (float)h1) + ((float)h2 + (float)h3);
        s += TSHIP_DPP_F(s, kDppXor1);
        s += TSHIP_DPP_F(s, kDppXor2);
        if (live) {
            const int e = it << 2;
            const int b = e >> 8, n = (e >> 7) & 1, r = (e >> 5) & 3, j = (e >> 4) & 1, i = (e >> 2) & 3;
            uint32_t* unit = lds + ((b * 2 + n) * 2 + j) * kLdsDwords;
            H2U lo, hi;
            lo.h = half2_t{h0, h2};
            hi.h = half2_t{h1, h3};
            uint2 w2;
            w2.x = lo.u;
            w2.y = hi.u;
            *reinterpret_cast<uint2*>(unit + (r & 1) * 16 + i * 4 + (r >> 1) * 2) = w2;
            if ((threadIdx.x & 3) == 0) {
                reinterpret_cast<float*>(unit)[32 + r] = s;
                reinterpret_cast<float*>(unit)[36 + r] = scale;
            }
        }
    }
    static __device__ __forceinline__ int stage_items(int K) { return K >> 2; }

    static constexpr int kSlotBytes = kLPR / 4 * 210;

    struct Lane {
        uint32_t voff;    // the lane's block: its row inside the group + inside the step
        uint32_t off_a;   // piece A inside the block (piece B is 32 bytes on)
        uint32_t off_h;   // piece H
        uint32_t off_s;   // the 8 scales of the lane's half
        int sc_shift;     // bit position of the scales of runs 0 and 2 inside their dwords (runs 1 and 3: 16 bits on)
    };
    static __device__ __forceinline__ Lane lane_setup(int sub, int l16, uint32_t row_bytes)
    {
        const uint32_t n = (uint32_t)(l16 >> 1) & 1u, j = (uint32_t)l16 & 1u;
        Lane L;
        L.voff = (uint32_t)sub * row_bytes + (uint32_t)(l16 >> 2) * 210u;
        L.off_a = 64u * n + 16u * j;
        L.off_h = 128u + 32u * n + 16u * j;
        L.off_s = 192u + 8u * n;
        L.sc_shift = (int)j * 8;
        return L;
    }

    // Every piece offset is a multiple of 4, so all windows share the block's byte position p & 3 (0 or 2), returned.
    static __device__ __forceinline__ uint32_t load(__amdgpu_buffer_rsrc_t rs, const Lane& L, uint32_t soff,
                                                    uint32_t row_delta, int /*slot*/, bool live, uint32_t (&w)[kRegs])
    {
        const uint32_t p = L.voff + row_delta;
        const uint32_t al = live ? (p & ~3u) : kDeadOffset;
        buf_load4(rs, al + L.off_a, soff, &w[0]);
        w[4] = buf_load1(rs, al + L.off_a + 16u, soff);
        buf_load4(rs, al + L.off_a + 32u, soff, &w[5]);
        w[9] = buf_load1(rs, al + L.off_a + 48u, soff);
        buf_load4(rs, al + L.off_h, soff, &w[10]);
        w[14] = buf_load1(rs, al + L.off_h + 16u, soff);
        w[15] = buf_load1(rs, al + L.off_s, soff);
        w[16] = buf_load1(rs, al + L.off_s + 4u, soff);
        w[17] = buf_load1(rs, al + L.off_s + 8u, soff);
        w[18] = buf_load1(rs, al + 208u, soff);
        return p & 3u;
    }

    static __device__ __forceinline__ float dot(const uint32_t (&w)[kRegs], const Lane& L, uint32_t o, const uint32_t* xu_dw)
    {
        const bool odd = (o & 2u) != 0;       // the block starts at byte 2 of its aligned window
        const uint4* xu = reinterpret_cast<const uint4*>(xu_dw);
        float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
        constexpr uint32_t kNib = 0x000f000fu, kTop = 0x00300030u;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t qa = odd ? __builtin_amdgcn_alignbyte(w[i + 1], w[i], 2) : w[i];
            const uint32_t qb = odd ? __builtin_amdgcn_alignbyte(w[i + 6], w[i + 5], 2) : w[i + 5];
            const uint32_t h = odd ? __builtin_amdgcn_alignbyte(w[i + 11], w[i + 10], 2) : w[i + 10];
            const uint4 xa = xu[i], xb = xu[4 + i];
            a0 = dot2((qa & kNib) | ((h << 4) & kTop), xa.x, a0);
            a0 = dot2(((qa >> 8) & kNib) | ((h >> 4) & kTop), xa.y, a0);
            a2 = dot2(((qa >> 4) & kNib) | (h & kTop), xa.z, a2);
            a2 = dot2(((qa >> 12) & kNib) | ((h >> 8) & kTop), xa.w, a2);
            a1 = dot2((qb & kNib) | ((h << 2) & kTop), xb.x, a1);
            a1 = dot2(((qb >> 8) & kNib) | ((h >> 6) & kTop), xb.y, a1);
            a3 = dot2(((qb >> 4) & kNib) | ((h >> 2) & kTop), xb.z, a3);
            a3 = dot2(((qb >> 12) & kNib) | ((h >> 10) & kTop), xb.w, a3);
        }
        // the half's 8 scale bytes: runs 0, 1 in bytes j, j + 2 of the first dword, runs 2, 3 of the second
        const uint32_t s01 = odd ? __builtin_amdgcn_alignbyte(w[16], w[15], 2) : w[15];
        const uint32_t s23 = odd ? __builtin_amdgcn_alignbyte(w[17], w[16], 2) : w[16];
        const float sc0 = (float)(int8_t)(s01 >> L.sc_shift), sc1 = (float)(int8_t)(s01 >> (L.sc_shift + 16));
        const float sc2 = (float)(int8_t)(s23 >> L.sc_shift), sc3 = (float)(int8_t)(s23 >> (L.sc_shift + 16));
        H2U dh;
        dh.u = odd ? (w[18] >> 16) : (w[18] & 0xffffu);
        const float d = (float)dh.h.x;
        const uint4 sums = xu[8], scl = xu[9];
        // a_r carries v * 2^-24; the stored value is v - 32
        const float t0 = (a0 * 16777216.f - 32.f * __uint_as_float(sums.x)) * __uint_as_float(scl.x);
        const float t1 = (a1 * 16777216.f - 32.f * __uint_as_float(sums.y)) * __uint_as_float(scl.y);
        const float t2 = (a2 * 16777216.f - 32.f * __uint_as_float(sums.z)) * __uint_as_float(scl.z);
        const float t3 = (a3 * 16777216.f - 32.f * __uint_as_float(sums.w)) * __uint_as_float(scl.w);
        return d * ((sc0 * t0 + sc1 * t1) + (sc2 * t2 + sc3 * t3));
    }
};

// ==========================================================================================
// The kernel body shared by all formats.
// ==========================================================================================
// Sum of a value over the LPR lanes of a row (16, 32 or 64 consecutive lanes); every lane of the row gets it.
template <int LPR>
__device__ __forceinline__ float row_sum(float v)
{
    typedef uint32_t u2_t __attribute__((ext_vector_type(2)));
    float t = v;
    t += TSHIP_DPP_F(t, kDppXor1);
    t += TSHIP_DPP_F(t, kDppXor2);
    t += TSHIP_DPP_F(t, kDppHalfMirror);
    t += TSHIP_DPP_F(t, kDppMirror);
    if (LPR >= 32) {     // 16-lane rows (r0 r1 r2 r3) swapped with themselves: (r0 r0 r2 r2) + (r1 r1 r3 r3)
        const u2_t a = __builtin_amdgcn_permlane16_swap(__float_as_uint(t), __float_as_uint(t), false, false);
        t = __uint_as_float(a.x) + __uint_as_float(a.y);
    }
    if (LPR == 64) {     // halves (lo hi): (lo lo) + (hi hi)
        const u2_t b = __builtin_amdgcn_permlane32_swap(__float_as_uint(t), __float_as_uint(t), false, false);
        t = __uint_as_float(b.x) + __uint_as_float(b.y);
    }
    return t;
}

// Sum of a double over the 64 lanes of a wavefront (every lane gets it): the permutations of row_sum on both halves of
// the value (register moves; a shuffle would make twelve trips through the LDS crossbar).
__device__ __forceinline__ double wave_sum_f64(double v)
{
    typedef uint32_t u2_t __attribute__((ext_vector_type(2)));
    auto moved = [](double d, auto perm) { return __hiloint2double(perm(__double2hiint(d)), perm(__double2loint(d))); };
    double t = v;
    t += moved(t, [](int x) { return __builtin_amdgcn_update_dpp(0, x, kDppXor1, 0xf, 0xf, true); });
    t += moved(t, [](int x) { return __builtin_amdgcn_update_dpp(0, x, kDppXor2, 0xf, 0xf, true); });
    t += moved(t, [](int x) { return __builtin_amdgcn_update_dpp(0, x, kDppHalfMirror, 0xf, 0xf, true); });
    t += moved(t, [](int x) { return __builtin_amdgcn_update_dpp(0, x, kDppMirror, 0xf, 0xf, true); });
    {
        const u2_t hi = __builtin_amdgcn_permlane16_swap((uint32_t)__double2hiint(t), (uint32_t)__double2hiint(t), false, false);
        const u2_t lo = __builtin_amdgcn_permlane16_swap((uint32_t)__double2loint(t), (uint32_t)__double2loint(t), false, false);
        t = __hiloint2double((int)hi.x, (int)lo.x) + __hiloint2double((int)hi.y, (int)lo.y);
    }
    {
        const u2_t hi = __builtin_amdgcn_permlane32_swap((uint32_t)__double2hiint(t), (uint32_t)__double2hiint(t), false, false);
        const u2_t lo = __builtin_amdgcn_permlane32_swap((uint32_t)__double2loint(t), (uint32_t)__double2loint(t), false, false);
        t = __hiloint2double((int)hi.x, (int)lo.x) + __hiloint2double((int)hi.y, (int)lo.y);
    }
    return t;
}

// A wavefront works on a group of 64 / LPR consecutive rows at a time, one row per LPR lanes (LPR = 16 unless the
// format says otherwise).
// One step = LPR consecutive units of each row of the group.  Steps of a wavefront are numbered group-major over
// (group, step); a step is fetched one step ahead of the compute.
template <typename F>
struct Step {
    uint32_t w[F::kRegs];
    uint32_t aux;     // format-specific lane datum produced by the load (byte position in its window)
    float extra;      // routed sum: the bias of the lane's slot for the group's row (leader lanes, first step)
    int step;         // uniform
    int group;        // uniform; >= ngroups marks a step past the end (its loads read zeros)
};

// ACT: the activation mode of every problem of the launch (compile time: the plain kernel carries none of
// the other modes' code or registers)
// TL: the timeline build of the kernel (diagnostics, see set_gemv_timeline): every wavefront leaves the 100 MHz
// constant-clock time of its entry, of the moment x is staged and of its exit in tl[]; the plain build has none of it.
// u64 per wavefront: entry, activations arrived, activations staged (behind the barrier), first weight step consumed, exit,
// (XCC id | problem << 8 | wavefront-in-launch << 16); the stamps stay in scalar registers until the exit, so that no store
// of theirs stands between the loads being timed
constexpr int kTimelineSlots = 8;
// EAGER > 0: the build for launches in which no wavefront has more than one row group and a group has at most EAGER
// steps.  Such a launch is all latency: with one step requested ahead a wavefront waits for memory once per step.
// Here the activations are requested first (so that their staging waits for nothing else: memory answers a wavefront
// in order), then every step of the wavefront's group at once, and the steps are consumed as they arrive.  Measured on
// one box against the streaming build: MXFP4 5760 x 2880 7.0 -> 6.0 us, 2880 x 2880 5.7 -> 5.0 us, Q4_K 4096 x 4096
// 5.9 -> 5.5 us; Q8_0 9728 x 2560 loses (9.9 -> 10.8 us) and has no eager build.
template <typename F, int ACT, bool TL, int EAGER>
__device__ __forceinline__ void gemv_body(const GemvProblem& P, int wg, int nwg, int mode, uint32_t* lds, uint64_t* tl, int prob)
{
    const int lane = threadIdx.x & 63;
    uint64_t t_entry = 0, t_x = 0, t_staged = 0, t_first = 0;
    if (TL) t_entry = __builtin_amdgcn_s_memrealtime();
    constexpr int LPR = F::kLPR, RPG = 64 / LPR;     // lanes per row, rows per group
    const int sub = lane / LPR, l16 = lane % LPR;    // row of the group, lane inside the row
    const int K = P.K;
    const int upr = K / F::kUnitElems;          // units per row
    const int nsteps = (upr + LPR - 1) / LPR;   // steps per row group
    // Plain: a group is RPG consecutive rows.  Paired (gate | up stacks of pair_rows rows each): a group is RPG / 2
    // consecutive gate rows in the lower half of the wavefront and the matching up rows in the upper half, so that gate j
    // and up j finish in lanes 32 apart and meet at the store.  (The other mapping - a group is RPG gate rows and then,
    // in the same lanes, their RPG up rows, the gate sums kept meanwhile, so that a wavefront's requests stay within one
    // stretch of rows - measured 0.3 us slower on a llama-3-8B decode layer and 1.0 us slower on a GPT-OSS token.)
    const int pair = P.pair_rows;                      // uniform
    constexpr int HALF = RPG / 2;
    const int gstep_plain = pair ? HALF : RPG;
    const int N = pair ? pair : P.N;                   // output rows
    const bool routed = P.slot_ids != nullptr;         // uniform; excludes pair and expert_id (the launcher sees to it)
    const int gstep = routed ? 1 : gstep_plain;        // output rows per group
    const int ngroups = (N + gstep - 1) / gstep;
    const int osub = routed ? 0 : pair ? sub % (HALF > 0 ? HALF : 1) : sub;          // the lane's output row inside the group
    const int lane_row = routed ? 0 : pair ? osub + (sub / (HALF > 0 ? HALF : 1)) * pair : sub;   // its weight row relative to the group's first
    const uint32_t row_bytes = (uint32_t)F::row_bytes(K);
    const int wave_stride = nwg * kWaves;
    const int gw = __builtin_amdgcn_readfirstlane(wg * kWaves + (int)(threadIdx.x >> 6));
    // The expert id is requested here and looked at after the activations have been requested: between the two lies a
    // memory round trip (a probe with a constant id: 2.2 us of a GPT-OSS token), which the activations' own then overlaps.
    const int eid_raw = P.expert_id ? P.expert_id[0] : 0;
    // x is requested first (it mostly hits L2 and memory answers a wavefront in order), then the
    // first weight steps, and only then is x converted into LDS - with the weights already in flight.
    const int kx = routed ? K * RPG : K;          // staged activations: one vector, or one per slot back to back
    const int items = F::stage_items(kx);
    const __amdgpu_buffer_rsrc_t xrs =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(P.x), 0, kx * 4, 0x00020000);
    // work items per thread per pass
    constexpr int kStageChunk = 8 / F::kStageF4;
    float4 xv[kStageChunk][F::kStageF4];
    // second operand of the activation modes: the norm weight (same offsets) or the "up" half (offsets + 4 K)
    constexpr int act = ACT;
    const __amdgpu_buffer_rsrc_t x2rs = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<float*>(act == kActRmsNorm ? P.norm_w : P.x + K), 0, K * 4, 0x00020000);
    float4 x2[kStageChunk][F::kStageF4];
    auto stage_issue = [&](int base) {
#pragma unroll
        for (int c = 0; c < kStageChunk; ++c) {
            const int it = base + c * kThreads + (int)threadIdx.x;
            uint32_t off[F::kStageF4];
            F::stage_offsets(it, off);
#pragma unroll
            for (int q = 0; q < F::kStageF4; ++q) {
                // items past the end fall outside the resource and read as zeros
                const uint4_t v = __builtin_amdgcn_raw_buffer_load_b128(xrs, (int)(it < items ? off[q] : kDeadOffset), 0, 0);
                xv[c][q] = float4{__uint_as_float(v.x), __uint_as_float(v.y), __uint_as_float(v.z), __uint_as_float(v.w)};
                if (act != kActPlain) {
                    const uint4_t u = __builtin_amdgcn_raw_buffer_load_b128(x2rs, (int)(it < items ? off[q] : kDeadOffset), 0, 0);
                    x2[c][q] = float4{__uint_as_float(u.x), __uint_as_float(u.y), __uint_as_float(u.z), __uint_as_float(u.w)};
                }
            }
        }
    };
    // kActRmsNorm: RMSNorm(x) * w = (x * w) * scale with the scalar scale = 1 / sqrt(mean(x^2) + eps), and a scalar
    // commutes with the matrix product.  So x * w is staged at once, each thread adds the squares of the values it
    // holds, and the scale meets the row sums at the store: no reduction and no barrier stands between the loads of x
    // and the staging.  (Sum of squares in double over fp32 squares, as ggml_rms_norm.)
    const int lds_units = (routed ? (RPG - 1) * upr : 0) + nsteps * LPR;               // unit slots the lanes may read
    double* red = reinterpret_cast<double*>(lds + lds_units * F::kLdsDwords);         // [kWaves], after the x area
    // four partial sums per thread, so that the double additions of a pass do not form one dependent chain
    double ss4[4] = {0.0, 0.0, 0.0, 0.0};
    auto apply_act = [&](int base) {
        if (act == kActRmsNorm) {
#pragma unroll
            for (int c = 0; c < kStageChunk; ++c) {
                if (base + c * kThreads >= items) continue;      // uniform: nothing was loaded for this chunk
#pragma unroll
                for (int q = 0; q < F::kStageF4; ++q) {
                    ss4[0] += (double)(xv[c][q].x * xv[c][q].x);
                    ss4[1] += (double)(xv[c][q].y * xv[c][q].y);
                    ss4[2] += (double)(xv[c][q].z * xv[c][q].z);
                    ss4[3] += (double)(xv[c][q].w * xv[c][q].w);
                    xv[c][q] = float4{xv[c][q].x * x2[c][q].x, xv[c][q].y * x2[c][q].y, xv[c][q].z * x2[c][q].z,
                                      xv[c][q].w * x2[c][q].w};
                }
            }
        } else if (act == kActSiluMul) {
            // hardware exp2 / reciprocal: relative error below 1e-5, far under the fp16 rounding the staged value gets
            // next (every workgroup evaluates the whole row, so the exact expf and division cost microseconds)
            auto silu = [](float g) { return g * __builtin_amdgcn_rcpf(1.0f + __expf(-g)); };
#pragma unroll
            for (int c = 0; c < kStageChunk; ++c)
#pragma unroll
                for (int q = 0; q < F::kStageF4; ++q)
                    xv[c][q] = float4{silu(xv[c][q].x) * x2[c][q].x, silu(xv[c][q].y) * x2[c][q].y,
                                      silu(xv[c][q].z) * x2[c][q].z, silu(xv[c][q].w) * x2[c][q].w};
        }
    };
    auto stage_commit = [&](int base) {
        if (act != kActPlain) apply_act(base);
#pragma unroll
        for (int c = 0; c < kStageChunk; ++c) {
            if (base + c * kThreads < items) {   // uniform
                const int it = base + c * kThreads + (int)threadIdx.x;
                F::stage_store(xv[c], it, it < items, lds);
            }
        }
    };

    stage_issue(0);
    __builtin_amdgcn_sched_barrier(0);       // the operands' loads stay ahead of everything that waits for the expert id
    // an expert id from the device is not trusted: one outside the table gets an empty resource (every load reads
    // zero, so the result row is the `add` term alone) instead of an address computed from it
    const int eid = P.expert_id ? __builtin_amdgcn_readfirstlane(eid_raw) : 0;
    const bool bad_expert = P.expert_id && (eid < 0 || eid >= P.n_experts);
    const uintptr_t w_begin = reinterpret_cast<uintptr_t>(P.w) + (P.expert_id && !bad_expert ? (uintptr_t)((int64_t)eid * P.expert_stride) : 0);
    // one range-checked resource for the whole tensor (host guarantees w_bytes < 2 GiB); the extent is
    // rounded up to whole dwords, which stay inside the last 4-byte word the tensor touches
    const uintptr_t base = w_begin & ~(uintptr_t)3;
    const uint32_t base_delta = (uint32_t)(w_begin & 3);
    const uint32_t extent = bad_expert ? 0u : ((uint32_t)P.w_bytes + base_delta + 3u) & ~3u;
    const __amdgpu_buffer_rsrc_t rs =
        __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>(base), 0, (int)extent, 0x00020000);
    typename F::Lane L = F::lane_setup(lane_row, l16, row_bytes);
    uint32_t lds_lane = (uint32_t)l16 * F::kLdsDwords;
    // routed sum: the lane's sub-row is a slot; its expert's matrix starts slot_id * expert_stride into the stack and
    // its activations are vector `slot` of the staged ones
    int slot_id = 0;
    bool slot_ok = true;
    // the four slot ids and weights come through the scalar cache in one round trip each (a per-lane load would stand in
    // front of every weight request, and memory answers a wavefront in order)
    typedef int int4v_t __attribute__((ext_vector_type(4)));
    typedef float float4v_t __attribute__((ext_vector_type(4)));
    int4v_t slot_id4 = {0, 0, 0, 0};
    float4v_t slot_w4 = {0.f, 0.f, 0.f, 0.f};
    if (routed) {
        if constexpr (RPG == 4) {
            asm volatile("s_load_dwordx4 %0, %2, 0x0\n\ts_load_dwordx4 %1, %3, 0x0\n\ts_waitcnt lgkmcnt(0)"
                         : "=&s"(slot_id4), "=&s"(slot_w4)
                         : "s"(P.slot_ids), "s"(P.slot_w)
                         : "memory");
        }
        slot_id = sub == 0 ? slot_id4.x : sub == 1 ? slot_id4.y : sub == 2 ? slot_id4.z : slot_id4.w;
        slot_ok = slot_id >= 0 && slot_id < P.n_experts;
        L.voff += slot_ok ? (uint32_t)slot_id * (uint32_t)P.expert_stride : 0u;
        lds_lane += (uint32_t)sub * (uint32_t)(upr * F::kLdsDwords);
    }

    // issue the loads of step (group, step); no waiting, no branches
    auto fetch = [&](int group, int step, Step<F>& st) {
        const bool group_ok = group < ngroups;                         // uniform
        const int row0 = group_ok ? group * gstep : 0;
        const uint32_t start = base_delta + (uint32_t)row0 * row_bytes + (uint32_t)step * F::kSlotBytes;
        const uint32_t soff = start & ~3u;                             // scalar part of the address
        const bool live = group_ok && (row0 + osub < N) && (l16 + step * LPR < upr) && slot_ok;
        st.step = step;
        st.group = group;
        st.aux = F::load(rs, L, soff, start & 3u, step, live, st.w);
        // routed sum: the slot's bias for this row rides with the group's first step
        st.extra = (routed && step == 0 && P.slot_bias && live && l16 == 0) ? P.slot_bias[(int64_t)slot_id * N + row0] : 0.f;
    };
    auto advance = [&](int& group, int& step) {
        if (++step == nsteps) {
            step = 0;
            group += wave_stride;
        }
    };

    // The first step of a wavefront is requested before x is staged, so weight latency overlaps the prologue; in the
    // loop the next step is requested before the current one is consumed.
    Step<F> cur, nxt;
    int fgroup = gw, fstep = 0;                // next step to fetch
    // deep: two steps requested before x is staged and two in flight afterwards.  Only the mode that evaluates a
    // function of two operands while staging uses it (their staging takes longer, and they are the short dependent
    // launches of a decode step: fused FFN 33.9 -> 32.2 us in an A/B on one box); plain launches lose (4096 x 14336
    // 12.7 -> 14.2 us) and so does the RMSNorm mode, whose staging is as short as the plain one (28672 x 4096 17.2 vs 16.0 us).
    const bool strict = mode == 1, deep = ACT == kActSiluMul && !strict;
    Step<F> eager[EAGER > 0 ? EAGER : 1];
    if constexpr (EAGER > 0) {
#pragma unroll
        for (int s = 0; s < EAGER; ++s) fetch(s < nsteps ? gw : ngroups, s, eager[s]);
    } else {
        // The activations (and the second operand of the activation modes) are asked for before the first weight step.
        // Asked for behind it they queue up behind the 37 MB that the launch's wavefronts request at the same moment -
        // the norm weight of the RMSNorm mode above all, which comes from HBM where the activations come from the launch
        // before: a probe that left the norm weight out gained 1.25 us per launch.  Measured on one box, weights first /
        // operands first: Q4_K 4096 x 14336 9.44 / 8.42 us, Q8_0 9728 x 2560 8.85 / 8.70, Q8_0 4096 x 4096 7.60 / 7.26, the
        // 123 MB grouped launch 23.31 / 23.24, a decode layer 47.7 / 46.2 (of which the norm weights 0.7).
        // (They are requested above, ahead of the expert id's use as well.)
        fetch(fgroup, fstep, cur);
        advance(fgroup, fstep);
        if (deep) {
            fetch(fgroup, fstep, nxt);
            advance(fgroup, fstep);
        }
    }
    if (TL && EAGER == 0) {
        // the first chunk of activations is in registers (the weight step requested before them has arrived too: memory
        // answers a wavefront in order)
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        t_x = __builtin_amdgcn_s_memrealtime();
    }
    stage_commit(0);
    for (int base = kThreads * kStageChunk; base < items; base += kThreads * kStageChunk) {
        stage_issue(base);
        stage_commit(base);
    }
    // lanes past the end of a row read their activations from the zero-filled tail of the last step
    for (int i = (kx / F::kUnitElems) * F::kLdsDwords + (int)threadIdx.x; i < lds_units * F::kLdsDwords; i += kThreads) lds[i] = 0u;
    if (act == kActRmsNorm) {
        const double ss = wave_sum_f64((ss4[0] + ss4[1]) + (ss4[2] + ss4[3]));
        if (lane == 0) red[threadIdx.x >> 6] = ss;
    }
    __syncthreads();
    if (TL) t_staged = __builtin_amdgcn_s_memrealtime();
    float out_scale = 1.0f;      // factor on every row sum
    if (act == kActRmsNorm) {
        double tot = 0.0;
#pragma unroll
        for (int i = 0; i < kWaves; ++i) tot += red[i];
        out_scale = 1.0f / sqrtf((float)(tot / (double)K) + P.eps);
    }

    float acc = 0.f, slot_b = 0.f;
    auto consume = [&](const Step<F>& st) {
        // lanes past the end of a row (and steps past the last group) hold zeros, zero scales included
        const uint32_t* xu = lds + lds_lane + (uint32_t)st.step * (uint32_t)(LPR * F::kLdsDwords);
        acc += F::dot(st.w, L, st.aux, xu);
        if (routed && st.step == 0) slot_b = st.extra;
        if (st.step == nsteps - 1) {   // uniform: the 4 rows of the group are complete
            float t = act == kActRmsNorm ? row_sum<LPR>(acc) * out_scale : row_sum<LPR>(acc);
            const int row = st.group * gstep + osub;
            bool writer = l16 == 0 && st.group < ngroups && row < N;
            if (routed) {
                // slot values sit in the leader lanes 0, LPR, 2 LPR, ...; the weighted sum runs in slot order
                const float v = t + slot_b;
                float o = 0.f;
#pragma unroll
                for (int sl = 0; sl < RPG; ++sl) {
                    const float vs = __shfl(v, sl * LPR);
                    const int id = slot_id4[sl & 3];                  // uniform
                    if (id >= 0 && id < P.n_experts) o = fmaf(slot_w4[sl & 3], vs, o);
                }
                t = o;
                writer = lane == 0 && st.group < ngroups;
            }
            if (pair) {
                const float up = __shfl_xor(t, 32);       // the up value sits 32 lanes above its gate value
                if (P.pair_kind == 0) {
                    // ggml_silu then ggml_mul (ggml-cpu/vec.h:958-960) on the fp32 sums
                    t = (t / (1.0f + expf(-t))) * up;
                } else {
                    // GptOssModel.cs:901-934: x = min(g + b_g, limit), y = clamp(u + b_u), x * sigmoid(alpha x) * (y + 1)
                    const bool biased = P.norm_w != nullptr && !bad_expert && writer;
                    const float* pb = P.norm_w + (int64_t)(P.expert_id ? eid : 0) * 2 * pair;
                    const float x = fminf(t + (biased ? pb[row] : 0.f), P.limit);
                    const float y = fminf(fmaxf(up + (biased ? pb[pair + row] : 0.f), -P.limit), P.limit);
                    t = (x / (1.0f + expf(P.eps * (-x)))) * (y + 1.0f);
                }
                writer = writer && lane < 32;
            }
            if (writer) P.y[row] = P.add ? P.add[row] + t : t;
            acc = 0.f;
        }
    };
    // Two steps per trip, the buffers swapping roles, so no step is ever copied between registers.
    // strict: a wavefront asks for its next step only once the previous one has arrived, so it never has more than
    // one step in flight and the wavefronts of the launch stay in step with each other.  Measured on one box
    // (strict / not): 123 MB grouped Q4_K launch 24.4 / 25.9 us, 559 MB Q8_0 matrix 92.0 / 98.7 us, but the fused
    // FFN's two launches (66 + 33 MB) 31.7 / 30.6 us and a whole layer 67.1 / 65.8 us: long launches that saturate
    // HBM lose bandwidth when requests run ahead, short ones gain from the extra overlap.
    auto one = [&](Step<F>& a, Step<F>& b) {
        if (strict) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        if (!deep) {
            fetch(fgroup, fstep, b);
            advance(fgroup, fstep);
        }
        consume(a);
        if (deep) {
            fetch(fgroup, fstep, a);
            advance(fgroup, fstep);
        }
    };
    if constexpr (EAGER > 0) {
#pragma unroll
        for (int s = 0; s < EAGER; ++s) {
            if (s < nsteps) consume(eager[s]);       // uniform
            if (TL && s == 0) t_first = __builtin_amdgcn_s_memrealtime();
        }
    } else {
        for (;;) {
            if (cur.group >= ngroups) break;
            one(cur, nxt);
            if (TL && t_first == 0) t_first = __builtin_amdgcn_s_memrealtime();
            if (nxt.group >= ngroups) break;
            one(nxt, cur);
        }
    }
    if (TL) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");       // the last stores have been acknowledged
        const uint64_t t_exit = __builtin_amdgcn_s_memrealtime();
        if (lane == 0) {
            const int wave_in_launch = (int)blockIdx.x * kWaves + (int)(threadIdx.x >> 6);
            uint64_t* my_tl = tl + (size_t)wave_in_launch * kTimelineSlots;
            my_tl[0] = t_entry, my_tl[1] = t_x, my_tl[2] = t_staged, my_tl[3] = t_first, my_tl[4] = t_exit;
            // hardware register 20 (XCC_ID), 4 bits from bit 0
            my_tl[5] = (uint64_t)(__builtin_amdgcn_s_getreg((3 << 11) | 20) & 0xfu) | ((uint64_t)prob << 8) | ((uint64_t)wave_in_launch << 16);
        }
    }
}

// The workgroup -> problem table and the flags travel as the kernel's first scalar arguments: built with
// -amdgpu-kernarg-preload-count the hardware delivers them in SGPRs at wave launch, so a workgroup knows its problem
// without a memory round trip and the one scalar load left (the problem's fields) is issued at once.
// What a workgroup needs before its first weight request, 32 bytes per problem (64 with expert indirection) at the head of
// the argument block: one scalar load instead of one per field.
struct GemvEarly {
    const uint8_t* w;
    const float* x;
    int N, K;
    uint32_t w_bytes;
    int pair_rows;
    // problems whose weight is chosen by an expert id read on the device
    const int* expert_id;
    int64_t expert_stride;
    int n_experts;
    int pair_kind;
    int64_t pad;
};
static_assert(sizeof(GemvEarly) == 64, "at most one 16-dword scalar load");
// (The size of the argument block does not matter: plain launches with a 512-byte block of their own instead of these
// 1.5 KB measured the same 23.2 us and the same gap between launches.)
struct GemvProblems {
    GemvEarly e[kMaxGroup];
    GemvProblem p[kMaxGroup];
};
// EARLY 1: no problem of the launch has expert indirection, a paired store or a routed sum; 2: every problem has expert
// indirection and none a routed sum (the streaming build then takes its first fields from the early records and has the
// absent features switched off at compile time); 0: fields read where the code needs them
template <int TYPE, int ACT, bool TL, int EAGER, int EARLY>
__global__ void __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(4))) gemv_kernel(int b0, int b1, int b2, int b3, int b4, int b5, int b6, int b7, int b8, int count,
                                                        int strict, const GemvProblems G, uint64_t* tl)
{
    static_assert(kMaxGroup == 8, "one scalar argument per table entry");
    extern __shared__ uint32_t lds[];
    const int bx = (int)blockIdx.x;
    int i = 0, lo = b0, hi = b1;
    if (1 < count && bx >= b1) { i = 1; lo = b1; hi = b2; }
    if (2 < count && bx >= b2) { i = 2; lo = b2; hi = b3; }
    if (3 < count && bx >= b3) { i = 3; lo = b3; hi = b4; }
    if (4 < count && bx >= b4) { i = 4; lo = b4; hi = b5; }
    if (5 < count && bx >= b5) { i = 5; lo = b5; hi = b6; }
    if (6 < count && bx >= b6) { i = 6; lo = b6; hi = b7; }
    if (7 < count && bx >= b7) { i = 7; lo = b7; hi = b8; }
    const int wg = bx - lo, nwg = hi - lo;
    // Read where the code first needs them, the problem's fields cost one dependent scalar load after the other (seven
    // before the first weight request, about 1 us).  Eager build: the whole struct in one round trip, pinned in SGPRs.
    // Streaming build: the early record in one load and the rest where it is used.  (Pinning the whole struct as the eager
    // build does starts the streaming build 1 us earlier too, by the per-wavefront timeline, but its loop then runs 10 %
    // slower - 123 MB grouped launch 25.1 against 24.4 us - where the early record gives 23.4.)
    GemvProblem Pv;
    if constexpr (EAGER > 0) {
        Pv = G.p[i];
        uint64_t w = reinterpret_cast<uint64_t>(Pv.w), x = reinterpret_cast<uint64_t>(Pv.x), y = reinterpret_cast<uint64_t>(Pv.y);
        uint64_t add = reinterpret_cast<uint64_t>(Pv.add), nw = reinterpret_cast<uint64_t>(Pv.norm_w), eid = reinterpret_cast<uint64_t>(Pv.expert_id);
        uint64_t si = reinterpret_cast<uint64_t>(Pv.slot_ids), sw = reinterpret_cast<uint64_t>(Pv.slot_w), sb = reinterpret_cast<uint64_t>(Pv.slot_bias);
        asm volatile("" : "+s"(si), "+s"(sw), "+s"(sb));
        Pv.slot_ids = reinterpret_cast<const int*>(si), Pv.slot_w = reinterpret_cast<const float*>(sw), Pv.slot_bias = reinterpret_cast<const float*>(sb);
        asm volatile("" : "+s"(w), "+s"(x), "+s"(y), "+s"(add), "+s"(nw), "+s"(eid), "+s"(Pv.w_bytes), "+s"(Pv.expert_stride));
        asm volatile("" : "+s"(Pv.N), "+s"(Pv.K), "+s"(Pv.pair_rows), "+s"(Pv.pair_kind), "+s"(Pv.n_experts), "+s"(Pv.eps), "+s"(Pv.limit));
        Pv.w = reinterpret_cast<const uint8_t*>(w), Pv.x = reinterpret_cast<const float*>(x), Pv.y = reinterpret_cast<float*>(y);
        Pv.add = reinterpret_cast<const float*>(add), Pv.norm_w = reinterpret_cast<const float*>(nw), Pv.expert_id = reinterpret_cast<const int*>(eid);
    }
    if constexpr (EAGER == 0 && EARLY == 1) {
        const GemvEarly E = G.e[i];
        Pv.w = E.w, Pv.x = E.x, Pv.N = E.N, Pv.K = E.K, Pv.w_bytes = (int64_t)E.w_bytes;
        Pv.y = G.p[i].y, Pv.add = G.p[i].add, Pv.norm_w = G.p[i].norm_w, Pv.eps = G.p[i].eps, Pv.limit = 0.f, Pv.act = ACT;
        Pv.expert_id = nullptr, Pv.expert_stride = 0, Pv.n_experts = 0, Pv.pair_rows = 0, Pv.pair_kind = 0;
        Pv.slot_ids = nullptr, Pv.slot_w = nullptr, Pv.slot_bias = nullptr;
    }
    if constexpr (EAGER == 0 && EARLY == 2) {
        const GemvEarly E = G.e[i];
        Pv.w = E.w, Pv.x = E.x, Pv.N = E.N, Pv.K = E.K, Pv.w_bytes = (int64_t)E.w_bytes, Pv.pair_rows = E.pair_rows;
        Pv.expert_id = E.expert_id, Pv.expert_stride = E.expert_stride, Pv.n_experts = E.n_experts, Pv.pair_kind = E.pair_kind;
        Pv.y = G.p[i].y, Pv.add = G.p[i].add, Pv.norm_w = G.p[i].norm_w, Pv.eps = G.p[i].eps, Pv.limit = G.p[i].limit, Pv.act = ACT;
        Pv.slot_ids = nullptr, Pv.slot_w = nullptr, Pv.slot_bias = nullptr;
    }
    // (a launch that mixes the features keeps the lazy reads)
    const GemvProblem& P = (EAGER > 0 || EARLY != 0) ? Pv : G.p[i];
    if (TYPE == kTypeQ4_K) gemv_body<FmtQ4K, ACT, TL, EAGER>(P, wg, nwg, strict, lds, tl, i);
    else if (TYPE == kTypeMXFP4) gemv_body<FmtMXFP4, ACT, TL, EAGER>(P, wg, nwg, strict, lds, tl, i);
    else if (TYPE == kTypeQ6_K) gemv_body<FmtQ6K, ACT, TL, EAGER>(P, wg, nwg, strict, lds, tl, i);
    else if (TYPE == kTypeQ5_K) gemv_body<FmtQ5K, ACT, TL, EAGER>(P, wg, nwg, strict, lds, tl, i);
    else if (TYPE == kTypeQ4_0 || TYPE == kTypeQ4_1 || TYPE == kTypeQ5_0 || TYPE == kTypeQ5_1 || TYPE == kTypeIQ4_NL)
        gemv_body<FmtLegacy<TYPE>, ACT, TL, EAGER>(P, wg, nwg, strict, lds, tl, i);
    else gemv_body<FmtQ80, ACT, TL, EAGER>(P, wg, nwg, strict, lds, tl, i);
}

// A launch of ONE problem without expert indirection: everything the kernel needs before its first weight request -
// weight, activations, result, sizes, the residual and the norm weight, and one word with the mode (bits 0..1), the kind
// of paired store (bits 2..3) and its row count (bits 4..) - are the first scalar arguments, which the hardware delivers
// in SGPRs at wave launch (14 dwords).  No scalar load stands between entry and that request; read one after the other
// from the argument block, as the grouped kernel must (its problem depends on the workgroup), the fields cost 1 - 1.8 us
// per launch (Q4_K 14336 x 4096 10.2 -> 8.4 us, 4096 x 4096 6.0 -> 4.8, MXFP4 5760 x 2880 6.4 -> 5.2, a decode layer
// 52.8 -> 49.2 us).  eps and limit are read where the code reaches them.
// (PAIR as a compile-time switch: with the row count of the paired store as a run-time value the plain launches carry its
// code and measured 0.1 - 0.25 us slower.)
constexpr int kOnePairShift = 4;
template <int TYPE, int ACT, bool TL, int EAGER, bool PAIR>
__global__ void __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(4))) gemv_one_kernel(
    const uint8_t* w, const float* x, float* y, int N, int K, int w_bytes, int flags, const float* add, const float* norm_w,
    float eps, float limit, uint64_t* tl)
{
    extern __shared__ uint32_t lds[];
    GemvProblem Pv;
    Pv.w = w, Pv.x = x, Pv.y = y, Pv.N = N, Pv.K = K, Pv.w_bytes = (int64_t)(uint32_t)w_bytes, Pv.add = add, Pv.norm_w = norm_w;
    Pv.act = ACT;
    Pv.eps = eps, Pv.limit = limit;
    Pv.expert_id = nullptr, Pv.expert_stride = 0, Pv.n_experts = 0;
    Pv.pair_rows = PAIR ? (int)((uint32_t)flags >> kOnePairShift) : 0, Pv.pair_kind = PAIR ? (flags >> 2) & 3 : 0;
    Pv.slot_ids = nullptr, Pv.slot_w = nullptr, Pv.slot_bias = nullptr;
    const int strict = flags & 3, wg = (int)blockIdx.x, nwg = (int)gridDim.x;
    if (TYPE == kTypeQ4_K) gemv_body<FmtQ4K, ACT, TL, EAGER>(Pv, wg, nwg, strict, lds, tl, 0);
    else if (TYPE == kTypeMXFP4) gemv_body<FmtMXFP4, ACT, TL, EAGER>(Pv, wg, nwg, strict, lds, tl, 0);
    else if (TYPE == kTypeQ6_K) gemv_body<FmtQ6K, ACT, TL, EAGER>(Pv, wg, nwg, strict, lds, tl, 0);
    else if (TYPE == kTypeQ5_K) gemv_body<FmtQ5K, ACT, TL, EAGER>(Pv, wg, nwg, strict, lds, tl, 0);
    else if (TYPE == kTypeQ4_0 || TYPE == kTypeQ4_1 || TYPE == kTypeQ5_0 || TYPE == kTypeQ5_1 || TYPE == kTypeIQ4_NL)
        gemv_body<FmtLegacy<TYPE>, ACT, TL, EAGER>(Pv, wg, nwg, strict, lds, tl, 0);
    else gemv_body<FmtQ80, ACT, TL, EAGER>(Pv, wg, nwg, strict, lds, tl, 0);
}

// The routed sum of one token (MoE decode: down projections + weighted sum) as a launch of its own argument list: the
// stack of expert matrices, the staged activation vectors, the slot tables and the geometry are the preloaded scalars; the
// result pointer and the bias are read where the code reaches them.
template <int TYPE>
__global__ void __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(4))) gemv_routed_kernel(
    const uint8_t* w, const float* x, int N, int K, int w_bytes, int flags, const int* slot_ids, const float* slot_w, int expert_stride,
    float* y, const float* slot_bias)
{
    extern __shared__ uint32_t lds[];
    GemvProblem Pv;
    Pv.w = w, Pv.x = x, Pv.y = y, Pv.N = N, Pv.K = K, Pv.w_bytes = (int64_t)(uint32_t)w_bytes, Pv.add = nullptr, Pv.norm_w = nullptr;
    Pv.act = kActPlain, Pv.eps = 0.f, Pv.limit = 0.f;
    Pv.expert_id = nullptr, Pv.expert_stride = (int64_t)(uint32_t)expert_stride, Pv.n_experts = (int)((uint32_t)flags >> 8);
    Pv.pair_rows = 0, Pv.pair_kind = 0;
    Pv.slot_ids = slot_ids, Pv.slot_w = slot_w, Pv.slot_bias = slot_bias;
    const int strict = flags & 3, wg = (int)blockIdx.x, nwg = (int)gridDim.x;
    if (TYPE == kTypeMXFP4) gemv_body<FmtMXFP4, kActPlain, false, 0>(Pv, wg, nwg, strict, lds, nullptr, 0);
    else gemv_body<FmtQ80, kActPlain, false, 0>(Pv, wg, nwg, strict, lds, nullptr, 0);
}

int unit_elems(int type) { return type == kTypeQ4_K || type == kTypeQ5_K || type == kTypeQ6_K ? 64 : 32; }
bool legacy_type(int type) { return type == kTypeQ4_0 || type == kTypeQ4_1 || type == kTypeQ5_0 || type == kTypeQ5_1 || type == kTypeIQ4_NL; }
int unit_lds_bytes(int type) { return type == kTypeMXFP4 || legacy_type(type) ? 80 : type == kTypeQ6_K ? 176 : 144; }
int lanes_per_row(int type)
{
    return type == kTypeQ4_K || type == kTypeQ5_K ? FmtQ4K::kLPR : type == kTypeMXFP4 ? FmtMXFP4::kLPR : type == kTypeQ6_K ? FmtQ6K::kLPR : FmtQ80::kLPR;
}

// x staged as whole steps of 16 units (the tail of the last step is zero-filled); routed sums stage one vector per slot
size_t lds_bytes_for(int type, int K, bool routed = false)
{
    const int lpr = lanes_per_row(type), upr = K / unit_elems(type);
    const size_t units = (size_t)((upr + lpr - 1) / lpr) * lpr + (routed ? (size_t)(64 / lpr - 1) * upr : 0);
    // + the RMSNorm reduction slots
    return units * unit_lds_bytes(type) + kWaves * sizeof(double);
}

constexpr size_t kMaxLds = 160 * 1024 - 1024;
constexpr double kStrictBytes = 96.0 * 1024 * 1024;   // launches streaming at least this much run strict (see gemv_body)

// Diagnostics: while a buffer is set, plain-activation launches run the timeline build of the kernel and leave
// kTimelineSlots stamps per wavefront in it (the last launch wins).  Not thread-safe; meant for a profiling run.
uint64_t* g_timeline = nullptr;
int64_t g_timeline_waves = 0;

template <int TYPE, int ACT, bool TL, int EAGER>
bool launch_type_tl(const GemvGroup& g, int grid, size_t lds, hipStream_t stream)
{
    if constexpr ((TYPE == kTypeMXFP4 || TYPE == kTypeQ8_0) && ACT == kActPlain && !TL && EAGER == 0) {
        const GemvProblem& p = g.p[0];
        if (g.count == 1 && p.slot_ids && !p.expert_id && !p.pair_rows && !p.add && p.n_experts < (1 << 23) &&
            p.expert_stride < ((int64_t)1 << 31)) {
            auto kern = gemv_routed_kernel<TYPE>;
            if (!raise_lds_limit(reinterpret_cast<const void*>(kern), lds)) return false;
            hipLaunchKernelGGL(kern, dim3(grid), dim3(kThreads), lds, stream, p.w, p.x, p.N, p.K, (int)(uint32_t)p.w_bytes,
                               (g.strict & 3) | (p.n_experts << 8), p.slot_ids, p.slot_w, (int)p.expert_stride, p.y, p.slot_bias);
            return hip_ok(hipGetLastError(), "gemv launch");
        }
    }
    if (g.count == 1 && !g.p[0].expert_id && !g.p[0].slot_ids &&
        g.p[0].pair_rows < (1 << (31 - kOnePairShift)) && g.p[0].pair_kind >= 0 && g.p[0].pair_kind < 4) {
        const GemvProblem& p = g.p[0];
        const int flags = (g.strict & 3) | (p.pair_kind << 2) | (int)((uint32_t)p.pair_rows << kOnePairShift);
        auto launch_one = [&](auto one) {
            if (!raise_lds_limit(reinterpret_cast<const void*>(one), lds)) return false;
            hipLaunchKernelGGL(one, dim3(grid), dim3(kThreads), lds, stream, p.w, p.x, p.y, p.N, p.K, (int)(uint32_t)p.w_bytes, flags, p.add,
                               p.norm_w, p.eps, p.limit, TL ? g_timeline : nullptr);
            return hip_ok(hipGetLastError(), "gemv launch");
        };
        // (one problem with a paired store and no expert indirection: the gate | up launch of the fused FFN, RMSNorm staging)
        if constexpr (!TL && EAGER == 0 && ACT == kActRmsNorm) {
            if (p.pair_rows) return launch_one(gemv_one_kernel<TYPE, ACT, TL, EAGER, true>);
        }
        if (!p.pair_rows) return launch_one(gemv_one_kernel<TYPE, ACT, TL, EAGER, false>);
    }
    GemvProblems gp;
    std::memcpy(gp.p, g.p, sizeof(gp.p));
    bool simple = EAGER == 0, expert = EAGER == 0;
    for (int i = 0; i < kMaxGroup; ++i) {
        const GemvProblem& p = g.p[i];
        gp.e[i] = GemvEarly{p.w, p.x, p.N, p.K, (uint32_t)p.w_bytes, p.pair_rows, p.expert_id, p.expert_stride, p.n_experts, p.pair_kind, 0};
        if (i < g.count) {
            simple = simple && !p.expert_id && !p.pair_rows && !p.slot_ids;
            expert = expert && p.expert_id && !p.slot_ids;
        }
    }
    auto launch = [&](auto kern) {
        if (!raise_lds_limit(reinterpret_cast<const void*>(kern), lds)) return false;
        hipLaunchKernelGGL(kern, dim3(grid), dim3(kThreads), lds, stream, g.wg_begin[0], g.wg_begin[1], g.wg_begin[2], g.wg_begin[3],
                           g.wg_begin[4], g.wg_begin[5], g.wg_begin[6], g.wg_begin[7], g.wg_begin[8], g.count, g.strict, gp,
                           TL ? g_timeline : nullptr);
        return hip_ok(hipGetLastError(), "gemv launch");
    };
    // (RMSNorm staging only ever comes as one problem per launch: it has the one-problem kernels above)
    if constexpr (EAGER == 0 && ACT != kActRmsNorm) {
        if (simple) return launch(gemv_kernel<TYPE, ACT, TL, EAGER, 1>);
    }
    // (expert indirection goes with plain staging: the MoE decode launches)
    constexpr bool kExpertRecords = EAGER == 0 && ACT == kActPlain && !TL && (TYPE == kTypeMXFP4 || TYPE == kTypeQ8_0 || TYPE == kTypeQ4_K);
    if constexpr (kExpertRecords) {
        if (expert) return launch(gemv_kernel<TYPE, ACT, TL, EAGER, 2>);
    }
    // The build that reads every field where it needs it serves what is left: the eager builds (they take the whole
    // problem in one load anyway) and expert indirection for the formats without early expert records.  Other
    // combinations are not instantiated.
    if constexpr (EAGER > 0 || (ACT == kActPlain && !TL && !kExpertRecords)) {
        return launch(gemv_kernel<TYPE, ACT, TL, EAGER, 0>);
    } else {
        set_last_error("gemv: no kernel for this combination of problems (activation mode, paired store, expert indirection).");
        return false;
    }
}

// steps the eager build of a format holds in registers (0: the format has no eager build)
template <int TYPE>
constexpr int kEagerSteps = TYPE == kTypeQ4_K ? 4 : TYPE == kTypeMXFP4 ? 6 : 0;
int eager_steps(int type)
{
    return type == kTypeQ4_K ? kEagerSteps<kTypeQ4_K> : type == kTypeMXFP4 ? kEagerSteps<kTypeMXFP4> : 0;
}

template <int TYPE, int ACT>
bool launch_type(const GemvGroup& g, int grid, size_t lds, hipStream_t stream)
{
    // (the timeline build stamps launches of plain problems only)
    bool plain = true;
    for (int i = 0; i < g.count; ++i) plain = plain && !g.p[i].expert_id && !g.p[i].pair_rows && !g.p[i].slot_ids;
    const bool tl = ACT == kActPlain && plain && g_timeline != nullptr && (int64_t)grid * kWaves <= g_timeline_waves;
    if constexpr (ACT == kActPlain && kEagerSteps<TYPE> > 0) {
        if (g.strict == 2)
            return tl ? launch_type_tl<TYPE, kActPlain, true, kEagerSteps<TYPE>>(g, grid, lds, stream)
                      : launch_type_tl<TYPE, kActPlain, false, kEagerSteps<TYPE>>(g, grid, lds, stream);
    }
    if (tl) return launch_type_tl<TYPE, kActPlain, true, 0>(g, grid, lds, stream);
    return launch_type_tl<TYPE, ACT, false, 0>(g, grid, lds, stream);
}

}  // namespace

int gemv_max_k(int type)
{
    switch (type) {
    case kTypeQ8_0: return (int)(kMaxLds / 144 / FmtQ80::kLPR) * FmtQ80::kLPR * 32;
    case kTypeQ4_K: return (int)(kMaxLds / 144 / FmtQ4K::kLPR) * FmtQ4K::kLPR * 64;
    case kTypeMXFP4: return (int)(kMaxLds / 80 / FmtMXFP4::kLPR) * FmtMXFP4::kLPR * 32;
    case kTypeQ6_K: return (int)(kMaxLds / 176 / FmtQ6K::kLPR) * FmtQ6K::kLPR * 64;
    case kTypeQ5_K: return (int)(kMaxLds / 144 / FmtQ4K::kLPR) * FmtQ4K::kLPR * 64;
    case kTypeQ4_0: case kTypeQ4_1: case kTypeQ5_0: case kTypeQ5_1: case kTypeIQ4_NL: return (int)(kMaxLds / 80 / 16) * 16 * 32;
    default: return 0;
    }
}

int gemv_max_group() { return kMaxGroup; }

int gemv_routed_slots(int type) { return type == kTypeMXFP4 || type == kTypeQ8_0 ? 4 : 0; }

int gemv_timeline_slots() { return kTimelineSlots; }
void set_gemv_timeline(uint64_t* device_buffer, int64_t wavefronts)
{
    g_timeline = device_buffer;
    g_timeline_waves = device_buffer ? wavefronts : 0;
}

// one staging pass covers 8 float4 per thread
// the RMSNorm mode stages rows of any length the kernel can hold (its scale is applied at the store)
int gemv_rms_max_k() { return 1 << 30; }

bool launch_gemv_group(int type, int count, const GemvArgs* args, hipStream_t stream)
{
    if (count < 1 || count > kMaxGroup) {
        set_last_error("gemv: group size out of range.");
        return false;
    }
    if (type != kTypeQ8_0 && type != kTypeQ4_K && type != kTypeMXFP4 && type != kTypeQ6_K && type != kTypeQ5_K && !legacy_type(type)) {
        set_last_error("gemv: unsupported type.");
        return false;
    }
    const DeviceInfo& di = device_info();
    size_t lds = 0;
    double total_bytes = 0;
    const int lpr = lanes_per_row(type), rpg = 64 / lpr;
    // bytes a problem streams: its matrix, or for a routed sum one row set per slot
    auto stream_bytes = [&](int i) {
        return args[i].slot_ids ? (double)rpg * args[i].N * (double)(args[i].K / unit_elems(type)) * block_bytes(type) *
                                      (unit_elems(type) / block_elems(type))
                                : (double)args[i].w_bytes;
    };
    // output rows of a problem and how many of them one row group yields
    auto out_rows_of = [&](int i) { return args[i].pair_rows ? args[i].pair_rows : args[i].N; };
    auto out_rpg_of = [&](int i) { return args[i].slot_ids ? 1 : args[i].pair_rows ? rpg / 2 : rpg; };
    for (int i = 0; i < count; ++i) {
        if (args[i].K > gemv_max_k(type)) {
            set_last_error("gemv: K exceeds what one workgroup can stage in LDS.");
            return false;
        }
        if (args[i].w_bytes >= ((int64_t)1 << 31) - 64) {
            set_last_error("gemv: a single weight of 2 GiB or more must be split by rows.");
            return false;
        }
        const bool routed = args[i].slot_ids != nullptr;
        if (routed && (gemv_routed_slots(type) == 0 || !args[i].slot_w || args[i].expert_id || args[i].pair_rows || args[i].add ||
                       args[i].act != kActPlain || args[i].n_experts <= 0 || (args[i].expert_stride & 3) != 0 ||
                       (int64_t)args[i].K * gemv_routed_slots(type) > gemv_max_k(type))) {
            set_last_error("gemv: the routed-sum mode takes a 16-lane format, plain activations, an expert stride of whole dwords and "
                           "all slot vectors in LDS.");
            return false;
        }
        lds = std::max(lds, lds_bytes_for(type, args[i].K, routed));
        total_bytes += stream_bytes(i);
    }
    int per_cu = (int)std::min<size_t>(kWgPerCu, (160 * 1024) / (lds + 256));
    if (per_cu < 1) per_cu = 1;
    // row groups per wavefront of the busiest problem when every CU holds `wgs` workgroups
    auto rounds = [&](int wgs) {
        int worst = 0;
        for (int i = 0; i < count; ++i) {
            const int out_rows = out_rows_of(i), out_rpg = out_rpg_of(i);
            const int groups = (out_rows + std::max(out_rpg, 1) - 1) / std::max(out_rpg, 1);
            const int share = std::max(1, (int)((double)(di.num_cus * wgs) * stream_bytes(i) / total_bytes + 0.5));
            worst = std::max(worst, (groups + share * kWaves - 1) / (share * kWaves));
        }
        return worst;
    };
    // Two workgroups per CU stream best (four: the 123 MB grouped launch 28 instead of 24 us, since twice as many
    // workgroups stage x).  The exception is a launch whose busiest problem has between one and two row groups per
    // wavefront AND long rows: half of the wavefronts then work twice as long as the rest, and four workgroups per CU
    // give every row group a wavefront of its own.  Measured: the four expert matrices of a GPT-OSS token (1440 groups
    // of 6 steps each) 13.8 -> 12.7 us; a 14336 x 4096 Q4_K matrix (7168 groups of 2 steps) loses, 9.7 -> 12.0 us, so
    // the rule asks for at least 8 steps per wavefront.
    int max_steps = 0;
    for (int i = 0; i < count; ++i) max_steps = std::max(max_steps, (args[i].K / unit_elems(type) + lpr - 1) / lpr);
    const int dense_cu = (int)std::min<size_t>(2 * kWgPerCu, (160 * 1024) / (lds + 256));
    if (per_cu == kWgPerCu && dense_cu == 2 * kWgPerCu && rounds(per_cu) == 2 && rounds(dense_cu) == 1 && 2 * max_steps >= 8)
        per_cu = dense_cu;
    const int budget = di.num_cus * per_cu;
    // (More workgroups than the CUs hold at once, so that later ones start while earlier ones stream, was measured slower:
    // the 123 MB grouped launch 28.0 us with 1.5 x and 2 x the workgroups against 24.3 us.)
    // (Cutting the K range of a row group over several wavefronts when a matrix has few rows was measured slower on
    // every shape: 4096 x 14336 Q4_K 13.7 vs 10.9 us, MXFP4 5760 x 2880 7.8 vs 6.7 us.  Requesting more up front - two extra
    // steps before x is staged, or a ring of four steps per wavefront - was slower too, the 123 MB grouped launch
    // included: 24.5 vs 24.2 us.)

    GemvGroup g;
    std::memset(&g, 0, sizeof(g));
    g.count = count;
    g.strict = total_bytes >= kStrictBytes ? 1 : 0;
    int begin = 0;
    for (int i = 0; i < count; ++i) {
        // workgroups in proportion to the bytes each problem streams
        int share = std::max(1, (int)((double)budget * stream_bytes(i) / total_bytes + 0.5));
        const int out_rows = out_rows_of(i), out_rpg = out_rpg_of(i);
        if (args[i].pair_rows && (args[i].N != 2 * args[i].pair_rows || rpg < 2)) {
            set_last_error("gemv: the paired gate | up mode needs N = 2 * pair_rows.");
            return false;
        }
        share = std::min(share, ((out_rows + out_rpg - 1) / out_rpg + kWaves - 1) / kWaves);
        g.p[i].w = static_cast<const uint8_t*>(args[i].w);
        g.p[i].w_bytes = args[i].w_bytes;
        g.p[i].x = args[i].x;
        g.p[i].y = args[i].y;
        g.p[i].add = args[i].add;
        g.p[i].act = args[i].act;
        g.p[i].norm_w = args[i].norm_w;
        g.p[i].eps = args[i].eps;
        g.p[i].limit = args[i].limit;
        if (args[i].act == kActRmsNorm && args[i].K > gemv_rms_max_k()) {
            set_last_error("gemv: the RMSNorm activation mode stages the row in one pass; K is too large.");
            return false;
        }
        g.p[i].N = args[i].N;
        g.p[i].K = args[i].K;
        g.p[i].expert_id = args[i].expert_id;
        g.p[i].expert_stride = args[i].expert_stride;
        g.p[i].n_experts = args[i].n_experts;
        g.p[i].pair_rows = args[i].pair_rows;
        g.p[i].pair_kind = args[i].pair_kind;
        g.p[i].slot_ids = args[i].slot_ids;
        g.p[i].slot_w = args[i].slot_w;
        g.p[i].slot_bias = args[i].slot_bias;
        if (args[i].pair_kind != 0 && (args[i].pair_rows == 0 || args[i].act != kActPlain)) {
            set_last_error("gemv: the GPT-OSS paired store needs pair_rows and plain activation staging.");
            return false;
        }
        if (args[i].expert_id && args[i].n_experts <= 0) {
            set_last_error("gemv: an expert indirection needs the number of experts.");
            return false;
        }
        g.wg_begin[i] = begin;
        begin += share;
    }
    for (int i = count; i <= kMaxGroup; ++i) g.wg_begin[i] = begin;
    const int act = args[0].act;
    // eager build: every problem has at most one row group per wavefront and few enough steps per group
    if (act == kActPlain && eager_steps(type) > 0) {
        // (not for the RMSNorm staging mode: an eager build of it with two steps measured 8.7 against 8.5 us on 6144 x 4096
        // and 0.5 us more per decode layer;
        // not with four workgroups per CU: the eager build's registers leave room for five wavefronts per SIMD, and the
        // gate | up launch of a GPT-OSS token measured 13.4 us with it against 12.0 us; not for routed sums, whose staging
        // of four activation vectors is what they wait for: 8.96 against 8.72 us)
        bool ok = per_cu == kWgPerCu;
        for (int i = 0; i < count; ++i) {
            const int out_rows = out_rows_of(i), out_rpg = out_rpg_of(i);
            const int groups = (out_rows + out_rpg - 1) / out_rpg, waves = (g.wg_begin[i + 1] - g.wg_begin[i]) * kWaves;
            const int steps = (args[i].K / unit_elems(type) + lpr - 1) / lpr;
            // (the eager build stages its activations in one pass of 8 float4 per thread)
            ok = ok && groups <= waves && steps <= eager_steps(type) && args[i].K <= kThreads * 32 && !args[i].slot_ids;
        }
        if (ok) g.strict = 2;
    }
    for (int i = 1; i < count; ++i)
        if (args[i].act != act) {
            set_last_error("gemv: the problems of one launch must share the activation mode.");
            return false;
        }
    if (act < kActPlain || act > kActSiluMul) {
        set_last_error("gemv: unknown activation mode.");
        return false;
    }
#define TSHIP_GEMV_DISPATCH(T)                                                           \
    (act == kActPlain     ? launch_type<T, kActPlain>(g, begin, lds, stream)             \
     : act == kActRmsNorm ? launch_type<T, kActRmsNorm>(g, begin, lds, stream)           \
                          : launch_type<T, kActSiluMul>(g, begin, lds, stream))
    switch (type) {
    case kTypeQ4_K: return TSHIP_GEMV_DISPATCH(kTypeQ4_K);
    case kTypeMXFP4: return TSHIP_GEMV_DISPATCH(kTypeMXFP4);
    case kTypeQ6_K: return TSHIP_GEMV_DISPATCH(kTypeQ6_K);
    case kTypeQ5_K: return TSHIP_GEMV_DISPATCH(kTypeQ5_K);
    case kTypeQ4_0: return TSHIP_GEMV_DISPATCH(kTypeQ4_0);
    case kTypeQ4_1: return TSHIP_GEMV_DISPATCH(kTypeQ4_1);
    case kTypeQ5_0: return TSHIP_GEMV_DISPATCH(kTypeQ5_0);
    case kTypeQ5_1: return TSHIP_GEMV_DISPATCH(kTypeQ5_1);
    case kTypeIQ4_NL: return TSHIP_GEMV_DISPATCH(kTypeIQ4_NL);
    default: return TSHIP_GEMV_DISPATCH(kTypeQ8_0);
    }
#undef TSHIP_GEMV_DISPATCH
}

bool launch_gemv(int type, const void* w, int64_t w_bytes, const float* x, float* y, int N, int K, hipStream_t stream,
                 const float* add, int act, const float* norm_w, float eps)
{
    GemvArgs a{};
    a.w = w, a.w_bytes = w_bytes, a.x = x, a.y = y, a.N = N, a.K = K, a.add = add, a.act = act, a.norm_w = norm_w, a.eps = eps;
    return launch_gemv_group(type, 1, &a, stream);
}

}  // namespace tship
