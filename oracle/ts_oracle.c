/*
 * TEST INFRASTRUCTURE — not part of the shipped library (see ts_oracle.h).
 *
 * CPU restatement of the reference arithmetic for Q8_0 / Q4_K / MXFP4:
 * quantizers, dequantizers, the two CPU matmul semantics and the GPT-OSS
 * MoE expert loop.  Build with -ffp-contract=off: the reference never fuses
 * a multiply with an add on this path, and Q4_K quantized bytes change when
 * the compiler does.
 *
 * Pinning status (what each group is checked against in tests/):
 *   fp16/E8M0 helpers  exhaustive vs numpy float16 / closed form / reference build
 *   dequantizers       reference-held vectors (InferenceWeb.Tests/ManagedQuantizedOpsTests.cs:29-103),
 *                      exhaustive closed forms, reference build (bit-exact)
 *   quantizers         Q8_0/MXFP4 closed form + brute force; Q4_K byte-compare with the
 *                      reference build + committed golden blocks
 *   matmuls            reference-held dot vectors (ManagedQuantizedOpsTests.cs:113-194),
 *                      dense fp64 GEMM on the dequantized matrix, reference-build vec_dot
 *   MoE                brute force on tiny cases; grouped == per-token loop
 */
#include "ts_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define Q8_0_ELEMS 32
#define Q8_0_BYTES 34
#define Q4_K_ELEMS 256
#define Q4_K_BYTES 144
#define MXFP4_ELEMS 32
#define MXFP4_BYTES 17
#define Q8_K_BYTES 292 /* float d; int8 qs[256]; int16 bsums[16]  (ggml-common.h:339-343) */

static inline uint32_t f32_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float bits_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline uint16_t rd16(const uint8_t* p) { return (uint16_t)(p[0] | (p[1] << 8)); }
static inline void wr16(uint8_t* p, uint16_t v) { p[0] = (uint8_t)v; p[1] = (uint8_t)(v >> 8); }

/* ------------------------------------------------------------------ */
/* scalar conversions                                                  */
/* ------------------------------------------------------------------ */

/* IEEE binary16 -> binary32, exact (subnormals included).
 * Reference: ggml-impl.h:378-399 (ggml_compute_fp16_to_fp32),
 * ManagedQuantizedOps.cs:675 (HalfToSingle). */
float tso_fp16_to_fp32(uint16_t h)
{
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    if (exp == 0x1f) return bits_f32(sign | 0x7f800000u | (man << 13));
    if (exp != 0) return bits_f32(sign | ((exp + 112u) << 23) | (man << 13));
    if (man == 0) return bits_f32(sign);
    /* subnormal: value = man * 2^-24; normalise */
    int shift = 0;
    while (!(man & 0x400u)) { man <<= 1; ++shift; }
    man &= 0x3ffu;
    return bits_f32(sign | ((uint32_t)(113 - shift) << 23) | (man << 13));
}

/* binary32 -> binary16, round to nearest even; NaN -> sign|0x7E00.
 * Reference: ggml-impl.h:401-425 (ggml_compute_fp32_to_fp16). */
uint16_t tso_fp32_to_fp16(float f)
{
    uint32_t u = f32_bits(f);
    uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    uint32_t a = u & 0x7fffffffu;
    if (a > 0x7f800000u) return (uint16_t)(sign | 0x7e00u);
    if (a >= 0x47800000u) return (uint16_t)(sign | 0x7c00u);     /* >= 65536 or inf */
    if (a >= 0x38800000u) {                                       /* normal half range */
        uint32_t m = a - 0x38000000u;
        uint32_t r = m + 0xfffu + ((m >> 13) & 1u);
        return (uint16_t)(sign | (r >> 13));                      /* carries into inf at 65520 */
    }
    uint32_t e = a >> 23;
    if (e < 102) return sign;                                     /* < 2^-25 -> 0 */
    uint32_t mant = (a & 0x7fffffu) | 0x800000u;
    uint32_t shift = 126u - e;                                    /* 14..24 */
    uint32_t hbits = mant >> shift;
    uint32_t rem = mant & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (hbits & 1u))) ++hbits;
    return (uint16_t)(sign | hbits);
}

/* E8M0 exponent byte -> 2^(e-128) as fp32 (the "half" scale MXFP4 uses because
 * its value table is doubled).  e < 2 gives the subnormal patterns 0x00200000<<e.
 * Reference: ggml-impl.h:471-489, ManagedQuantizedOps.cs:678-682. */
float tso_e8m0_to_fp32_half(uint8_t e)
{
    return bits_f32(e < 2 ? (0x00200000u << e) : ((uint32_t)(e - 1) << 23));
}

/* E2M1 values doubled. Reference: ggml-common.h:1094-1096, ManagedQuantizedOps.cs:35-38. */
static const int8_t k_mxfp4_values[16] = { 0, 1, 2, 3, 4, 6, 8, 12, 0, -1, -2, -3, -4, -6, -8, -12 };

/* ------------------------------------------------------------------ */
/* type tables — TensorSharp.Runtime/GgufReader.cs:303-369,            */
/* ManagedQuantizedOps.cs:77-88 (RowSize), ggml_ops_core.cpp:1320-1329 */
/* ------------------------------------------------------------------ */
int64_t tso_block_size(int type)
{
    switch (type) {
    case TSO_TYPE_F32: return 1;
    case TSO_TYPE_Q8_0: return Q8_0_ELEMS;
    case TSO_TYPE_Q4_K: return Q4_K_ELEMS;
    case TSO_TYPE_MXFP4: return MXFP4_ELEMS;
    case TSO_TYPE_F16: case TSO_TYPE_BF16: return 1;
    case TSO_TYPE_Q4_0: case TSO_TYPE_Q4_1: case TSO_TYPE_Q5_0: case TSO_TYPE_Q5_1: case TSO_TYPE_IQ4_NL: case TSO_TYPE_Q8_1: return 32;
    case TSO_TYPE_Q5_K: case TSO_TYPE_Q6_K: return 256;
    default: return 0;
    }
}

int64_t tso_type_size(int type)
{
    switch (type) {
    case TSO_TYPE_F32: return 4;
    case TSO_TYPE_Q8_0: return Q8_0_BYTES;
    case TSO_TYPE_Q4_K: return Q4_K_BYTES;
    case TSO_TYPE_MXFP4: return MXFP4_BYTES;
    case TSO_TYPE_F16: case TSO_TYPE_BF16: return 2;
    case TSO_TYPE_Q4_0: return 18;
    case TSO_TYPE_Q4_1: return 20;
    case TSO_TYPE_Q5_0: return 22;
    case TSO_TYPE_Q5_1: return 24;
    case TSO_TYPE_Q8_1: return 36;
    case TSO_TYPE_IQ4_NL: return 18;
    case TSO_TYPE_Q5_K: return 176;
    case TSO_TYPE_Q6_K: return 210;
    default: return 0;
    }
}

int64_t tso_row_size(int type, int64_t ne)
{
    int64_t bs = tso_block_size(type);
    if (bs == 0 || ne <= 0 || ne % bs != 0) return 0;
    return ne / bs * tso_type_size(type);
}

/* ------------------------------------------------------------------ */
/* quantizers                                                          */
/* ------------------------------------------------------------------ */

/* Q8_0: d = amax/127 (fp32), q = roundf(x * (1/d)), d stored as fp16 afterwards.
 * Reference: ggml-quants.c:199-222. */
void tso_quantize_q8_0(const float* xin, void* dst, int64_t n)
{
#pragma omp parallel for schedule(static)
    for (int64_t b = 0; b < n / Q8_0_ELEMS; ++b) {
        const float* x = xin + b * Q8_0_ELEMS;
        uint8_t* out = (uint8_t*)dst + b * Q8_0_BYTES;
        float amax = 0.0f;
        for (int j = 0; j < Q8_0_ELEMS; ++j) {
            float a = fabsf(x[j]);
            if (a > amax) amax = a;
        }
        const float d = amax / 127.0f;
        const float inv = d != 0.0f ? 1.0f / d : 0.0f;
        wr16(out, tso_fp32_to_fp16(d));
        for (int j = 0; j < Q8_0_ELEMS; ++j) {
            float scaled = x[j] * inv;
            out[2 + j] = (uint8_t)(int8_t)roundf(scaled);
        }
    }
}

/* round to nearest, ties to even, |v| <= 4194303.
 * Reference: ggml-quants.c:444-449 (nearest_int, magic-number form). */
static inline int rne_int(float v) { return (int)lrintf(v); }

/* Weighted least-squares search for (scale, min) of one 32-value sub-block
 * quantised to 0..nmax.  Restates make_qkx2_quants with rmin=-1, rdelta=0.1,
 * nstep=20, use_mad=false; every float operation is kept in reference order
 * because the resulting bytes depend on it.
 * Reference: ggml-quants.c:622-701. */
static float search_scale_min(int n, int nmax, const float* x, const float* w,
                              uint8_t* L, float* neg_min_out, uint8_t* Ltmp)
{
    const float rmin = -1.0f, rdelta = 0.1f;
    const int nstep = 20;
    float lo = x[0], hi = x[0];
    float sum_w = w[0];
    float sum_x = sum_w * x[0];
    for (int i = 1; i < n; ++i) {
        if (x[i] < lo) lo = x[i];
        if (x[i] > hi) hi = x[i];
        float wi = w[i];
        sum_w += wi;
        sum_x += wi * x[i];
    }
    if (lo > 0) lo = 0;
    if (hi == lo) {
        for (int i = 0; i < n; ++i) L[i] = 0;
        *neg_min_out = -lo;
        return 0.0f;
    }
    float iscale = nmax / (hi - lo);
    float scale = 1 / iscale;
    float best = 0;
    for (int i = 0; i < n; ++i) {
        int l = rne_int(iscale * (x[i] - lo));
        if (l < 0) l = 0;
        if (l > nmax) l = nmax;
        L[i] = (uint8_t)l;
        float diff = scale * L[i] + lo - x[i];
        diff = diff * diff;
        best += w[i] * diff;
    }
    for (int is = 0; is <= nstep; ++is) {
        iscale = (rmin + rdelta * is + nmax) / (hi - lo);
        float sum_l = 0, sum_l2 = 0, sum_xl = 0;
        for (int i = 0; i < n; ++i) {
            int l = rne_int(iscale * (x[i] - lo));
            if (l < 0) l = 0;
            if (l > nmax) l = nmax;
            Ltmp[i] = (uint8_t)l;
            float wi = w[i];
            sum_l += wi * l;
            sum_l2 += wi * l * l;
            sum_xl += wi * l * x[i];
        }
        float D = sum_w * sum_l2 - sum_l * sum_l;
        if (D > 0) {
            float s = (sum_w * sum_xl - sum_x * sum_l) / D;
            float m = (sum_l2 * sum_x - sum_l * sum_xl) / D;
            if (m > 0) {
                m = 0;
                s = sum_xl / sum_l2;
            }
            float err = 0;
            for (int i = 0; i < n; ++i) {
                float diff = s * Ltmp[i] + m - x[i];
                diff = diff * diff;
                err += w[i] * diff;
            }
            if (err < best) {
                memcpy(L, Ltmp, (size_t)n);
                best = err;
                scale = s;
                lo = m;
            }
        }
    }
    *neg_min_out = -lo;
    return scale;
}

/* 6-bit scale / min of sub-block j from the 12 packed bytes.
 * Reference: ggml-quants.c:703-710, ManagedQuantizedOps.cs:685-696. */
static inline void unpack_scale_min(int j, const uint8_t* p, uint8_t* sc, uint8_t* mn)
{
    if (j < 4) {
        *sc = p[j] & 63;
        *mn = p[j + 4] & 63;
    } else {
        *sc = (uint8_t)((p[j + 4] & 0x0f) | ((p[j - 4] >> 6) << 4));
        *mn = (uint8_t)((p[j + 4] >> 4) | ((p[j] >> 6) << 4));
    }
}

/* Q4_K. Reference: ggml-quants.c:1280-1350. */
void tso_quantize_q4_K(const float* xin, void* dst, int64_t n)
{
#pragma omp parallel for schedule(static)
    for (int64_t b = 0; b < n / Q4_K_ELEMS; ++b) {
        const float* x = xin + b * Q4_K_ELEMS;
        uint8_t* out = (uint8_t*)dst + b * Q4_K_BYTES;
        uint8_t L[Q4_K_ELEMS], Ltmp[32];
        float wts[32], mins[8], scales[8];
        uint8_t* packed = out + 4;
        uint8_t* qs = out + 16;
        memset(packed, 0, 12);
        float max_scale = 0, max_min = 0;
        for (int j = 0; j < 8; ++j) {
            const float* xs = x + 32 * j;
            float sum_x2 = 0;
            for (int l = 0; l < 32; ++l) sum_x2 += xs[l] * xs[l];
            float av_x = sqrtf(sum_x2 / 32);
            for (int l = 0; l < 32; ++l) wts[l] = av_x + fabsf(xs[l]);
            scales[j] = search_scale_min(32, 15, xs, wts, L + 32 * j, &mins[j], Ltmp);
            if (scales[j] > max_scale) max_scale = scales[j];
            if (mins[j] > max_min) max_min = mins[j];
        }
        float inv_scale = max_scale > 0 ? 63.f / max_scale : 0.f;
        float inv_min = max_min > 0 ? 63.f / max_min : 0.f;
        for (int j = 0; j < 8; ++j) {
            uint8_t ls = (uint8_t)rne_int(inv_scale * scales[j]);
            uint8_t lm = (uint8_t)rne_int(inv_min * mins[j]);
            if (ls > 63) ls = 63;
            if (lm > 63) lm = 63;
            if (j < 4) {
                packed[j] = ls;
                packed[j + 4] = lm;
            } else {
                packed[j + 4] = (uint8_t)((ls & 0x0f) | ((lm & 0x0f) << 4));
                packed[j - 4] |= (uint8_t)((ls >> 4) << 6);
                packed[j] |= (uint8_t)((lm >> 4) << 6);
            }
        }
        uint16_t hd = tso_fp32_to_fp16(max_scale / 63.f);
        uint16_t hm = tso_fp32_to_fp16(max_min / 63.f);
        wr16(out, hd);
        wr16(out + 2, hm);
        const float fd = tso_fp16_to_fp32(hd), fm = tso_fp16_to_fp32(hm);
        /* re-quantise with the stored (rounded) scales */
        for (int j = 0; j < 8; ++j) {
            uint8_t sc, mn;
            unpack_scale_min(j, packed, &sc, &mn);
            const float d = fd * sc;
            if (!d) continue;
            const float dm = fm * mn;
            for (int i = 0; i < 32; ++i) {
                int l = rne_int((x[32 * j + i] + dm) / d);
                if (l < 0) l = 0;
                if (l > 15) l = 15;
                L[32 * j + i] = (uint8_t)l;
            }
        }
        for (int g = 0; g < 4; ++g)
            for (int l = 0; l < 32; ++l)
                qs[32 * g + l] = (uint8_t)(L[64 * g + l] | (L[64 * g + 32 + l] << 4));
    }
}

/* MXFP4: shared exponent e = floor(log2(amax)) - 2 + 127, each value mapped to the
 * nearest doubled-E2M1 table entry times 2^(e-128); first minimum wins.
 * Reference: ggml-quants.c:260-305. */
void tso_quantize_mxfp4(const float* xin, void* dst, int64_t n)
{
#pragma omp parallel for schedule(static)
    for (int64_t b = 0; b < n / MXFP4_ELEMS; ++b) {
        const float* x = xin + b * MXFP4_ELEMS;
        uint8_t* out = (uint8_t*)dst + b * MXFP4_BYTES;
        float amax = 0.0f;
        for (int j = 0; j < MXFP4_ELEMS; ++j) {
            float a = fabsf(x[j]);
            if (amax < a) amax = a;
        }
        const uint8_t e = amax > 0.0f ? (uint8_t)(floorf(log2f(amax)) - 2 + 127) : 0;
        const float d = tso_e8m0_to_fp32_half(e);
        out[0] = e;
        for (int j = 0; j < 16; ++j) {
            uint8_t nib[2];
            for (int h = 0; h < 2; ++h) {
                const float v = x[j + 16 * h];
                int best = 0;
                float best_err = fabsf(k_mxfp4_values[0] * d - v);
                for (int i = 1; i < 16; ++i) {
                    float err = fabsf(k_mxfp4_values[i] * d - v);
                    if (err < best_err) { best = i; best_err = err; }
                }
                nib[h] = (uint8_t)best;
            }
            out[1 + j] = (uint8_t)(nib[0] | (nib[1] << 4));
        }
    }
}

int tso_quantize(int type, const float* x, void* dst, int64_t n)
{
    int64_t bs = tso_block_size(type);
    if (!x || !dst || bs == 0 || n < 0 || n % bs != 0) return -1;
    switch (type) {
    case TSO_TYPE_Q8_0: tso_quantize_q8_0(x, dst, n); return 0;
    case TSO_TYPE_Q4_K: tso_quantize_q4_K(x, dst, n); return 0;
    case TSO_TYPE_MXFP4: tso_quantize_mxfp4(x, dst, n); return 0;
    case TSO_TYPE_F32: memcpy(dst, x, (size_t)n * 4); return 0;
    default: return -2;
    }
}

/* Q8_K activation blocks: iscale = -127/max (max = signed value of largest magnitude),
 * q = min(127, rne(iscale*x)), d = 1/iscale, bsums over groups of 16.
 * Reference: ggml-quants.c:2555-2592. */
void tso_quantize_q8_K(const float* x, void* dst, int64_t n)
{
    uint8_t* out = (uint8_t*)dst;
    for (int64_t b = 0; b < n / 256; ++b, x += 256, out += Q8_K_BYTES) {
        int8_t* qs = (int8_t*)(out + 4);
        float max = 0, amax = 0;
        for (int j = 0; j < 256; ++j) {
            float ax = fabsf(x[j]);
            if (ax > amax) { amax = ax; max = x[j]; }
        }
        if (!amax) {
            memset(out, 0, Q8_K_BYTES);
            continue;
        }
        const float iscale = -127.f / max;
        for (int j = 0; j < 256; ++j) {
            int v = rne_int(iscale * x[j]);
            qs[j] = (int8_t)(v > 127 ? 127 : v);
        }
        for (int g = 0; g < 16; ++g) {
            int s = 0;
            for (int i = 0; i < 16; ++i) s += qs[16 * g + i];
            int16_t s16 = (int16_t)s;
            memcpy(out + 4 + 256 + 2 * g, &s16, 2);
        }
        float d = 1 / iscale;
        memcpy(out, &d, 4);
    }
}

/* ------------------------------------------------------------------ */
/* dequantizers                                                        */
/* ------------------------------------------------------------------ */

/* Reference: ManagedQuantizedOps.cs:411-427. */
static void dequant_q8_0(const uint8_t* src, int64_t n, float* y)
{
    for (int64_t b = 0; b < n / Q8_0_ELEMS; ++b, src += Q8_0_BYTES, y += Q8_0_ELEMS) {
        const float d = tso_fp16_to_fp32(rd16(src));
        const int8_t* q = (const int8_t*)(src + 2);
        for (int j = 0; j < Q8_0_ELEMS; ++j) y[j] = q[j] * d;
    }
}

/* Q8_1 block: fp16 d, fp16 s (= d * sum of the quants, not read here), int8 qs[32]; y = q * d.
 * Reference: ManagedQuantizedOps.cs:429-445, GgufReader.cs:342 (36 bytes). */
static void dequant_q8_1(const uint8_t* src, int64_t n, float* y)
{
    for (int64_t b = 0; b < n / 32; ++b, src += 36, y += 32) {
        const float d = tso_fp16_to_fp32(rd16(src));
        const int8_t* q = (const int8_t*)(src + 4);
        for (int j = 0; j < 32; ++j) y[j] = q[j] * d;
    }
}

/* y = (d*sc)*q - (dmin*m); low nibbles are the first 32 of each 64-group.
 * Reference: ManagedQuantizedOps.cs:447-479, ggml-quants.c:1352-1374. */
static void dequant_q4_K(const uint8_t* src, int64_t n, float* y)
{
    for (int64_t b = 0; b < n / Q4_K_ELEMS; ++b, src += Q4_K_BYTES, y += Q4_K_ELEMS) {
        const float d = tso_fp16_to_fp32(rd16(src));
        const float dmin = tso_fp16_to_fp32(rd16(src + 2));
        const uint8_t* packed = src + 4;
        const uint8_t* q = src + 16;
        for (int g = 0; g < 4; ++g, q += 32) {
            uint8_t sc1, m1, sc2, m2;
            unpack_scale_min(2 * g, packed, &sc1, &m1);
            unpack_scale_min(2 * g + 1, packed, &sc2, &m2);
            const float d1 = d * sc1, d2 = d * sc2;
            const float o1 = dmin * m1, o2 = dmin * m2;
            for (int l = 0; l < 32; ++l) y[64 * g + l] = d1 * (q[l] & 0x0f) - o1;
            for (int l = 0; l < 32; ++l) y[64 * g + 32 + l] = d2 * (q[l] >> 4) - o2;
        }
    }
}

/* low nibble -> element j, high nibble -> element j+16.
 * Reference: ManagedQuantizedOps.cs:579-598. */
static void dequant_mxfp4(const uint8_t* src, int64_t n, float* y)
{
    for (int64_t b = 0; b < n / MXFP4_ELEMS; ++b, src += MXFP4_BYTES, y += MXFP4_ELEMS) {
        const float d = tso_e8m0_to_fp32_half(src[0]);
        for (int j = 0; j < 16; ++j) {
            y[j] = d * k_mxfp4_values[src[1 + j] & 0x0f];
            y[j + 16] = d * k_mxfp4_values[src[1 + j] >> 4];
        }
    }
}


/* ---- the other formats the managed code reads (dequantize / embedding gather only, plus Q6_K matmuls) ---- */

/* Reference: ManagedQuantizedOps.cs:268-281 (F16: exact widening; BF16: bits << 16). */
static void dequant_f16(const uint8_t* src, int64_t n, float* y)
{
    for (int64_t i = 0; i < n; ++i) y[i] = tso_fp16_to_fp32(rd16(src + 2 * i));
}
static void dequant_bf16(const uint8_t* src, int64_t n, float* y)
{
    for (int64_t i = 0; i < n; ++i) y[i] = bits_f32((uint32_t)rd16(src + 2 * i) << 16);
}

/* y[j] = (q - 8) * d, low nibble -> j, high nibble -> j + 16.
 * Reference: ManagedQuantizedOps.cs:313-333, ggml-quants.c dequantize_row_q4_0. */
static void dequant_q4_0(const uint8_t* src, int64_t n, float* y)
{
    for (int64_t b = 0; b < n / 32; ++b, src += 18, y += 32) {
        const float d = tso_fp16_to_fp32(rd16(src));
        for (int j = 0; j < 16; ++j) {
            y[j] = ((src[2 + j] & 0x0f) - 8) * d;
            y[j + 16] = ((src[2 + j] >> 4) - 8) * d;
        }
    }
}

/* y[j] = q * d + m (a product and a separately rounded sum).
 * Reference: ManagedQuantizedOps.cs:335-356, ggml-quants.c dequantize_row_q4_1. */
static void dequant_q4_1(const uint8_t* src, int64_t n, float* y)
{
    for (int64_t b = 0; b < n / 32; ++b, src += 20, y += 32) {
        const float d = tso_fp16_to_fp32(rd16(src)), m = tso_fp16_to_fp32(rd16(src + 2));
        for (int j = 0; j < 16; ++j) {
            y[j] = (src[4 + j] & 0x0f) * d + m;
            y[j + 16] = (src[4 + j] >> 4) * d + m;
        }
    }
}

/* fifth bit of element j from bit j of qh (elements 16.. from bits 16..).
 * Reference: ManagedQuantizedOps.cs:358-382, ggml-quants.c dequantize_row_q5_0. */
static void dequant_q5_0(const uint8_t* src, int64_t n, float* y)
{
    for (int64_t b = 0; b < n / 32; ++b, src += 22, y += 32) {
        const float d = tso_fp16_to_fp32(rd16(src));
        const uint32_t qh = (uint32_t)src[2] | ((uint32_t)src[3] << 8) | ((uint32_t)src[4] << 16) | ((uint32_t)src[5] << 24);
        for (int j = 0; j < 16; ++j) {
            const int xh0 = (int)(((qh >> j) << 4) & 0x10), xh1 = (int)((qh >> (j + 12)) & 0x10);
            y[j] = (((src[6 + j] & 0x0f) | xh0) - 16) * d;
            y[j + 16] = (((src[6 + j] >> 4) | xh1) - 16) * d;
        }
    }
}

/* Reference: ManagedQuantizedOps.cs:384-409, ggml-quants.c dequantize_row_q5_1. */
static void dequant_q5_1(const uint8_t* src, int64_t n, float* y)
{
    for (int64_t b = 0; b < n / 32; ++b, src += 24, y += 32) {
        const float d = tso_fp16_to_fp32(rd16(src)), m = tso_fp16_to_fp32(rd16(src + 2));
        const uint32_t qh = (uint32_t)src[4] | ((uint32_t)src[5] << 8) | ((uint32_t)src[6] << 16) | ((uint32_t)src[7] << 24);
        for (int j = 0; j < 16; ++j) {
            const int xh0 = (int)(((qh >> j) << 4) & 0x10), xh1 = (int)((qh >> (j + 12)) & 0x10);
            y[j] = ((src[8 + j] & 0x0f) | xh0) * d + m;
            y[j + 16] = ((src[8 + j] >> 4) | xh1) * d + m;
        }
    }
}

/* Q4_K with a fifth bit per weight: block = d, dmin, scales[12], qh[32], ql[128];
 * y = (d*sc) * (nibble + 16*bit) - (dmin*m).
 * Reference: ManagedQuantizedOps.cs:481-518, ggml-quants.c dequantize_row_q5_K. */
static void dequant_q5_K(const uint8_t* src, int64_t n, float* y)
{
    for (int64_t b = 0; b < n / 256; ++b, src += 176, y += 256) {
        const float d = tso_fp16_to_fp32(rd16(src)), dmin = tso_fp16_to_fp32(rd16(src + 2));
        const uint8_t* packed = src + 4;
        const uint8_t* qh = src + 16;
        const uint8_t* ql = src + 48;
        uint8_t u1 = 1, u2 = 2;
        for (int g = 0; g < 4; ++g, ql += 32, u1 <<= 2, u2 <<= 2) {
            uint8_t sc1, m1, sc2, m2;
            unpack_scale_min(2 * g, packed, &sc1, &m1);
            unpack_scale_min(2 * g + 1, packed, &sc2, &m2);
            const float d1 = d * sc1, d2 = d * sc2;
            const float o1 = dmin * m1, o2 = dmin * m2;
            for (int l = 0; l < 32; ++l) y[64 * g + l] = d1 * ((ql[l] & 0x0f) + ((qh[l] & u1) ? 16 : 0)) - o1;
            for (int l = 0; l < 32; ++l) y[64 * g + 32 + l] = d2 * ((ql[l] >> 4) + ((qh[l] & u2) ? 16 : 0)) - o2;
        }
    }
}

/* block = ql[128], qh[64], int8 scales[16], fp16 d; per 128 weights: 4 groups of 32 taken from the low / high
 * nibbles of ql[l], ql[l + 32] and two bits of qh[l]; y = d * scale * (q - 32), exact in fp32.
 * Reference: ManagedQuantizedOps.cs:520-557, ggml-quants.c:1762-1791. */
static void dequant_q6_K(const uint8_t* src, int64_t n, float* y)
{
    for (int64_t b = 0; b < n / 256; ++b, src += 210, y += 256) {
        const uint8_t* ql = src;
        const uint8_t* qh = src + 128;
        const int8_t* sc = (const int8_t*)(src + 192);
        const float d = tso_fp16_to_fp32(rd16(src + 208));
        for (int half = 0; half < 2; ++half, ql += 64, qh += 32, sc += 8) {
            float* o = y + 128 * half;
            for (int l = 0; l < 32; ++l) {
                const int is = l / 16;
                const int8_t q1 = (int8_t)(((ql[l] & 0x0f) | (((qh[l] >> 0) & 3) << 4)) - 32);
                const int8_t q2 = (int8_t)(((ql[l + 32] & 0x0f) | (((qh[l] >> 2) & 3) << 4)) - 32);
                const int8_t q3 = (int8_t)(((ql[l] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32);
                const int8_t q4 = (int8_t)(((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32);
                o[l] = d * sc[is] * q1;
                o[l + 32] = d * sc[is + 2] * q2;
                o[l + 64] = d * sc[is + 4] * q3;
                o[l + 96] = d * sc[is + 6] * q4;
            }
        }
    }
}

/* y = d * table[nibble].  Reference: ManagedQuantizedOps.cs:30-33, :559-577. */
static const int8_t k_iq4nl_values[16] = { -127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113 };
static void dequant_iq4_nl(const uint8_t* src, int64_t n, float* y)
{
    for (int64_t b = 0; b < n / 32; ++b, src += 18, y += 32) {
        const float d = tso_fp16_to_fp32(rd16(src));
        for (int j = 0; j < 16; ++j) {
            y[j] = d * k_iq4nl_values[src[2 + j] & 0x0f];
            y[j + 16] = d * k_iq4nl_values[src[2 + j] >> 4];
        }
    }
}

/* Return codes follow TSGgml_DequantizeToF32: 0 ok, -1 bad args, -2 unsupported type.
 * Reference: ggml_ops_core.cpp:1331-1354. */
int tso_dequantize(int type, const void* src, int64_t n, float* dst)
{
    if (!src || !dst || n < 0) return -1;
    int64_t bs = tso_block_size(type);
    if (bs == 0) return -2;
    if (n % bs != 0) return -1;
    switch (type) {
    case TSO_TYPE_F32: memcpy(dst, src, (size_t)n * 4); return 0;
    case TSO_TYPE_Q8_0: dequant_q8_0((const uint8_t*)src, n, dst); return 0;
    case TSO_TYPE_Q8_1: dequant_q8_1((const uint8_t*)src, n, dst); return 0;
    case TSO_TYPE_Q4_K: dequant_q4_K((const uint8_t*)src, n, dst); return 0;
    case TSO_TYPE_MXFP4: dequant_mxfp4((const uint8_t*)src, n, dst); return 0;
    case TSO_TYPE_F16: dequant_f16((const uint8_t*)src, n, dst); return 0;
    case TSO_TYPE_BF16: dequant_bf16((const uint8_t*)src, n, dst); return 0;
    case TSO_TYPE_Q4_0: dequant_q4_0((const uint8_t*)src, n, dst); return 0;
    case TSO_TYPE_Q4_1: dequant_q4_1((const uint8_t*)src, n, dst); return 0;
    case TSO_TYPE_Q5_0: dequant_q5_0((const uint8_t*)src, n, dst); return 0;
    case TSO_TYPE_Q5_1: dequant_q5_1((const uint8_t*)src, n, dst); return 0;
    case TSO_TYPE_Q5_K: dequant_q5_K((const uint8_t*)src, n, dst); return 0;
    case TSO_TYPE_Q6_K: dequant_q6_K((const uint8_t*)src, n, dst); return 0;
    case TSO_TYPE_IQ4_NL: dequant_iq4_nl((const uint8_t*)src, n, dst); return 0;
    default: return -2;
    }
}

/* ------------------------------------------------------------------ */
/* matmuls                                                             */
/* ------------------------------------------------------------------ */

static int check_mm(int type, const void* w, int64_t N, int64_t K, const float* x, int64_t M,
                    int64_t x_stride, const void* out)
{
    if (!w || !x || !out || N <= 0 || M <= 0 || K <= 0 || x_stride < K) return -1;
    if (tso_block_size(type) == 0 || type == TSO_TYPE_F32) return -2;
    if (K % tso_block_size(type) != 0) return -1;
    return 0;
}

int tso_max_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* Ground truth both CPU semantics approximate: bit-exact dequantised weights times
 * fp32 activations, accumulated in fp64. */
int tso_matmul_f64(int type, const void* w, int64_t N, int64_t K, const float* x, int64_t M,
                   int64_t x_stride, double* out)
{
    int rc = check_mm(type, w, N, K, x, M, x_stride, out);
    if (rc) return rc;
    const int64_t row_bytes = tso_row_size(type, K);
#pragma omp parallel
    {
        float* row = (float*)malloc((size_t)K * sizeof(float));
#pragma omp for schedule(static)
        for (int64_t n = 0; n < N; ++n) {
            tso_dequantize(type, (const uint8_t*)w + n * row_bytes, K, row);
            for (int64_t m = 0; m < M; ++m) {
                const float* xr = x + m * x_stride;
                double acc = 0.0;
                for (int64_t k = 0; k < K; ++k) acc += (double)row[k] * (double)xr[k];
                out[m * N + n] = acc;
            }
        }
        free(row);
    }
    return 0;
}

/* fp32 dot in the order of the managed SIMD loop: two vectors of vec_width lanes,
 * summed lane-wise, then a horizontal sum, then a scalar tail.
 * Reference: ManagedQuantizedOps.cs:631-657 (DotFloat). */
static float dot_managed(const float* a, const float* b, int len, int vw)
{
    float acc0[16] = { 0 }, acc1[16] = { 0 };
    int i = 0;
    for (; i <= len - 2 * vw; i += 2 * vw)
        for (int l = 0; l < vw; ++l) {
            acc0[l] += a[i + l] * b[i + l];
            acc1[l] += a[i + vw + l] * b[i + vw + l];
        }
    for (int l = 0; l < vw; ++l) acc0[l] += acc1[l];
    for (; i <= len - vw; i += vw)
        for (int l = 0; l < vw; ++l) acc0[l] += a[i + l] * b[i + l];
    float sum = 0.0f;
    for (int l = 0; l < vw; ++l) sum += acc0[l];
    for (; i < len; ++i) sum += a[i] * b[i];
    return sum;
}

/* Managed (pure C#) semantics: per output column, dequantise one block at a time into
 * scratch, fp32-dot it against every activation row, add chunk results sequentially.
 * Reference: ModelBase.cs:924-991 (AddmmQuantManaged),
 * ManagedQuantizedOps.cs:156-200 (DotRowBatchToFloat32). */
int tso_matmul_managed(int type, const void* w, int64_t N, int64_t K, const float* x, int64_t M,
                       int64_t x_stride, float* out, int vec_width, int n_threads)
{
    int rc = check_mm(type, w, N, K, x, M, x_stride, out);
    if (rc) return rc;
    if (vec_width < 1 || vec_width > 16) return -1;
    const int64_t row_bytes = tso_row_size(type, K);
    const int bs = (int)tso_block_size(type);
    const int bb = (int)tso_type_size(type);
    if (n_threads < 1) n_threads = 1;
#pragma omp parallel num_threads(n_threads)
    {
        float scratch[256];
        float* sums = (float*)malloc((size_t)M * sizeof(float));
#pragma omp for schedule(static)
        for (int64_t n = 0; n < N; ++n) {
            const uint8_t* chunk = (const uint8_t*)w + n * row_bytes;
            for (int64_t m = 0; m < M; ++m) sums[m] = 0.0f;
            for (int64_t k0 = 0; k0 < K; k0 += bs, chunk += bb) {
                tso_dequantize(type, chunk, bs, scratch);
                for (int64_t m = 0; m < M; ++m)
                    sums[m] += dot_managed(x + m * x_stride + k0, scratch, bs, vec_width);
            }
            for (int64_t m = 0; m < M; ++m) out[m * N + n] = sums[m];
        }
        free(sums);
    }
    return 0;
}

/* Reference: ggml-cpu/quants.c:305-333 (q8_0 x q8_0). */
static float vdot_q8_0(int64_t K, const uint8_t* w, const uint8_t* a)
{
    float sumf = 0;
    for (int64_t b = 0; b < K / 32; ++b, w += Q8_0_BYTES, a += Q8_0_BYTES) {
        const int8_t* qw = (const int8_t*)(w + 2);
        const int8_t* qa = (const int8_t*)(a + 2);
        int sumi = 0;
        for (int j = 0; j < 32; ++j) sumi += qw[j] * qa[j];
        sumf += sumi * (tso_fp16_to_fp32(rd16(w)) * tso_fp16_to_fp32(rd16(a)));
    }
    return sumf;
}

/* Reference: ggml-cpu/quants.c:188-217 (mxfp4 x q8_0). */
static float vdot_mxfp4(int64_t K, const uint8_t* w, const uint8_t* a)
{
    float sumf = 0;
    for (int64_t b = 0; b < K / 32; ++b, w += MXFP4_BYTES, a += Q8_0_BYTES) {
        const int8_t* qa = (const int8_t*)(a + 2);
        const float d = tso_fp16_to_fp32(rd16(a)) * tso_e8m0_to_fp32_half(w[0]);
        int s1 = 0, s2 = 0;
        for (int j = 0; j < 16; ++j) {
            s1 += qa[j] * k_mxfp4_values[w[1 + j] & 0x0f];
            s2 += qa[j + 16] * k_mxfp4_values[w[1 + j] >> 4];
        }
        sumf += d * (s1 + s2);
    }
    return sumf;
}

/* Reference: ggml-cpu/quants.c:550-623 (q4_K x q8_K): eight interleaved fp32 partial
 * sums of d*(scale * sum q4*q8), minus dmin * sum(bsums * mins). */
static float vdot_q4_K(int64_t K, const uint8_t* w, const uint8_t* a)
{
    float lanes[8] = { 0 };
    float sumf = 0;
    int8_t nib[256];
    for (int64_t b = 0; b < K / 256; ++b, w += Q4_K_BYTES, a += Q8_K_BYTES) {
        float ad;
        memcpy(&ad, a, 4);
        const int8_t* q8 = (const int8_t*)(a + 4);
        int16_t bsums[16];
        memcpy(bsums, a + 4 + 256, 32);
        const uint8_t* q4 = w + 16;
        for (int g = 0; g < 4; ++g)
            for (int l = 0; l < 32; ++l) {
                nib[64 * g + l] = (int8_t)(q4[32 * g + l] & 0x0f);
                nib[64 * g + 32 + l] = (int8_t)(q4[32 * g + l] >> 4);
            }
        uint8_t sc[8], mn[8];
        for (int j = 0; j < 8; ++j) unpack_scale_min(j, w + 4, &sc[j], &mn[j]);
        int summ = 0;
        for (int j = 0; j < 16; ++j) summ += bsums[j] * mn[j / 2];
        int32_t part[8] = { 0 };
        for (int j = 0; j < 8; ++j)
            for (int c = 0; c < 4; ++c)
                for (int l = 0; l < 8; ++l) {
                    int idx = 32 * j + 8 * c + l;
                    part[l] += (int32_t)sc[j] * (int16_t)(q8[idx] * nib[idx]);
                }
        const float d = tso_fp16_to_fp32(rd16(w)) * ad;
        for (int l = 0; l < 8; ++l) lanes[l] += d * part[l];
        const float dmin = tso_fp16_to_fp32(rd16(w + 2)) * ad;
        sumf -= dmin * summ;
    }
    for (int l = 0; l < 8; ++l) sumf += lanes[l];
    return sumf;
}

/* GGML CPU semantics: activations are quantised row-wise to the weight type's
 * vec_dot_type (Q8_0 for Q8_0/MXFP4 weights, Q8_K for Q4_K), then integer dots.
 * Reference: ggml-cpu/ggml-cpu.c:251-292 (traits), :1290-1327 (from_float), :1138-1226. */
int tso_matmul_ggml(int type, const void* w, int64_t N, int64_t K, const float* x, int64_t M,
                    int64_t x_stride, float* out, int n_threads)
{
    int rc = check_mm(type, w, N, K, x, M, x_stride, out);
    if (rc) return rc;
    if (type != TSO_TYPE_Q8_0 && type != TSO_TYPE_Q4_K && type != TSO_TYPE_MXFP4) return -2;
    const int64_t row_bytes = tso_row_size(type, K);
    const int64_t act_bytes = type == TSO_TYPE_Q4_K ? K / 256 * Q8_K_BYTES : K / 32 * Q8_0_BYTES;
    uint8_t* act = (uint8_t*)malloc((size_t)(act_bytes * M));
    if (!act) return -1;
    for (int64_t m = 0; m < M; ++m) {
        if (type == TSO_TYPE_Q4_K) tso_quantize_q8_K(x + m * x_stride, act + m * act_bytes, K);
        else tso_quantize_q8_0(x + m * x_stride, act + m * act_bytes, K);
    }
    if (n_threads < 1) n_threads = 1;
#pragma omp parallel for schedule(static) num_threads(n_threads)
    for (int64_t n = 0; n < N; ++n) {
        const uint8_t* wr = (const uint8_t*)w + n * row_bytes;
        for (int64_t m = 0; m < M; ++m) {
            const uint8_t* ar = act + m * act_bytes;
            float v = type == TSO_TYPE_Q8_0 ? vdot_q8_0(K, wr, ar)
                    : type == TSO_TYPE_Q4_K ? vdot_q4_K(K, wr, ar)
                                            : vdot_mxfp4(K, wr, ar);
            out[m * N + n] = v;
        }
    }
    free(act);
    return 0;
}

/* ------------------------------------------------------------------ */
/* MoE (GPT-OSS)                                                       */
/* ------------------------------------------------------------------ */

/* Per token: top-k by repeated argmax (strict >, so the first maximum wins ties),
 * then softmax over the k selected logits.
 * Reference: GptOssModel.cs:814-865 (MoERoute, after the router linear). */
void tso_moe_route(const float* logits, int T, int E, int k, int32_t* ids, float* weights)
{
    for (int t = 0; t < T; ++t) {
        const float* row = logits + (size_t)t * E;
        int32_t* sel = ids + (size_t)t * k;
        float* wv = weights + (size_t)t * k;
        for (int s = 0; s < k; ++s) {
            int best = 0;
            float best_val = -INFINITY;
            for (int i = 0; i < E; ++i) {
                int taken = 0;
                for (int j = 0; j < s; ++j)
                    if (sel[j] == i) { taken = 1; break; }
                if (!taken && row[i] > best_val) { best_val = row[i]; best = i; }
            }
            sel[s] = best;
            wv[s] = row[best];
        }
        float mx = -INFINITY;
        for (int s = 0; s < k; ++s)
            if (wv[s] > mx) mx = wv[s];
        float sum = 0;
        for (int s = 0; s < k; ++s) {
            wv[s] = expf(wv[s] - mx);
            sum += wv[s];
        }
        if (sum > 0)
            for (int s = 0; s < k; ++s) wv[s] /= sum;
    }
}

/* Stable counting sort of the T*k (token, slot) assignments by expert id.
 * Reference: GptOssModel.cs:755-777. */
void tso_moe_group(const int32_t* ids, const float* weights, int T, int E, int k,
                   int32_t* expert_offsets, int32_t* token_map, float* weight_map)
{
    int32_t* fill = (int32_t*)calloc((size_t)E + 1, sizeof(int32_t));
    for (int i = 0; i < T * k; ++i) fill[ids[i]]++;
    expert_offsets[0] = 0;
    for (int e = 0; e < E; ++e) expert_offsets[e + 1] = expert_offsets[e] + fill[e];
    for (int e = 0; e < E; ++e) fill[e] = expert_offsets[e];
    for (int t = 0; t < T; ++t)
        for (int s = 0; s < k; ++s) {
            int e = ids[t * k + s];
            int pos = fill[e]++;
            token_map[pos] = t;
            if (weights && weight_map) weight_map[pos] = weights[t * k + s];
        }
    free(fill);
}

/* gate = gu[0:F], up = gu[F:2F]; x = min(gate, limit); y = clamp(up, -limit, limit);
 * out = x * sigmoid(alpha * x) * (y + 1).  Scalar form of the reference (its SIMD body
 * uses a polynomial exp; the scalar tail uses MathF.Exp).
 * Reference: GptOssModel.cs:901-934, constants :45-46 (alpha 1.702, limit 7). */
void tso_swiglu_oai(float* gate_up, int rows, int half_dim, float alpha, float limit, float* out)
{
    for (int r = 0; r < rows; ++r) {
        const float* g = gate_up + (size_t)r * 2 * half_dim;
        const float* u = g + half_dim;
        float* o = out + (size_t)r * half_dim;
        for (int i = 0; i < half_dim; ++i) {
            float xg = g[i] < limit ? g[i] : limit;
            float yu = u[i] < -limit ? -limit : (u[i] > limit ? limit : u[i]);
            float glu = xg / (1.0f + expf(alpha * (-xg)));
            o[i] = glu * (yu + 1.0f);
        }
    }
}

/* ---- fused wrappers of the bridge (ggml graphs of ggml_ops_fused.cpp:21-640) ------------------- */

/* ggml_rms_norm followed by ggml_mul with the norm weight.
 * Reference: ggml-cpu/ops.cpp:3646-3695 (ggml_compute_forward_rms_norm_f32: squares in fp32, summed in
 * ggml_float = double in index order, mean = sum/ne00 and scale = 1.0f/sqrtf(mean + eps) in fp32,
 * y = x * scale), then the graph's ggml_mul (ggml_ops_fused.cpp:161-162): (x * scale) * w. */
void tso_rms_norm_mul(const float* x, int64_t rows, int64_t K, int64_t ldx, const float* w, float eps, float* out)
{
    for (int64_t r = 0; r < rows; ++r) {
        const float* xr = x + r * ldx;
        double sum = 0.0;
        for (int64_t i = 0; i < K; ++i) sum += (double)(xr[i] * xr[i]);
        const float mean = (float)(sum / (double)K);
        const float scale = 1.0f / sqrtf(mean + eps);
        for (int64_t i = 0; i < K; ++i) out[r * K + i] = (xr[i] * scale) * w[i];
    }
}

/* ggml_silu on the first half of each row times the second half.
 * Reference: ggml-cpu/vec.h:958-960 (ggml_silu_f32 = x / (1 + expf(-x))), graph ggml_ops_fused.cpp:577-588. */
void tso_silu_mul(const float* gate_up, int64_t rows, int64_t half_dim, float* out)
{
    for (int64_t r = 0; r < rows; ++r) {
        const float* g = gate_up + r * 2 * half_dim;
        const float* u = g + half_dim;
        for (int64_t i = 0; i < half_dim; ++i) out[r * half_dim + i] = (g[i] / (1.0f + expf(-g[i]))) * u[i];
    }
}

static void linear_bias(int type, const void* w, const float* bias, int64_t N, int64_t K,
                        const float* x, int64_t M, float* out)
{
    double* tmp = (double*)malloc((size_t)(M * N) * sizeof(double));
    tso_matmul_f64(type, w, N, K, x, M, K, tmp);
    for (int64_t m = 0; m < M; ++m)
        for (int64_t n = 0; n < N; ++n) {
            float v = (float)tmp[m * N + n];
            out[m * N + n] = bias ? v + bias[n] : v;
        }
    free(tmp);
}

/* Full expert stage given routing: gather rows per expert, gate_up linear (+bias),
 * SwiGLU-OAI, down linear (+bias), weighted scatter-add into out[T x H] (zeroed first).
 * T == 1 visits experts in selection order, T > 1 in ascending expert order.
 * Weights are [E][rows][K] raw blocks, gate_up rows = 2F (gate rows then up rows).
 * Reference: GptOssModel.cs:699-812 (MoEForward*), :867-898 (ExpertFFN), :974-994 (bias). */
int tso_moe_forward(int type, const void* gate_up_w, const float* gate_up_b, const void* down_w,
                    const float* down_b, int E, int H, int F, const float* hidden, int T, int k,
                    const int32_t* ids, const float* weights, float* out)
{
    if (!gate_up_w || !down_w || !hidden || !ids || !weights || !out) return -1;
    const int64_t gu_bytes = tso_row_size(type, H) * 2 * F;
    const int64_t dn_bytes = tso_row_size(type, F) * H;
    if (gu_bytes == 0 || dn_bytes == 0) return -1;
    memset(out, 0, (size_t)T * H * sizeof(float));
    int A = T * k;
    int32_t* offs = (int32_t*)malloc(((size_t)E + 1) * sizeof(int32_t));
    int32_t* tmap = (int32_t*)malloc((size_t)A * sizeof(int32_t));
    float* wmap = (float*)malloc((size_t)A * sizeof(float));
    int32_t* emap = (int32_t*)malloc((size_t)(A > E ? A : E) * sizeof(int32_t));   /* T > 1 lists all E experts */
    int groups;
    if (T == 1) {
        groups = k;
        for (int s = 0; s < k; ++s) { offs[s] = s; tmap[s] = 0; wmap[s] = weights[s]; emap[s] = ids[s]; }
        offs[k] = k;
    } else {
        groups = E;
        tso_moe_group(ids, weights, T, E, k, offs, tmap, wmap);
        for (int e = 0; e < E; ++e) emap[e] = e;
    }
    for (int g = 0; g < groups; ++g) {
        int cnt = offs[g + 1] - offs[g];
        if (cnt == 0) continue;
        int e = (T == 1) ? emap[g] : g;
        float* xin = (float*)malloc((size_t)cnt * H * sizeof(float));
        for (int i = 0; i < cnt; ++i)
            memcpy(xin + (size_t)i * H, hidden + (size_t)tmap[offs[g] + i] * H, (size_t)H * sizeof(float));
        float* gu = (float*)malloc((size_t)cnt * 2 * F * sizeof(float));
        linear_bias(type, (const uint8_t*)gate_up_w + (size_t)e * gu_bytes,
                    gate_up_b ? gate_up_b + (size_t)e * 2 * F : NULL, 2 * F, H, xin, cnt, gu);
        float* act = (float*)malloc((size_t)cnt * F * sizeof(float));
        tso_swiglu_oai(gu, cnt, F, 1.702f, 7.0f, act);
        float* dn = (float*)malloc((size_t)cnt * H * sizeof(float));
        linear_bias(type, (const uint8_t*)down_w + (size_t)e * dn_bytes,
                    down_b ? down_b + (size_t)e * H : NULL, H, F, act, cnt, dn);
        for (int i = 0; i < cnt; ++i) {
            float* o = out + (size_t)tmap[offs[g] + i] * H;
            const float wgt = wmap[offs[g] + i];
            for (int h = 0; h < H; ++h) o[h] += wgt * dn[(size_t)i * H + h];
        }
        free(xin); free(gu); free(act); free(dn);
    }
    free(offs); free(tmap); free(wmap); free(emap);
    return 0;
}

/* ---- whole-layer decode of the bridge (ggml graph of ggml_ops_transformer.cpp:379-470) ---------------- */

/* ggml_rope_ext with n_dims = head_dim, ext_factor 0, attn_factor 1, no frequency factors, in place on
 * x[n_heads][head_dim].  theta_scale = powf(base, -2/n_dims); theta starts at pos and is multiplied by theta_scale
 * once per pair (fp32); the angle is freq_scale * theta.  mode 0 rotates (x[2i], x[2i+1]), mode 2 (NeoX)
 * (x[i], x[i + n_dims/2]).
 * Reference: ggml-cpu/ops.cpp:5532-5563 (rope_yarn, ggml_rope_cache_init), :5636-5652 (rotate_pairs), :5711, :5742-5775. */
void tso_rope(float* x, int n_heads, int head_dim, int pos, int mode, float base, float freq_scale)
{
    const float theta_scale = powf(base, -2.0f / (float)head_dim);
    const int half = head_dim / 2;
    for (int h = 0; h < n_heads; ++h) {
        float* v = x + (size_t)h * head_dim;
        float theta = (float)pos;
        for (int p = 0; p < half; ++p) {
            const float ang = freq_scale * theta;
            const float c = cosf(ang), s = sinf(ang);
            const int i0 = mode == 2 ? p : 2 * p, i1 = mode == 2 ? p + half : 2 * p + 1;
            const float x0 = v[i0], x1 = v[i1];
            v[i0] = x0 * c - x1 * s;
            v[i1] = x0 * s + x1 * c;
            theta *= theta_scale;
        }
    }
}

/* One query row per head against cache rows [0, total): softmax(q . k * scale) v with scale = 1/sqrt(head_dim),
 * query head h reads KV head h / (heads / kv_heads); caches are [kv_heads][max_seq][head_dim] fp32.  fp64 inside.
 * Reference: the ggml_flash_attn_ext call of ggml_ops_transformer.cpp:436-441 (q [head_dim,1,heads], k/v windows of the
 * caches, scale, no bias, no soft cap) — for one query row that is exactly this softmax-weighted sum. */
void tso_attention_decode(const float* q, const float* kc, const float* vc, int heads, int kv_heads, int head_dim,
                          int max_seq, int total, float* out)
{
    const double scale = 1.0 / sqrt((double)head_dim);
    double* s = (double*)malloc((size_t)total * sizeof(double));
    for (int h = 0; h < heads; ++h) {
        const int kvh = h / (heads / kv_heads);
        const float* qh = q + (size_t)h * head_dim;
        double mx = -INFINITY;
        for (int t = 0; t < total; ++t) {
            const float* kr = kc + ((size_t)kvh * max_seq + t) * head_dim;
            double d = 0.0;
            for (int i = 0; i < head_dim; ++i) d += (double)qh[i] * (double)kr[i];
            s[t] = d * scale;
            if (s[t] > mx) mx = s[t];
        }
        double sum = 0.0;
        for (int t = 0; t < total; ++t) { s[t] = exp(s[t] - mx); sum += s[t]; }
        for (int i = 0; i < head_dim; ++i) {
            double acc = 0.0;
            for (int t = 0; t < total; ++t) acc += s[t] * (double)vc[((size_t)kvh * max_seq + t) * head_dim + i];
            out[(size_t)h * head_dim + i] = (float)(acc / sum);
        }
    }
    free(s);
}

static void linear_f32(int type, const void* w, int64_t N, int64_t K, const float* x, float* out)
{
    double* tmp = (double*)malloc((size_t)N * sizeof(double));
    tso_matmul_f64(type, w, N, K, x, 1, K, tmp);
    for (int64_t n = 0; n < N; ++n) out[n] = (float)tmp[n];
    free(tmp);
}

/* One token through one layer, hidden [hidden_size] in place, K / V rows written at `position`.  Matmuls are the exact
 * (fp64-accumulated) products with the dequantized weights; q_norm / k_norm may be NULL.
 * Reference: ggml_ops_transformer.cpp:379-470 (steps 1-14 of transformer_layer_decode_impl). */
int tso_layer_decode(float* hidden, int hidden_size, const float* attn_norm, const void* qkv_w, int qkv_type,
                     const float* q_norm, const float* k_norm, int head_dim, const void* o_w, int o_type,
                     const float* ffn_norm, const void* gu_w, int gu_type, const void* down_w, int down_type,
                     float* k_cache, float* v_cache, int heads, int kv_heads, int max_seq, int position, float eps,
                     float rope_base, float rope_freq_scale, int intermediate, int rope_mode)
{
    const int q_dim = heads * head_dim, k_dim = kv_heads * head_dim, qkv_n = q_dim + 2 * k_dim;
    if (!hidden || !attn_norm || !qkv_w || !o_w || !ffn_norm || !gu_w || !down_w || !k_cache || !v_cache) return -1;
    if (position < 0 || position >= max_seq || heads % kv_heads) return -1;
    float* normed = (float*)malloc((size_t)hidden_size * sizeof(float));
    float* qkv = (float*)malloc((size_t)qkv_n * sizeof(float));
    float* attn = (float*)malloc((size_t)q_dim * sizeof(float));
    float* o = (float*)malloc((size_t)hidden_size * sizeof(float));
    float* gu = (float*)malloc((size_t)2 * intermediate * sizeof(float));
    float* act = (float*)malloc((size_t)intermediate * sizeof(float));
    tso_rms_norm_mul(hidden, 1, hidden_size, hidden_size, attn_norm, eps, normed);
    linear_f32(qkv_type, qkv_w, qkv_n, hidden_size, normed, qkv);
    float* q = qkv;
    float* k = qkv + q_dim;
    float* v = qkv + q_dim + k_dim;
    if (q_norm)
        for (int h = 0; h < heads; ++h) tso_rms_norm_mul(q + (size_t)h * head_dim, 1, head_dim, head_dim, q_norm, eps, q + (size_t)h * head_dim);
    if (k_norm)
        for (int h = 0; h < kv_heads; ++h) tso_rms_norm_mul(k + (size_t)h * head_dim, 1, head_dim, head_dim, k_norm, eps, k + (size_t)h * head_dim);
    tso_rope(q, heads, head_dim, position, rope_mode, rope_base, rope_freq_scale);
    tso_rope(k, kv_heads, head_dim, position, rope_mode, rope_base, rope_freq_scale);
    for (int h = 0; h < kv_heads; ++h) {
        memcpy(k_cache + ((size_t)h * max_seq + position) * head_dim, k + (size_t)h * head_dim, (size_t)head_dim * sizeof(float));
        memcpy(v_cache + ((size_t)h * max_seq + position) * head_dim, v + (size_t)h * head_dim, (size_t)head_dim * sizeof(float));
    }
    tso_attention_decode(q, k_cache, v_cache, heads, kv_heads, head_dim, max_seq, position + 1, attn);
    linear_f32(o_type, o_w, hidden_size, q_dim, attn, o);
    for (int i = 0; i < hidden_size; ++i) hidden[i] = hidden[i] + o[i];
    tso_rms_norm_mul(hidden, 1, hidden_size, hidden_size, ffn_norm, eps, normed);
    linear_f32(gu_type, gu_w, 2 * (int64_t)intermediate, hidden_size, normed, gu);
    tso_silu_mul(gu, 1, intermediate, act);
    linear_f32(down_type, down_w, hidden_size, intermediate, act, o);
    for (int i = 0; i < hidden_size; ++i) hidden[i] = hidden[i] + o[i];
    free(normed); free(qkv); free(attn); free(o); free(gu); free(act);
    return 0;
}
