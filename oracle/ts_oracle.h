/*
 * TEST INFRASTRUCTURE — not part of the shipped library.
 *
 * CPU restatement of the reference arithmetic for the GGUF quantized-matmul
 * path (Q8_0 / Q4_K / MXFP4 matmuls; dequantizers also for the other formats the managed code reads).  Only tests, the smoke check and the
 * cpu_baseline leg of the benchmark may load this library; the HIP library
 * never links or calls it.
 *
 * Every function cites the reference file:line it restates
 * (paths relative to the reference checkout).
 */
#ifndef TS_ORACLE_H
#define TS_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* GGUF tensor type ids: TensorSharp.Runtime/GgufReader.cs:26-37 */
enum {
    TSO_TYPE_F32 = 0, TSO_TYPE_F16 = 1, TSO_TYPE_Q4_0 = 2, TSO_TYPE_Q4_1 = 3, TSO_TYPE_Q5_0 = 6, TSO_TYPE_Q5_1 = 7,
    TSO_TYPE_Q8_0 = 8, TSO_TYPE_Q8_1 = 9, TSO_TYPE_Q4_K = 12, TSO_TYPE_Q5_K = 13, TSO_TYPE_Q6_K = 14, TSO_TYPE_IQ4_NL = 20,
    TSO_TYPE_BF16 = 30, TSO_TYPE_MXFP4 = 39
};

/* scalar helpers */
float    tso_fp16_to_fp32(uint16_t h);
uint16_t tso_fp32_to_fp16(float f);
float    tso_e8m0_to_fp32_half(uint8_t e);

/* type tables */
int64_t tso_block_size(int type);              /* elements per block, 0 if unsupported */
int64_t tso_type_size(int type);               /* bytes per block, 0 if unsupported    */
int64_t tso_row_size(int type, int64_t ne);    /* bytes per row, 0 on error            */

/* weight quantizers (fp32 -> raw GGUF blocks); n must be a block multiple */
void tso_quantize_q8_0(const float* x, void* dst, int64_t n);
void tso_quantize_q4_K(const float* x, void* dst, int64_t n);
void tso_quantize_mxfp4(const float* x, void* dst, int64_t n);
int  tso_quantize(int type, const float* x, void* dst, int64_t n);

/* dequantizers (raw blocks -> fp32); returns 0 ok, -1 bad args, -2 unsupported */
int tso_dequantize(int type, const void* src, int64_t n, float* dst);

/* activation quantizers of the ggml CPU path */
void tso_quantize_q8_K(const float* x, void* dst, int64_t n);

/* matmuls: result[M x N] = x[M x K] * W[N x K]^T ; W raw blocks, row-major */
int tso_matmul_f64(int type, const void* w, int64_t N, int64_t K,
                   const float* x, int64_t M, int64_t x_stride, double* out);
int tso_matmul_managed(int type, const void* w, int64_t N, int64_t K,
                       const float* x, int64_t M, int64_t x_stride,
                       float* out, int vec_width, int n_threads);
int tso_matmul_ggml(int type, const void* w, int64_t N, int64_t K,
                    const float* x, int64_t M, int64_t x_stride,
                    float* out, int n_threads);

/* MoE (GPT-OSS) */
void tso_moe_route(const float* logits, int T, int E, int k, int32_t* ids, float* weights);
void tso_moe_group(const int32_t* ids, const float* weights, int T, int E, int k,
                   int32_t* expert_offsets /* E+1 */, int32_t* token_map /* T*k */,
                   float* weight_map /* T*k */);
void tso_swiglu_oai(float* gate_up, int rows, int half_dim, float alpha, float limit,
                    float* out /* rows x half_dim */);
int tso_moe_forward(int type, const void* gate_up_w, const float* gate_up_b,
                    const void* down_w, const float* down_b,
                    int E, int H, int F, const float* hidden, int T, int k,
                    const int32_t* ids, const float* weights, float* out);

/* whole-layer decode (ggml semantics): RoPE in place on x[n_heads][head_dim]; single-query attention over fp32 caches
 * [kv_heads][max_seq][head_dim]; one token through one layer (hidden in place, caches written at `position`) */
void tso_rope(float* x, int n_heads, int head_dim, int pos, int mode, float base, float freq_scale);
void tso_attention_decode(const float* q, const float* kc, const float* vc, int heads, int kv_heads, int head_dim,
                          int max_seq, int total, float* out);
int tso_layer_decode(float* hidden, int hidden_size, const float* attn_norm, const void* qkv_w, int qkv_type,
                     const float* q_norm, const float* k_norm, int head_dim, const void* o_w, int o_type,
                     const float* ffn_norm, const void* gu_w, int gu_type, const void* down_w, int down_type,
                     float* k_cache, float* v_cache, int heads, int kv_heads, int max_seq, int position, float eps,
                     float rope_base, float rope_freq_scale, int intermediate, int rope_mode);

/* fused wrappers: RMSNorm * weight, SiLU-gated product (ggml semantics) */
void tso_rms_norm_mul(const float* x, int64_t rows, int64_t K, int64_t ldx, const float* w, float eps, float* out);
void tso_silu_mul(const float* gate_up, int64_t rows, int64_t half_dim, float* out);

int tso_max_threads(void);

#ifdef __cplusplus
}
#endif
#endif
