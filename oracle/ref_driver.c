/*
 * TEST INFRASTRUCTURE. Thin harness over the REFERENCE's own ggml sources, compiled
 * in place from the reference checkout by `make ref` into oracle/_ref/ (never copied
 * into this repository).  It only calls ggml's public C API; no reference arithmetic
 * is restated here.  Used to pin the restatement in ts_oracle.c.
 */
#include "ggml.h"
#include "ggml-cpu.h"

#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* fp32 -> raw blocks with the reference quantizer (ggml_quantize_chunk, no imatrix). */
size_t ref_quantize(int type, const float* src, void* dst, int64_t nrows, int64_t n_per_row)
{
    ggml_quantize_init((enum ggml_type)type);
    return ggml_quantize_chunk((enum ggml_type)type, src, dst, 0, nrows, n_per_row, NULL);
}

/* raw blocks -> fp32 with the reference's to_float trait. */
int ref_dequantize(int type, const void* src, int64_t n, float* dst)
{
    const struct ggml_type_traits* tr = ggml_get_type_traits((enum ggml_type)type);
    if (!tr || !tr->to_float) return -2;
    tr->to_float(src, dst, n);
    return 0;
}

size_t ref_row_size(int type, int64_t ne) { return ggml_row_size((enum ggml_type)type, ne); }
float ref_fp16_to_fp32(uint16_t h) { return ggml_fp16_to_fp32(h); }
uint16_t ref_fp32_to_fp16(float f) { return ggml_fp32_to_fp16(f); }

/* out[M x N] = x[M x K] * W[N x K]^T through ggml_mul_mat on the reference's CPU backend
 * (activations get quantised to the weight type's vec_dot_type inside ggml). */
int ref_mul_mat(int type, const void* w, int64_t N, int64_t K, const float* x, int64_t M,
                float* out, int n_threads)
{
    const size_t wbytes = ggml_row_size((enum ggml_type)type, K) * (size_t)N;
    const size_t need = wbytes + (size_t)(M * K + M * N) * sizeof(float) + (64u << 20);
    struct ggml_init_params ip = { need, NULL, false };
    struct ggml_context* ctx = ggml_init(ip);
    if (!ctx) return -1;
    struct ggml_tensor* tw = ggml_new_tensor_2d(ctx, (enum ggml_type)type, K, N);
    struct ggml_tensor* tx = ggml_new_tensor_2d(ctx, GGML_TYPE_F32, K, M);
    memcpy(tw->data, w, wbytes);
    memcpy(tx->data, x, (size_t)(M * K) * sizeof(float));
    struct ggml_tensor* ty = ggml_mul_mat(ctx, tw, tx);
    struct ggml_cgraph* g = ggml_new_graph(ctx);
    ggml_build_forward_expand(g, ty);
    enum ggml_status st = ggml_graph_compute_with_ctx(ctx, g, n_threads);
    if (st == GGML_STATUS_SUCCESS) memcpy(out, ty->data, (size_t)(M * N) * sizeof(float));
    ggml_free(ctx);
    return st == GGML_STATUS_SUCCESS ? 0 : -3;
}
