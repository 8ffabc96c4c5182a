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

/* A small GGUF file written by the reference's own writer (gguf.cpp): fixed metadata of every value kind the
 * managed reader handles, plus the given 2-D tensors (raw block bytes, ne0 = row length).  Pins the GGUF reader. */
#include "gguf.h"

int ref_write_gguf(const char* path, int alignment, int n_tensors, const char** names, const int* types,
                   const int64_t* ne0, const int64_t* ne1, const void** data)
{
    size_t total = 1u << 20;
    for (int i = 0; i < n_tensors; ++i) total += ggml_row_size((enum ggml_type)types[i], ne0[i]) * (size_t)ne1[i] + 4096;
    struct ggml_init_params ip = { total, NULL, false };
    struct ggml_context* ctx = ggml_init(ip);
    if (!ctx) return -1;
    struct gguf_context* g = gguf_init_empty();
    gguf_set_val_str(g, "general.architecture", "llama");
    gguf_set_val_str(g, "general.name", "tiny \xe2\x9c\x93 model");          /* non-ASCII UTF-8 */
    if (alignment != 32) gguf_set_val_u32(g, "general.alignment", (uint32_t)alignment);
    gguf_set_val_u32(g, "llama.block_count", 2);
    gguf_set_val_i32(g, "test.i32", -7);
    gguf_set_val_u8(g, "test.u8", 200);
    gguf_set_val_i8(g, "test.i8", -100);
    gguf_set_val_u16(g, "test.u16", 65000);
    gguf_set_val_i16(g, "test.i16", -30000);
    gguf_set_val_u64(g, "test.u64", 1ull << 40);
    gguf_set_val_i64(g, "test.i64", -(1ll << 41));
    gguf_set_val_f32(g, "llama.attention.layer_norm_rms_epsilon", 1e-5f);
    gguf_set_val_f64(g, "test.f64", 0.1);
    gguf_set_val_bool(g, "test.flag", true);
    const char* toks[4] = { "<s>", "</s>", "hello", "w\xc3\xb6rld" };
    gguf_set_arr_str(g, "tokenizer.ggml.tokens", toks, 4);
    const float scores[4] = { 0.0f, -1.5f, 2.25f, -1000.0f };
    gguf_set_arr_data(g, "tokenizer.ggml.scores", GGUF_TYPE_FLOAT32, scores, 4);
    const int32_t ttypes[4] = { 3, 3, 1, 1 };
    gguf_set_arr_data(g, "tokenizer.ggml.token_type", GGUF_TYPE_INT32, ttypes, 4);
    const uint32_t u32s[3] = { 1, 2, 4000000000u };
    gguf_set_arr_data(g, "test.u32s", GGUF_TYPE_UINT32, u32s, 3);
    for (int i = 0; i < n_tensors; ++i) {
        struct ggml_tensor* t = ggml_new_tensor_2d(ctx, (enum ggml_type)types[i], ne0[i], ne1[i]);
        ggml_set_name(t, names[i]);
        memcpy(t->data, data[i], ggml_nbytes(t));
        gguf_add_tensor(g, t);
    }
    const int ok = gguf_write_to_file(g, path, false) ? 0 : -2;
    gguf_free(g);
    ggml_free(ctx);
    return ok;
}
