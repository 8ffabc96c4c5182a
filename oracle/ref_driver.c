/*
 * TEST INFRASTRUCTURE. Thin harness over the REFERENCE's own ggml sources, compiled
 * in place from the reference checkout by `make ref` into oracle/_ref/ (never copied
 * into this repository).  It only calls ggml's public C API; no reference arithmetic
 * is restated here.  Used to pin the restatement in ts_oracle.c.
 */
#include "ggml.h"
#include "ggml-cpu.h"

#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <math.h>

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

/* Small GGUF files written by the reference's own writer (gguf.cpp): fixed metadata of every value kind the
 * managed reader handles, plus the given tensors (raw block bytes, ne0 = row length; ne2 > 1 makes a 3-D tensor such as
 * the stacked experts of a MoE layer; ne1 = 1 with ne2 = 1 stays 2-D as ggml writes it).  Pins the GGUF reader. */
#include "gguf.h"

static int write_gguf(const char* path, int alignment, const char* arch, int expert_count, int expert_used, int n_tensors,
                      const char** names, const int* types, const int64_t* ne0, const int64_t* ne1, const int64_t* ne2,
                      const void** data)
{
    size_t total = 1u << 20;
    for (int i = 0; i < n_tensors; ++i)
        total += ggml_row_size((enum ggml_type)types[i], ne0[i]) * (size_t)ne1[i] * (size_t)(ne2 ? ne2[i] : 1) + 4096;
    struct ggml_init_params ip = { total, NULL, false };
    struct ggml_context* ctx = ggml_init(ip);
    if (!ctx) return -1;
    struct gguf_context* g = gguf_init_empty();
    char key[128];
    gguf_set_val_str(g, "general.architecture", arch);
    gguf_set_val_str(g, "general.name", "tiny \xe2\x9c\x93 model");          /* non-ASCII UTF-8 */
    if (alignment != 32) gguf_set_val_u32(g, "general.alignment", (uint32_t)alignment);
    snprintf(key, sizeof key, "%s.block_count", arch);
    gguf_set_val_u32(g, key, 2);
    if (expert_count > 0) {
        snprintf(key, sizeof key, "%s.expert_count", arch);
        gguf_set_val_u32(g, key, (uint32_t)expert_count);
        snprintf(key, sizeof key, "%s.expert_used_count", arch);
        gguf_set_val_u32(g, key, (uint32_t)expert_used);
    }
    gguf_set_val_i32(g, "test.i32", -7);
    gguf_set_val_u8(g, "test.u8", 200);
    gguf_set_val_i8(g, "test.i8", -100);
    gguf_set_val_u16(g, "test.u16", 65000);
    gguf_set_val_i16(g, "test.i16", -30000);
    gguf_set_val_u64(g, "test.u64", 1ull << 40);
    gguf_set_val_i64(g, "test.i64", -(1ll << 41));
    snprintf(key, sizeof key, "%s.attention.layer_norm_rms_epsilon", arch);
    gguf_set_val_f32(g, key, 1e-5f);
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
        struct ggml_tensor* t = (ne2 && ne2[i] > 1) ? ggml_new_tensor_3d(ctx, (enum ggml_type)types[i], ne0[i], ne1[i], ne2[i])
                                                    : ggml_new_tensor_2d(ctx, (enum ggml_type)types[i], ne0[i], ne1[i]);
        ggml_set_name(t, names[i]);
        memcpy(t->data, data[i], ggml_nbytes(t));
        gguf_add_tensor(g, t);
    }
    const int ok = gguf_write_to_file(g, path, false) ? 0 : -2;
    gguf_free(g);
    ggml_free(ctx);
    return ok;
}

int ref_write_gguf(const char* path, int alignment, int n_tensors, const char** names, const int* types,
                   const int64_t* ne0, const int64_t* ne1, const void** data)
{
    return write_gguf(path, alignment, "llama", 0, 0, n_tensors, names, types, ne0, ne1, NULL, data);
}

/* A MoE layer as llama.cpp's converter stores it: the experts of a projection stacked in one 3-D tensor [ne0, ne1, experts]. */
int ref_write_gguf_moe(const char* path, const char* arch, int expert_count, int expert_used, int n_tensors, const char** names,
                       const int* types, const int64_t* ne0, const int64_t* ne1, const int64_t* ne2, const void** data)
{
    return write_gguf(path, 32, arch, expert_count, expert_used, n_tensors, names, types, ne0, ne1, ne2, data);
}

/* ---- known answers for the whole-layer decode, computed by the reference's ggml CPU ops ---------------- */

static int run_graph(struct ggml_context* ctx, struct ggml_tensor* out)
{
    struct ggml_cgraph* g = ggml_new_graph(ctx);
    ggml_build_forward_expand(g, out);
    return ggml_graph_compute_with_ctx(ctx, g, 1) == GGML_STATUS_SUCCESS ? 0 : -3;
}

/* ggml_add_id as the bridge builds it (ggml_ops_matmul.cpp:1218): src [rows, cols, T], bias [rows, E], ids [cols, T] */
int ref_add_id(const float* src, const float* bias, const int32_t* ids, int T, int cols, int rows, int E, float* out)
{
    struct ggml_init_params ip = { 16u << 20, NULL, false };
    struct ggml_context* ctx = ggml_init(ip);
    if (!ctx) return -1;
    struct ggml_tensor* a = ggml_new_tensor_3d(ctx, GGML_TYPE_F32, rows, cols, T);
    struct ggml_tensor* b = ggml_new_tensor_2d(ctx, GGML_TYPE_F32, rows, E);
    struct ggml_tensor* i = ggml_new_tensor_2d(ctx, GGML_TYPE_I32, cols, T);
    memcpy(a->data, src, (size_t)T * cols * rows * sizeof(float));
    memcpy(b->data, bias, (size_t)E * rows * sizeof(float));
    memcpy(i->data, ids, (size_t)T * cols * sizeof(int32_t));
    struct ggml_tensor* y = ggml_add_id(ctx, a, b, i);
    const int rc = run_graph(ctx, y);
    if (rc == 0) memcpy(out, y->data, (size_t)T * cols * rows * sizeof(float));
    ggml_free(ctx);
    return rc;
}

/* ggml_rope_ext as the bridge calls it (ggml_ops_transformer.cpp:403-406): n_dims = head_dim, n_ctx_orig 0,
 * ext_factor 0, attn_factor 1, beta 0 / 0. */
int ref_rope(const float* x, int n_heads, int head_dim, int pos, int mode, float base, float freq_scale, float* out)
{
    struct ggml_init_params ip = { 16u << 20, NULL, false };
    struct ggml_context* ctx = ggml_init(ip);
    if (!ctx) return -1;
    struct ggml_tensor* t = ggml_new_tensor_3d(ctx, GGML_TYPE_F32, head_dim, n_heads, 1);
    memcpy(t->data, x, (size_t)n_heads * head_dim * sizeof(float));
    struct ggml_tensor* p = ggml_new_tensor_1d(ctx, GGML_TYPE_I32, 1);
    ((int32_t*)p->data)[0] = pos;
    struct ggml_tensor* r = ggml_rope_ext(ctx, t, p, NULL, head_dim, mode, 0, base, freq_scale, 0, 1, 0, 0);
    int rc = run_graph(ctx, r);
    if (rc == 0) memcpy(out, r->data, (size_t)n_heads * head_dim * sizeof(float));
    ggml_free(ctx);
    return rc;
}

/* ggml_flash_attn_ext as the bridge calls it (ggml_ops_transformer.cpp:436-441) on fp32 caches
 * [kv_heads][max_seq][head_dim], one query row per head, rows [0, total), no mask. */
int ref_flash_attn(const float* q, const float* kc, const float* vc, int heads, int kv_heads, int head_dim, int max_seq,
                   int total, float* out)
{
    const size_t cache = (size_t)kv_heads * max_seq * head_dim * sizeof(float);
    struct ggml_init_params ip = { 2 * cache + (64u << 20), NULL, false };
    struct ggml_context* ctx = ggml_init(ip);
    if (!ctx) return -1;
    struct ggml_tensor* tq = ggml_new_tensor_3d(ctx, GGML_TYPE_F32, head_dim, 1, heads);
    memcpy(tq->data, q, (size_t)heads * head_dim * sizeof(float));
    struct ggml_tensor* tk = ggml_new_tensor_3d(ctx, GGML_TYPE_F32, head_dim, max_seq, kv_heads);
    struct ggml_tensor* tv = ggml_new_tensor_3d(ctx, GGML_TYPE_F32, head_dim, max_seq, kv_heads);
    memcpy(tk->data, kc, cache);
    memcpy(tv->data, vc, cache);
    struct ggml_tensor* kw = ggml_view_3d(ctx, tk, head_dim, total, kv_heads, tk->nb[1], tk->nb[2], 0);
    struct ggml_tensor* vw = ggml_view_3d(ctx, tv, head_dim, total, kv_heads, tv->nb[1], tv->nb[2], 0);
    struct ggml_tensor* a = ggml_flash_attn_ext(ctx, tq, kw, vw, NULL, 1.0f / sqrtf((float)head_dim), 0.0f, 0.0f);
    int rc = run_graph(ctx, a);
    if (rc == 0) memcpy(out, a->data, (size_t)heads * head_dim * sizeof(float));   /* [head_dim, heads, 1] */
    ggml_free(ctx);
    return rc;
}

/* The layer graph of transformer_layer_decode_impl (ggml_ops_transformer.cpp:379-470), op for op through ggml's public
 * API, computed by the reference's CPU backend (its mul_mat quantizes the activations to int8 blocks, so this is a
 * coarse known answer: it pins the wiring of the graph, not the last digits).  hidden is updated in place; the caches
 * [kv_heads][max_seq][head_dim] receive row `position`. */
int ref_layer_decode(float* hidden, int hidden_size, const float* attn_norm, const void* qkv_w, int qkv_type,
                     const float* q_norm, const float* k_norm, int head_dim, const void* o_w, int o_type,
                     const float* ffn_norm, const void* gu_w, int gu_type, const void* down_w, int down_type,
                     float* k_cache, float* v_cache, int heads, int kv_heads, int max_seq, int position, float eps,
                     float rope_base, float rope_freq_scale, int inter, int rope_mode)
{
    const int q_dim = heads * head_dim, k_dim = kv_heads * head_dim, total = position + 1;
    const size_t cache = (size_t)kv_heads * max_seq * head_dim * sizeof(float);
    const size_t wb = ggml_row_size((enum ggml_type)qkv_type, hidden_size) * (size_t)(q_dim + 2 * k_dim) +
                      ggml_row_size((enum ggml_type)o_type, q_dim) * (size_t)hidden_size +
                      ggml_row_size((enum ggml_type)gu_type, hidden_size) * (size_t)(2 * inter) +
                      ggml_row_size((enum ggml_type)down_type, inter) * (size_t)hidden_size;
    struct ggml_init_params ip = { wb + 2 * cache + (128u << 20), NULL, false };
    struct ggml_context* ctx = ggml_init(ip);
    if (!ctx) return -1;
#define NEW1(n) ggml_new_tensor_1d(ctx, GGML_TYPE_F32, n)
    struct ggml_tensor* input = NEW1(hidden_size);
    struct ggml_tensor* an = NEW1(hidden_size);
    struct ggml_tensor* qn = NEW1(head_dim);
    struct ggml_tensor* kn = NEW1(head_dim);
    struct ggml_tensor* fn = NEW1(hidden_size);
    memcpy(input->data, hidden, (size_t)hidden_size * 4);
    memcpy(an->data, attn_norm, (size_t)hidden_size * 4);
    memcpy(qn->data, q_norm, (size_t)head_dim * 4);
    memcpy(kn->data, k_norm, (size_t)head_dim * 4);
    memcpy(fn->data, ffn_norm, (size_t)hidden_size * 4);
    struct ggml_tensor* wqkv = ggml_new_tensor_2d(ctx, (enum ggml_type)qkv_type, hidden_size, q_dim + 2 * k_dim);
    struct ggml_tensor* wo = ggml_new_tensor_2d(ctx, (enum ggml_type)o_type, q_dim, hidden_size);
    struct ggml_tensor* wgu = ggml_new_tensor_2d(ctx, (enum ggml_type)gu_type, hidden_size, 2 * inter);
    struct ggml_tensor* wdn = ggml_new_tensor_2d(ctx, (enum ggml_type)down_type, inter, hidden_size);
    memcpy(wqkv->data, qkv_w, ggml_nbytes(wqkv));
    memcpy(wo->data, o_w, ggml_nbytes(wo));
    memcpy(wgu->data, gu_w, ggml_nbytes(wgu));
    memcpy(wdn->data, down_w, ggml_nbytes(wdn));
    struct ggml_tensor* pos = ggml_new_tensor_1d(ctx, GGML_TYPE_I32, 1);
    ((int32_t*)pos->data)[0] = position;
    struct ggml_tensor* kcb = ggml_new_tensor_3d(ctx, GGML_TYPE_F32, head_dim, max_seq, kv_heads);
    struct ggml_tensor* vcb = ggml_new_tensor_3d(ctx, GGML_TYPE_F32, head_dim, max_seq, kv_heads);
    memcpy(kcb->data, k_cache, cache);
    memcpy(vcb->data, v_cache, cache);

    struct ggml_tensor* normed = ggml_mul(ctx, ggml_rms_norm(ctx, input, eps), an);
    struct ggml_tensor* qkv = ggml_reshape_1d(ctx, ggml_mul_mat(ctx, wqkv, ggml_reshape_2d(ctx, normed, hidden_size, 1)), q_dim + 2 * k_dim);
    struct ggml_tensor* q_raw = ggml_view_1d(ctx, qkv, q_dim, 0);
    struct ggml_tensor* k_raw = ggml_view_1d(ctx, qkv, k_dim, (size_t)q_dim * 4);
    struct ggml_tensor* v_raw = ggml_view_1d(ctx, qkv, k_dim, (size_t)(q_dim + k_dim) * 4);
    struct ggml_tensor* q_n = ggml_mul(ctx, ggml_rms_norm(ctx, ggml_reshape_2d(ctx, q_raw, head_dim, heads), eps), qn);
    struct ggml_tensor* k_n = ggml_mul(ctx, ggml_rms_norm(ctx, ggml_reshape_2d(ctx, k_raw, head_dim, kv_heads), eps), kn);
    struct ggml_tensor* q_r = ggml_rope_ext(ctx, ggml_reshape_3d(ctx, q_n, head_dim, heads, 1), pos, NULL, head_dim, rope_mode, 0, rope_base, rope_freq_scale, 0, 1, 0, 0);
    struct ggml_tensor* k_r = ggml_rope_ext(ctx, ggml_reshape_3d(ctx, k_n, head_dim, kv_heads, 1), pos, NULL, head_dim, rope_mode, 0, rope_base, rope_freq_scale, 0, 1, 0, 0);
    struct ggml_tensor* q_attn = ggml_permute(ctx, q_r, 0, 2, 1, 3);
    struct ggml_tensor* k_write = ggml_cont(ctx, ggml_permute(ctx, k_r, 0, 2, 1, 3));
    struct ggml_tensor* v_write = ggml_cont(ctx, ggml_permute(ctx, ggml_reshape_3d(ctx, v_raw, head_dim, kv_heads, 1), 0, 2, 1, 3));
    const size_t off = (size_t)position * head_dim * 4;
    struct ggml_tensor* k_cpy = ggml_cpy(ctx, k_write, ggml_view_3d(ctx, kcb, head_dim, 1, kv_heads, kcb->nb[1], kcb->nb[2], off));
    struct ggml_tensor* v_cpy = ggml_cpy(ctx, v_write, ggml_view_3d(ctx, vcb, head_dim, 1, kv_heads, vcb->nb[1], vcb->nb[2], off));
    struct ggml_tensor* k_full = ggml_view_3d(ctx, kcb, head_dim, total, kv_heads, kcb->nb[1], kcb->nb[2], 0);
    struct ggml_tensor* v_full = ggml_view_3d(ctx, vcb, head_dim, total, kv_heads, vcb->nb[1], vcb->nb[2], 0);
    struct ggml_tensor* attn = ggml_flash_attn_ext(ctx, q_attn, k_full, v_full, NULL, 1.0f / sqrtf((float)head_dim), 0.0f, 0.0f);
    struct ggml_tensor* o_flat = ggml_reshape_1d(ctx, ggml_mul_mat(ctx, wo, ggml_reshape_2d(ctx, attn, q_dim, 1)), hidden_size);
    struct ggml_tensor* res1 = ggml_add(ctx, input, o_flat);
    struct ggml_tensor* normed2 = ggml_mul(ctx, ggml_rms_norm(ctx, res1, eps), fn);
    struct ggml_tensor* gu = ggml_reshape_1d(ctx, ggml_mul_mat(ctx, wgu, ggml_reshape_2d(ctx, normed2, hidden_size, 1)), 2 * inter);
    struct ggml_tensor* gate = ggml_view_1d(ctx, gu, inter, 0);
    struct ggml_tensor* up = ggml_view_1d(ctx, gu, inter, (size_t)inter * 4);
    struct ggml_tensor* ffn = ggml_mul(ctx, ggml_silu(ctx, gate), up);
    struct ggml_tensor* down = ggml_reshape_1d(ctx, ggml_mul_mat(ctx, wdn, ggml_reshape_2d(ctx, ffn, inter, 1)), hidden_size);
    struct ggml_tensor* result = ggml_add(ctx, res1, down);
    struct ggml_cgraph* g = ggml_new_graph(ctx);
    ggml_build_forward_expand(g, k_cpy);          /* cache writes first, as the bridge orders them */
    ggml_build_forward_expand(g, v_cpy);
    ggml_build_forward_expand(g, result);
    const int rc = ggml_graph_compute_with_ctx(ctx, g, 1) == GGML_STATUS_SUCCESS ? 0 : -3;
    if (rc == 0) {
        memcpy(hidden, result->data, (size_t)hidden_size * 4);
        memcpy(k_cache, kcb->data, cache);
        memcpy(v_cache, vcb->data, cache);
    }
    ggml_free(ctx);
    return rc;
#undef NEW1
}
