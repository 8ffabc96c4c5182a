// Internal declarations shared by the C-ABI shim and the gfx950 kernels.
#pragma once

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>
#include <string>

namespace tship {

// GGUF tensor type ids (TensorSharp.Runtime/GgufReader.cs:26-37)
constexpr int kTypeF32 = 0;
constexpr int kTypeF16 = 1;
constexpr int kTypeQ4_0 = 2;
constexpr int kTypeQ4_1 = 3;
constexpr int kTypeQ5_0 = 6;
constexpr int kTypeQ5_1 = 7;
constexpr int kTypeQ8_0 = 8;
constexpr int kTypeQ8_1 = 9;
constexpr int kTypeQ4_K = 12;
constexpr int kTypeQ5_K = 13;
constexpr int kTypeQ6_K = 14;
constexpr int kTypeIQ4_NL = 20;
constexpr int kTypeBF16 = 30;
constexpr int kTypeMXFP4 = 39;

// elements per block / bytes per block; 0 for unsupported types
// (sizes: TensorSharp.Runtime/GgufReader.cs:303-369)
inline int64_t block_elems(int type)
{
    switch (type) {
    case kTypeF32: return 1;
    case kTypeQ8_0: return 32;
    case kTypeQ4_K: return 256;
    case kTypeMXFP4: return 32;
    case kTypeF16: case kTypeBF16: return 1;
    case kTypeQ4_0: case kTypeQ4_1: case kTypeQ5_0: case kTypeQ5_1: case kTypeIQ4_NL: case kTypeQ8_1: return 32;
    case kTypeQ5_K: case kTypeQ6_K: return 256;
    default: return 0;
    }
}

inline int64_t block_bytes(int type)
{
    switch (type) {
    case kTypeF32: return 4;
    case kTypeQ8_0: return 34;
    case kTypeQ4_K: return 144;
    case kTypeMXFP4: return 17;
    case kTypeF16: case kTypeBF16: return 2;
    case kTypeQ4_0: case kTypeIQ4_NL: return 18;
    case kTypeQ4_1: return 20;
    case kTypeQ5_0: return 22;
    case kTypeQ5_1: return 24;
    case kTypeQ8_1: return 36;
    case kTypeQ5_K: return 176;
    case kTypeQ6_K: return 210;
    default: return 0;
    }
}

// formats the GEMV / GEMM kernels read: every block format of ManagedQuantizedOps.cs:40-59 except Q8_1 (an activation
// format that no GGUF file stores weights in; see is_matmul_type)
inline bool is_quant_type(int type)
{
    switch (type) {
    case kTypeQ8_0: case kTypeQ4_K: case kTypeMXFP4: case kTypeQ6_K: case kTypeQ5_K: case kTypeQ4_0: case kTypeQ4_1:
    case kTypeQ5_0: case kTypeQ5_1: case kTypeIQ4_NL:
        return true;
    default: return false;
    }
}
inline bool has_gemv(int type)
{
    return type == kTypeQ8_0 || type == kTypeQ4_K || type == kTypeMXFP4 || type == kTypeQ6_K || type == kTypeQ5_K ||
           type == kTypeQ4_0 || type == kTypeQ4_1 || type == kTypeQ5_0 || type == kTypeQ5_1 || type == kTypeIQ4_NL;
}
// formats with a dequantizer (DequantizeToF32, embedding gather): every block format the managed code reads
// (ManagedQuantizedOps.cs:40-59)
inline bool is_dequant_type(int type) { return type != kTypeF32 && block_elems(type) != 0; }

void set_last_error(const std::string& msg);
void clear_last_error();
bool hip_ok(hipError_t e, const char* what);   // sets last error on failure
bool raise_lds_limit(const void* kernel, size_t dynamic_lds_bytes);   // remembered per kernel and device

struct DeviceInfo {
    int num_cus;
    size_t lds_per_block_optin;
};
const DeviceInfo& device_info();

// ---- kernel launchers (all asynchronous on `stream`; return false + last error on bad launch) ----

// dst[n] fp32 = dequant(src); bit-exact with the managed dequantizers.
bool launch_dequant(int type, const void* src, int64_t n, float* dst, hipStream_t stream);
// dst[i, 0..K) = row ids[i] of the weight (type F32 or quantized), rows of bad indices are zero-filled; n_ids <= 65535
bool launch_get_rows(int type, const void* src, int64_t row_bytes, int64_t ne1, const int32_t* ids, int64_t n_ids, int64_t K,
                     float* dst, int64_t ldd, hipStream_t stream);

// y[N] = W[N x K] * x[K] (+ add[N] when given; add may be y); W raw GGUF blocks, row-major; w_bytes = N * row_size.
// act: 0 plain x; 1 RMSNorm(x, eps) * norm_w (x * norm_w is staged, the scale applied to the row sums); 2 x is a [2K]
// row gate|up and the staged activation is silu(gate) * up.
bool launch_gemv(int type, const void* w, int64_t w_bytes, const float* x, float* y, int N, int K,
                 hipStream_t stream, const float* add = nullptr, int act = 0, const float* norm_w = nullptr, float eps = 0.f);
int gemv_rms_max_k();
// largest K the GEMV kernel stages in LDS for this type
int gemv_max_k(int type);

// `count` independent GEMVs of one block type in a single launch (count <= gemv_max_group()).
struct GemvArgs {
    const void* w;
    int64_t w_bytes;
    const float* x;
    float* y;
    int N;
    int K;
    const int* expert_id = nullptr;   // optional device pointer (MoE): weight = w + expert_id[0] * expert_stride
    int64_t expert_stride = 0;
    int n_experts = 0;                // with expert_id: ids outside [0, n_experts) make the problem read zeros
    int pair_rows = 0;                // F > 0: W is F gate rows then F up rows (N = 2F) and y[j] = glu(gate_j, up_j), j < F
    int pair_kind = 0;                // 0: glu = silu(g) * u; 1: GPT-OSS SwiGLU at the store (act must be 0; norm_w the optional
                                      // [E][2F] bias indexed by expert_id, eps = alpha, limit = clamp)
    // routed sum (MoE down projection of one token): w is the stack of n_experts matrices expert_stride bytes apart
    // (w_bytes spans the stack), x holds gemv_routed_slots(type) activation vectors of K floats back to back, and
    // y[h] = sum_slot slot_w[slot] * (W[slot_ids[slot]][h] . x[slot] + slot_bias[slot_ids[slot]][h]) in slot order; slots
    // whose id lies outside [0, n_experts) add nothing.  Excludes expert_id, pair_rows, add and the activation modes.
    const int* slot_ids = nullptr;    // device [slots]
    const float* slot_w = nullptr;    // device [slots]
    const float* slot_bias = nullptr; // device [n_experts][N], optional
    const float* add = nullptr;       // optional: y = add + W x (add may be y)
    int act = 0;                      // activation mode, see launch_gemv
    const float* norm_w = nullptr;
    float eps = 0.f;
    float limit = 0.f;
};
int gemv_max_group();
// slots (experts per token) the routed-sum mode of a format combines: 64 / lanes per row, 0 where the format has none
int gemv_routed_slots(int type);
// diagnostics: per-wavefront time stamps of the GEMV launches (see TSHip_SetGemvTimeline)
int gemv_timeline_slots();
void set_gemv_timeline(uint64_t* device_buffer, int64_t wavefronts);
bool launch_gemv_group(int type, int count, const GemvArgs* args, hipStream_t stream);

// ---- prefill GEMM ---------------------------------------------------------------------------
// Workspace layout: [M floats of row scales, padded to 256 B][M x Kp fp16 activations].
size_t gemm_workspace_bytes(int M, int K);
int gemm_tile_m(int type, int M, int N);   // rows of activations per tile for a plain (ungrouped) launch

// fp32 activations -> workspace (fp16 in the weight format's unpack order + per-row scales);
// row_map (device, optional) gathers source rows.
// norm_w (device, optional) applies RMSNorm first: x <- x / sqrt(mean(x^2) + eps) * norm_w.
bool launch_convert_x(int type, const float* x, int64_t ldx, const int* row_map, int M, int K, void* workspace,
                      hipStream_t stream, const float* norm_w = nullptr, float eps = 0.f, int layout = 0);
// layout of the converted activations the GEMM of this shape reads (plain launches): 0 fp16, 1 MX fp6 pairs (MXFP4 on the
// block-scaled matrix instruction); pass it to launch_convert_x and to launch_gemm
int gemm_x_layout(int type, int M, int N, int K);
// The same for the activations of an expert's down projection: row m is SwiGLU-OAI of (gate | up)[m] (+ the bias
// row of expert_of[m]), formed while it is read.
bool launch_convert_x_swiglu(int type, const float* gate_up, const float* bias, const int* expert_of, float alpha, float limit,
                             int M, int F, void* workspace, hipStream_t stream, int layout = 0);

// Grouped launches (MoE): m-tiles enumerated by device tables; weights of expert e start at
// w + e * expert_stride (or, for experts held by pointer, at w + expert_off[e]) and span expert_stride bytes each.
struct GemmTiles {
    const int* expert;
    const int* row0;
    const int* rows;
    int count;
    int bm;
    int64_t expert_stride;
    const int64_t* expert_off = nullptr;   // device table, optional
};

// The gate_up GEMM of MXFP4 gpt-oss experts on 32-row tiles with the down projection's activations as its result:
// bias + SwiGLU-OAI of every (gate, up) column pair, converted to the MX activation layout in workspace_out (a
// gemm_workspace_bytes(M, F) buffer), without the [M x 2 F] matrix in between (48-row tiles pass through act, an
// [M x F] fp32 scratch matrix, on the way).  workspace holds the MX activations of
// the M rows x K (launch_convert_x with layout 1).  gemm_swiglu_mx_fits: whether the shape can take this path.
bool gemm_swiglu_mx_fits(int F, int K);
bool launch_gemm_swiglu_mx(const void* w, const void* workspace, void* workspace_out, float* act, const float* bias, float alpha,
                           float limit, int M, int F, int K, const GemmTiles* tiles, hipStream_t stream);

// c[row] (row = c_rows ? c_rows[m] : m) [N] = x16[m] . W^T * scale[m], m < M
// accumulate: c[row] += ... instead of c[row] = ...
// chunk_ws (device): where the sums of K chunks go, gemm_chunk_ws_bytes() of them (a shape whose chunk sums do not fit
// what is passed runs with whole K per tile, or fails when its kernel cannot do without chunks).  Nothing is allocated.
bool launch_gemm(int type, const void* w, int64_t w_bytes, const void* workspace, float* c, int64_t ldc,
                 const int* c_rows, int M, int N, int K, const GemmTiles* tiles, hipStream_t stream, bool accumulate = false,
                 void* chunk_ws = nullptr, size_t chunk_ws_bytes = 0, int x_layout = 0);
// bytes of chunk_ws the same launch uses (0 for most shapes); only tiles->bm and tiles->count are read
size_t gemm_chunk_ws_bytes(int type, int M, int N, int K, const GemmTiles* tiles, bool accumulate, int x_layout = -1);
// the kernels address one weight (or one launch's converted activations) with 32-bit offsets
constexpr int64_t kMaxOperandBytes = ((int64_t)1 << 31) - 64;

// ---- fused wrappers around the matmul (RMSNorm prologue, SiLU-gated FFN) ------------------------
// out[m, 0..K) = x[m] / sqrt(mean(x[m]^2) + eps) * w   (ggml_rms_norm then ggml_mul), contiguous rows
bool launch_rms_norm_rows(const float* x, int64_t ldx, const float* w, float eps, int M, int K, float* out, hipStream_t stream);
// out[m, j] = silu(gu[m, j]) * gu[m, half + j], j < half
bool launch_silu_mul(const float* gu, int64_t ldgu, int M, int half, float* out, hipStream_t stream);

// x[i] = max(x[i], 0)^2 in place
bool launch_relu_sqr(float* x, int64_t n, hipStream_t stream);
// out[m][j] = (base ? base[m][j] : 0) + sum_{e < count} w.v[e] * rows[e * set_stride + m * N + j], added in index order;
// base may be out
constexpr int kMaxWeightedRows = 36;
struct WeightedSumCoeffs {
    float v[kMaxWeightedRows];
};
bool launch_weighted_sum(const float* rows, int64_t set_stride, const WeightedSumCoeffs& w, int count, int M, int N, const float* base,
                         int64_t ldb, float* out, int64_t ldo, hipStream_t stream);
// Tables of a tile-table GEMM launch (GemmTiles with expert_off) over experts held by pointer, all on the same M rows:
// member e of the launch has its weight at base + off[e] and its activation / result rows at slot[e] * M; row_map
// (optional, map_rows entries) becomes i -> i % M, the gather that repeats the M source rows per member of the set.
struct ExpertTileSpec {
    int64_t off[kMaxWeightedRows];
    int slot[kMaxWeightedRows];
    int count;
};
bool launch_expert_tiles(const ExpertTileSpec& spec, int M, int bm, int* tile_expert, int* tile_row0, int* tile_rows, int64_t* off_table,
                         int* row_map, int map_rows, hipStream_t stream);
// y[m][n] (+)= sum_k W[n][k] x[m][k] for a dense row-major weight of type F32, F16 or BF16
bool launch_dense_matmul(int type, const void* w, const float* x, int64_t ldx, float* y, int64_t ldy, int M, int N, int K,
                         bool accumulate, hipStream_t stream);
// out[t][s][0..rows) = W[ids[t][s]] (rows x K, fp32) * x[t][s % slots]; strides in elements, innermost stride 1;
// T * cols <= 65535; rows of an id outside [0, E) are zero
bool launch_add_id_f32(const float* src, int64_t s_s0, int64_t s_s1, const float* bias, int64_t b_s0, int E, const int32_t* ids, int T,
                       int cols, int rows, float* out, int64_t o_s0, int64_t o_s1, hipStream_t stream);
bool launch_mul_mat_id_f32(const float* w, int64_t w_s0, int64_t w_s1, int E, int rows, int K, const float* x, int64_t x_s0, int64_t x_s1,
                           int slots, const int32_t* ids, int T, int cols, float* out, int64_t o_s0, int64_t o_s1, hipStream_t stream);
inline bool is_dense_type(int type) { return type == kTypeF32 || type == kTypeF16 || type == kTypeBF16; }
// every weight type the matmul entry points take; Q8_1 weights are dequantized to fp32 in slices of rows and then take
// the dense kernel
inline bool is_matmul_type(int type) { return is_quant_type(type) || is_dense_type(type) || type == kTypeQ8_1; }

// ---- single-token attention of the whole-layer decode ---------------------------------------
// qkv = [q heads | k heads | v heads], head_dim each.  Per head: RMSNorm (weights may be null) + RoPE at `position`; the
// new k / v row goes into row `position` of the caches [num_kv_heads][max_seq_len][head_dim];
// out[h] = softmax(q[h] . K^T / sqrt(head_dim)) V over cache rows [0, position]
size_t attention_decode_ws_bytes(int num_heads, int total);
bool launch_attention_decode(const float* qkv, const float* q_norm_w, const float* k_norm_w, float eps, float rope_base,
                             float rope_freq_scale, int rope_mode, float* k_cache, float* v_cache, int num_heads, int num_kv_heads,
                             int head_dim, int max_seq_len, int position, float* partial_ws, float* out, hipStream_t stream,
                             const float* prefetch0 = nullptr, const float* prefetch1 = nullptr, int prefetch_floats = 0);
// prefetch0 / prefetch1: optional vectors of prefetch_floats floats that later launches ask for first (norm weights); spare
// workgroups of the attention launch read them so that they wait in the caches

// ---- MoE (GPT-OSS expert stage) -------------------------------------------------------------
// ids / weights: [T x k] device; top-k by repeated argmax (first maximum wins), softmax over the k logits.
bool launch_moe_route(const float* logits, int64_t ld, int T, int E, int k, int* ids, float* weights, hipStream_t stream);

struct MoeMaps {            // all device pointers, A = T * k assignments
    int* offsets;           // [E + 1]
    int* token_of;          // [A] token of sorted row
    int* expert_of;         // [A] expert of sorted row
    int* pos_of;            // [A] sorted row of assignment (t, s); -1 for an invalid expert id
    int* tile_expert;       // [max_tiles]
    int* tile_row0;         // [max_tiles]
    int* tile_rows;         // [max_tiles], 0 past the last tile
};
// counting sort of the assignments by expert (row order inside an expert is unspecified) + m-tile table for the grouped GEMM
bool launch_moe_group(const int* ids, int A, int k, int E, int bm, int max_tiles, const MoeMaps& maps, hipStream_t stream);
// out[t][h] = sum_s w[t][s] * (dn[pos_of[t*k+s]][h] + b[e][h]); order: ascending expert (or slot order); assignments whose
// expert id lies outside [0, E) contribute nothing
bool launch_moe_combine(const float* dn, const float* bias, const int* ids, const float* weights, const int* pos_of, int T,
                        int k, int E, int H, bool slot_order, float* out, int64_t ldo, hipStream_t stream);

}  // namespace tship
