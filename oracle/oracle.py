"""TEST INFRASTRUCTURE: ctypes loader for the CPU oracle (liboracle.so) and, where it
was built, the reference's own ggml CPU code (oracle/_ref/libggml_ref.so).

Only tests, the smoke check and the benchmark's cpu_baseline leg may import this
module.  The shipped HIP library never depends on it.
"""
import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))

F32, Q8_0, Q4_K, MXFP4 = 0, 8, 12, 39
F16, Q4_0, Q4_1, Q5_0, Q5_1, Q5_K, Q6_K, IQ4_NL, BF16 = 1, 2, 3, 6, 7, 13, 14, 20, 30
Q8_1 = 9
TYPES = {"q8_0": Q8_0, "q4_k": Q4_K, "mxfp4": MXFP4}
# formats with a dequantizer only (embedding gather, DequantizeToF32); Q6_K also has matmuls on the GPU
MORE_TYPES = {"f16": F16, "bf16": BF16, "q4_0": Q4_0, "q4_1": Q4_1, "q5_0": Q5_0, "q5_1": Q5_1, "q5_k": Q5_K,
              "q6_k": Q6_K, "iq4_nl": IQ4_NL}
BLOCK = {F32: (1, 4), Q8_0: (32, 34), Q4_K: (256, 144), MXFP4: (32, 17), F16: (1, 2), BF16: (1, 2), Q4_0: (32, 18),
         Q4_1: (32, 20), Q5_0: (32, 22), Q5_1: (32, 24), Q5_K: (256, 176), Q6_K: (256, 210), IQ4_NL: (32, 18), Q8_1: (32, 36)}

_f32p = C.POINTER(C.c_float)
_f64p = C.POINTER(C.c_double)
_i32p = C.POINTER(C.c_int32)


# argument list shared by tso_layer_decode and the reference driver's ref_layer_decode
LAYER_ARGS = [_f32p, C.c_int, _f32p, C.c_void_p, C.c_int, _f32p, _f32p, C.c_int, C.c_void_p, C.c_int, _f32p, C.c_void_p, C.c_int,
              C.c_void_p, C.c_int, _f32p, _f32p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_float, C.c_float, C.c_float, C.c_int,
              C.c_int]


def _layer_call(fn, hidden, layer, k_cache, v_cache, heads, kv_heads, head_dim, position, eps, rope_base, rope_freq_scale,
                rope_mode):
    """layer: dict attn_norm, qkv=(type, bytes), q_norm, k_norm, o=(type, bytes), ffn_norm, gate_up=(type, bytes),
    down=(type, bytes), intermediate.  hidden / caches are updated in place (fp32, C-contiguous)."""
    f = lambda a: None if a is None else _ptr(a, _f32p)
    rc = fn(_ptr(hidden, _f32p), hidden.size, f(layer["attn_norm"]), _vp(layer["qkv"][1]), layer["qkv"][0], f(layer["q_norm"]),
            f(layer["k_norm"]), head_dim, _vp(layer["o"][1]), layer["o"][0], f(layer["ffn_norm"]), _vp(layer["gate_up"][1]),
            layer["gate_up"][0], _vp(layer["down"][1]), layer["down"][0], _ptr(k_cache, _f32p), _ptr(v_cache, _f32p), heads,
            kv_heads, k_cache.shape[1], position, eps, rope_base, rope_freq_scale, layer["intermediate"], rope_mode)
    assert rc == 0, rc


def build(fast=True):
    """Compile the oracle libraries (gcc only)."""
    targets = ["liboracle.so"] + (["liboracle_fast.so"] if fast else [])
    subprocess.run(["make", "-s", "-C", HERE] + targets, check=True)


def build_ref(reference="/root/reference"):
    """Compile the reference's ggml CPU sources in place (only where the checkout exists)."""
    if not os.path.isdir(reference):
        return False
    subprocess.run(["make", "-s", "-j8", "-C", HERE, "ref", f"REF={reference}"], check=True)
    return True


def _ptr(a, ty):
    return a.ctypes.data_as(ty)


def _vp(a):
    return C.c_void_p(a.ctypes.data)


class Oracle:
    def __init__(self, fast=False):
        name = "liboracle_fast.so" if fast else "liboracle.so"
        path = os.path.join(HERE, name)
        if not os.path.exists(path):
            build(fast=fast)
        self.lib = L = C.CDLL(path)
        L.tso_fp16_to_fp32.restype = C.c_float
        L.tso_fp16_to_fp32.argtypes = [C.c_uint16]
        L.tso_fp32_to_fp16.restype = C.c_uint16
        L.tso_fp32_to_fp16.argtypes = [C.c_float]
        L.tso_e8m0_to_fp32_half.restype = C.c_float
        L.tso_e8m0_to_fp32_half.argtypes = [C.c_uint8]
        for f in (L.tso_block_size, L.tso_type_size):
            f.restype = C.c_int64
            f.argtypes = [C.c_int]
        L.tso_row_size.restype = C.c_int64
        L.tso_row_size.argtypes = [C.c_int, C.c_int64]
        L.tso_quantize.restype = C.c_int
        L.tso_quantize.argtypes = [C.c_int, _f32p, C.c_void_p, C.c_int64]
        L.tso_quantize_q8_K.restype = None
        L.tso_quantize_q8_K.argtypes = [_f32p, C.c_void_p, C.c_int64]
        L.tso_dequantize.restype = C.c_int
        L.tso_dequantize.argtypes = [C.c_int, C.c_void_p, C.c_int64, _f32p]
        L.tso_matmul_f64.restype = C.c_int
        L.tso_matmul_f64.argtypes = [C.c_int, C.c_void_p, C.c_int64, C.c_int64, _f32p, C.c_int64,
                                     C.c_int64, _f64p]
        L.tso_matmul_managed.restype = C.c_int
        L.tso_matmul_managed.argtypes = [C.c_int, C.c_void_p, C.c_int64, C.c_int64, _f32p, C.c_int64,
                                         C.c_int64, _f32p, C.c_int, C.c_int]
        L.tso_matmul_ggml.restype = C.c_int
        L.tso_matmul_ggml.argtypes = [C.c_int, C.c_void_p, C.c_int64, C.c_int64, _f32p, C.c_int64,
                                      C.c_int64, _f32p, C.c_int]
        L.tso_moe_route.restype = None
        L.tso_moe_route.argtypes = [_f32p, C.c_int, C.c_int, C.c_int, _i32p, _f32p]
        L.tso_moe_group.restype = None
        L.tso_moe_group.argtypes = [_i32p, _f32p, C.c_int, C.c_int, C.c_int, _i32p, _i32p, _f32p]
        L.tso_rms_norm_mul.restype = None
        L.tso_rms_norm_mul.argtypes = [_f32p, C.c_int64, C.c_int64, C.c_int64, _f32p, C.c_float, _f32p]
        L.tso_silu_mul.restype = None
        L.tso_silu_mul.argtypes = [_f32p, C.c_int64, C.c_int64, _f32p]
        L.tso_swiglu_oai.restype = None
        L.tso_swiglu_oai.argtypes = [_f32p, C.c_int, C.c_int, C.c_float, C.c_float, _f32p]
        L.tso_moe_forward.restype = C.c_int
        L.tso_moe_forward.argtypes = [C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                      C.c_int, C.c_int, C.c_int, _f32p, C.c_int, C.c_int, _i32p,
                                      _f32p, _f32p]
        L.tso_max_threads.restype = C.c_int
        L.tso_rope.restype = None
        L.tso_rope.argtypes = [_f32p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_float, C.c_float]
        L.tso_attention_decode.restype = None
        L.tso_attention_decode.argtypes = [_f32p, _f32p, _f32p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, _f32p]
        L.tso_layer_decode.restype = C.c_int
        L.tso_layer_decode.argtypes = LAYER_ARGS

    # -- helpers ---------------------------------------------------------
    def row_size(self, t, ne):
        return int(self.lib.tso_row_size(t, ne))

    def quantize(self, t, x):
        x = np.ascontiguousarray(x, dtype=np.float32)
        bs, bb = BLOCK[t]
        assert x.size % bs == 0
        out = np.empty(x.size // bs * bb, dtype=np.uint8)
        rc = self.lib.tso_quantize(t, _ptr(x, _f32p), _vp(out), x.size)
        assert rc == 0, rc
        return out

    def quantize_q8_K(self, x):
        x = np.ascontiguousarray(x, dtype=np.float32)
        out = np.empty(x.size // 256 * 292, dtype=np.uint8)
        self.lib.tso_quantize_q8_K(_ptr(x, _f32p), _vp(out), x.size)
        return out

    def dequantize(self, t, raw, n=None):
        raw = np.ascontiguousarray(raw, dtype=np.uint8)
        bs, bb = BLOCK[t]
        if n is None:
            n = raw.size // bb * bs
        out = np.empty(n, dtype=np.float32)
        rc = self.lib.tso_dequantize(t, _vp(raw), n, _ptr(out, _f32p))
        assert rc == 0, rc
        return out

    def matmul_f64(self, t, w, N, K, x):
        x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1, K)
        M = x.shape[0]
        out = np.empty((M, N), dtype=np.float64)
        rc = self.lib.tso_matmul_f64(t, _vp(w), N, K, _ptr(x, _f32p), M, K, _ptr(out, _f64p))
        assert rc == 0, rc
        return out

    def matmul_managed(self, t, w, N, K, x, vec_width=8, threads=1):
        x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1, K)
        M = x.shape[0]
        out = np.empty((M, N), dtype=np.float32)
        rc = self.lib.tso_matmul_managed(t, _vp(w), N, K, _ptr(x, _f32p), M, K, _ptr(out, _f32p),
                                         vec_width, threads)
        assert rc == 0, rc
        return out

    def matmul_ggml(self, t, w, N, K, x, threads=1):
        x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1, K)
        M = x.shape[0]
        out = np.empty((M, N), dtype=np.float32)
        rc = self.lib.tso_matmul_ggml(t, _vp(w), N, K, _ptr(x, _f32p), M, K, _ptr(out, _f32p), threads)
        assert rc == 0, rc
        return out

    def moe_route(self, logits, k):
        logits = np.ascontiguousarray(logits, dtype=np.float32)
        T, E = logits.shape
        ids = np.empty((T, k), dtype=np.int32)
        wts = np.empty((T, k), dtype=np.float32)
        self.lib.tso_moe_route(_ptr(logits, _f32p), T, E, k, _ptr(ids, _i32p), _ptr(wts, _f32p))
        return ids, wts

    def moe_group(self, ids, wts, E):
        ids = np.ascontiguousarray(ids, dtype=np.int32)
        wts = np.ascontiguousarray(wts, dtype=np.float32)
        T, k = ids.shape
        offs = np.empty(E + 1, dtype=np.int32)
        tmap = np.empty(T * k, dtype=np.int32)
        wmap = np.empty(T * k, dtype=np.float32)
        self.lib.tso_moe_group(_ptr(ids, _i32p), _ptr(wts, _f32p), T, E, k, _ptr(offs, _i32p),
                               _ptr(tmap, _i32p), _ptr(wmap, _f32p))
        return offs, tmap, wmap

    def rms_norm_mul(self, x, w, eps):
        x = np.ascontiguousarray(x, dtype=np.float32)
        w = np.ascontiguousarray(w, dtype=np.float32)
        rows, K = x.shape
        out = np.empty((rows, K), dtype=np.float32)
        self.lib.tso_rms_norm_mul(_ptr(x, _f32p), rows, K, K, _ptr(w, _f32p), eps, _ptr(out, _f32p))
        return out

    def silu_mul(self, gate_up):
        gu = np.ascontiguousarray(gate_up, dtype=np.float32)
        rows, two_f = gu.shape
        out = np.empty((rows, two_f // 2), dtype=np.float32)
        self.lib.tso_silu_mul(_ptr(gu, _f32p), rows, two_f // 2, _ptr(out, _f32p))
        return out

    def swiglu_oai(self, gate_up, alpha=1.702, limit=7.0):
        gu = np.ascontiguousarray(gate_up, dtype=np.float32)
        rows, two_f = gu.shape
        out = np.empty((rows, two_f // 2), dtype=np.float32)
        self.lib.tso_swiglu_oai(_ptr(gu, _f32p), rows, two_f // 2, alpha, limit, _ptr(out, _f32p))
        return out

    def rope(self, x, pos, mode, base, freq_scale=1.0):
        y = np.ascontiguousarray(x, dtype=np.float32).copy()
        self.lib.tso_rope(_ptr(y, _f32p), y.shape[0], y.shape[1], pos, mode, base, freq_scale)
        return y

    def attention_decode(self, q, k_cache, v_cache, total):
        q = np.ascontiguousarray(q, dtype=np.float32)
        out = np.empty_like(q)
        self.lib.tso_attention_decode(_ptr(q, _f32p), _ptr(k_cache, _f32p), _ptr(v_cache, _f32p), q.shape[0], k_cache.shape[0],
                                      q.shape[1], k_cache.shape[1], total, _ptr(out, _f32p))
        return out

    def layer_decode(self, hidden, layer, k_cache, v_cache, heads, kv_heads, head_dim, position, eps, rope_base,
                     rope_freq_scale=1.0, rope_mode=2):
        _layer_call(self.lib.tso_layer_decode, hidden, layer, k_cache, v_cache, heads, kv_heads, head_dim, position, eps,
                    rope_base, rope_freq_scale, rope_mode)

    def moe_forward(self, t, gu_w, gu_b, dn_w, dn_b, E, H, F, hidden, ids, wts):
        hidden = np.ascontiguousarray(hidden, dtype=np.float32)
        ids = np.ascontiguousarray(ids, dtype=np.int32)
        wts = np.ascontiguousarray(wts, dtype=np.float32)
        T, k = ids.shape
        out = np.empty((T, H), dtype=np.float32)
        rc = self.lib.tso_moe_forward(
            t, _vp(gu_w), None if gu_b is None else _vp(gu_b), _vp(dn_w),
            None if dn_b is None else _vp(dn_b), E, H, F, _ptr(hidden, _f32p), T, k,
            _ptr(ids, _i32p), _ptr(wts, _f32p), _ptr(out, _f32p))
        assert rc == 0, rc
        return out

    # -- compositions for the bridge's larger fused calls -----------------------------------------
    # Each chains restatements that are pinned on their own (dequantizers, fp64 product, RMSNorm, SiLU) in the order
    # of the bridge's ggml graph; intermediate tensors are rounded to fp32 where the graph holds fp32 tensors.
    def weight_rows(self, t, w, N, K):
        """[N, K] fp32 values of a weight of any type the matmul entry points take"""
        if t == F32:
            return np.ascontiguousarray(w).view(np.float32)[:N * K].reshape(N, K)
        return self.dequantize(t, w, N * K).reshape(N, K)

    def matmul_any_f64(self, t, w, N, K, x):
        """x [M, K] times W^T in fp64; dense types (F32 / F16 / BF16) through numpy, block formats through tso_matmul_f64"""
        if t in (F32, F16, BF16):
            x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1, K)
            return x.astype(np.float64) @ self.weight_rows(t, w, N, K).astype(np.float64).T
        return self.matmul_f64(t, w, N, K, x)

    @staticmethod
    def relu_sqr(x):
        """ggml_relu then ggml_sqr on fp32 (ggml_ops_fused.cpp:1700-1710)"""
        r = np.maximum(np.asarray(x, dtype=np.float32), np.float32(0))
        return r * r

    def expert_ffn(self, x, expert):
        """One expert: W_down * act(x) in fp64 from fp32 activations.  expert: dict(up=(t, raw, N, K), down=(...),
        gate=(...) or None); gate present: silu(W_gate x) * (W_up x) (ggml_ops_fused.cpp:1876-1885), else
        max(W_up x, 0)^2 (ggml_ops_fused.cpp:1700-1712)."""
        up = self.matmul_any_f64(*expert["up"], x).astype(np.float32)
        if expert.get("gate") is not None:
            gate = self.matmul_any_f64(*expert["gate"], x).astype(np.float32)
            act = self.silu_mul(np.concatenate([gate, up], axis=1))
        else:
            act = self.relu_sqr(up)
        return self.matmul_any_f64(*expert["down"], act)

    def expert_set(self, x, experts, weights, base=None):
        """(base +) sum_e weights[e] * expert_e(x), experts added in index order and the base last
        (ggml_ops_fused.cpp:1716-1722, :2094-2121); returns (result fp64, list of per-expert fp64 down outputs)."""
        parts = [self.expert_ffn(x, e) for e in experts]
        acc = None
        for p, wgt in zip(parts, weights):
            term = p * float(np.float32(wgt))
            acc = term if acc is None else acc + term
        if base is not None:
            acc = np.asarray(base, dtype=np.float64) + acc
        return acc, parts

    def outproj_ffn(self, residual, x, out_w, norm_w, eps, gate_up, down, half):
        """FusedOutProjFFN (ggml_ops_fused.cpp:1164-1190): res = residual + W_out x; res + W_down(silu(g) * u) with
        [g | u] = W_gate_up (RMSNorm(res) * norm_w).  Weights are (type, raw, N, K) tuples.  Returns (result fp64,
        fp64 out-projection product, fp64 down product)."""
        mm1 = self.matmul_any_f64(*out_w, x)
        res = (np.asarray(residual, dtype=np.float64) + mm1).astype(np.float32)
        xn = self.rms_norm_mul(res, norm_w, eps)
        gu = self.matmul_any_f64(*gate_up, xn).astype(np.float32)
        assert gu.shape[1] == 2 * half
        mm2 = self.matmul_any_f64(*down, self.silu_mul(gu))
        return res.astype(np.float64) + mm2, mm1, mm2

    def outproj_norm_router(self, residual, x, out_w, norm_w, eps, router):
        """FusedOutProjNormRouter (ggml_ops_fused.cpp:1310-1330): returns (residual + W_out x in fp64, its RMSNorm * norm_w
        in fp32, the router logits in fp64, the fp64 out-projection product)."""
        mm1 = self.matmul_any_f64(*out_w, x)
        res = np.asarray(residual, dtype=np.float64) + mm1
        normed = self.rms_norm_mul(res.astype(np.float32), norm_w, eps)
        return res, normed, self.matmul_any_f64(*router, normed), mm1

    @staticmethod
    def mul_mat_id(experts, x, ids):
        """ggml_mul_mat_id with F32 experts (include/ggml.h:1409-1413; bridge call ggml_ops_matmul.cpp:958-1121):
        out[t, s, :] = experts[ids[t, s]] @ x[t, s % slots], accumulated in fp64.  experts [E, rows, K], x [T, slots, K]."""
        experts = np.asarray(experts, dtype=np.float64)
        x = np.asarray(x, dtype=np.float64)
        ids = np.asarray(ids).astype(np.int64)
        T, cols = ids.shape
        out = np.empty((T, cols, experts.shape[1]), dtype=np.float64)
        for t in range(T):
            for s in range(cols):
                out[t, s] = experts[ids[t, s]] @ x[t, s % x.shape[1]]
        return out


def add_id(src, bias, ids):
    """ggml_add_id (include/ggml.h:886-891; bridge call ggml_ops_matmul.cpp:1123-1290): out[t, s, :] = src[t, s, :] +
    bias[ids[t, s], :] in fp32.  The definition itself, element by element."""
    src = np.asarray(src, dtype=np.float32)
    out = np.empty_like(src)
    for t in range(src.shape[0]):
        for s in range(src.shape[1]):
            out[t, s] = src[t, s] + np.asarray(bias, dtype=np.float32)[int(ids[t, s])]
    return out


class Reference:
    """The reference's own ggml code, compiled from its sources by `make ref`.
    Exists only where the reference checkout was available at build time."""

    PATH = os.path.join(HERE, "_ref", "libggml_ref.so")

    @classmethod
    def available(cls):
        return os.path.exists(cls.PATH)

    def __init__(self):
        self.lib = L = C.CDLL(self.PATH)
        L.ref_quantize.restype = C.c_size_t
        L.ref_quantize.argtypes = [C.c_int, _f32p, C.c_void_p, C.c_int64, C.c_int64]
        L.ref_dequantize.restype = C.c_int
        L.ref_dequantize.argtypes = [C.c_int, C.c_void_p, C.c_int64, _f32p]
        L.ref_row_size.restype = C.c_size_t
        L.ref_row_size.argtypes = [C.c_int, C.c_int64]
        L.ref_fp16_to_fp32.restype = C.c_float
        L.ref_fp16_to_fp32.argtypes = [C.c_uint16]
        L.ref_fp32_to_fp16.restype = C.c_uint16
        L.ref_fp32_to_fp16.argtypes = [C.c_float]
        L.ref_mul_mat.restype = C.c_int
        L.ref_mul_mat.argtypes = [C.c_int, C.c_void_p, C.c_int64, C.c_int64, _f32p, C.c_int64, _f32p,
                                  C.c_int]
        L.quantize_row_q8_K_ref.restype = None
        L.quantize_row_q8_K_ref.argtypes = [_f32p, C.c_void_p, C.c_int64]
        L.ref_rope.restype = C.c_int
        L.ref_rope.argtypes = [_f32p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_float, C.c_float, _f32p]
        L.ref_flash_attn.restype = C.c_int
        L.ref_flash_attn.argtypes = [_f32p, _f32p, _f32p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, _f32p]
        L.ref_layer_decode.restype = C.c_int
        L.ref_layer_decode.argtypes = LAYER_ARGS

    def quantize(self, t, x, n_per_row=None):
        x = np.ascontiguousarray(x, dtype=np.float32)
        bs, bb = BLOCK[t]
        if n_per_row is None:
            n_per_row = x.size
        out = np.empty(x.size // bs * bb, dtype=np.uint8)
        got = self.lib.ref_quantize(t, _ptr(x, _f32p), _vp(out), x.size // n_per_row, n_per_row)
        assert got == out.size, (got, out.size)
        return out

    def quantize_q8_K(self, x):
        x = np.ascontiguousarray(x, dtype=np.float32)
        # zero-filled: the reference leaves bsums of an all-zero block unwritten
        out = np.zeros(x.size // 256 * 292, dtype=np.uint8)
        self.lib.quantize_row_q8_K_ref(_ptr(x, _f32p), _vp(out), x.size)
        return out

    def dequantize(self, t, raw, n=None):
        raw = np.ascontiguousarray(raw, dtype=np.uint8)
        bs, bb = BLOCK[t]
        if n is None:
            n = raw.size // bb * bs
        out = np.empty(n, dtype=np.float32)
        assert self.lib.ref_dequantize(t, _vp(raw), n, _ptr(out, _f32p)) == 0
        return out

    def rope(self, x, pos, mode, base, freq_scale=1.0):
        x = np.ascontiguousarray(x, dtype=np.float32)
        out = np.empty_like(x)
        assert self.lib.ref_rope(_ptr(x, _f32p), x.shape[0], x.shape[1], pos, mode, base, freq_scale, _ptr(out, _f32p)) == 0
        return out

    def flash_attn(self, q, k_cache, v_cache, total):
        q = np.ascontiguousarray(q, dtype=np.float32)
        out = np.empty_like(q)
        assert self.lib.ref_flash_attn(_ptr(q, _f32p), _ptr(k_cache, _f32p), _ptr(v_cache, _f32p), q.shape[0], k_cache.shape[0],
                                       q.shape[1], k_cache.shape[1], total, _ptr(out, _f32p)) == 0
        return out

    def layer_decode(self, hidden, layer, k_cache, v_cache, heads, kv_heads, head_dim, position, eps, rope_base,
                     rope_freq_scale=1.0, rope_mode=2):
        _layer_call(self.lib.ref_layer_decode, hidden, layer, k_cache, v_cache, heads, kv_heads, head_dim, position, eps,
                    rope_base, rope_freq_scale, rope_mode)

    def add_id(self, src, bias, ids):
        """ggml_add_id on the reference's CPU backend"""
        src = np.ascontiguousarray(src, dtype=np.float32)
        bias = np.ascontiguousarray(bias, dtype=np.float32)
        ids = np.ascontiguousarray(ids, dtype=np.int32)
        out = np.empty_like(src)
        T, cols, rows = src.shape
        self.lib.ref_add_id.restype = C.c_int
        assert self.lib.ref_add_id(_ptr(src, _f32p), _ptr(bias, _f32p), _vp(ids), T, cols, rows, bias.shape[0], _ptr(out, _f32p)) == 0
        return out

    def mul_mat(self, t, w, N, K, x, threads=4):
        x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1, K)
        M = x.shape[0]
        out = np.empty((M, N), dtype=np.float32)
        rc = self.lib.ref_mul_mat(t, _vp(w), N, K, _ptr(x, _f32p), M, _ptr(out, _f32p), threads)
        assert rc == 0, rc
        return out
