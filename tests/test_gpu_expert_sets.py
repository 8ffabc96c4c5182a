"""GPU parity: the bridge's larger fused calls through the C ABI, host-pointer and device forms.

  FusedOutProjFFN / FusedOutProjNormRouter   (ggml_ops_fused.cpp:1057-1380)
  MoEExpertsForward (squared-ReLU experts), MoEExpertsSwiGLUForward, MoEExpertsSwiGLUResidual
                                             (ggml_ops_fused.cpp:1576-2160)
and dense (F32 / F16 / BF16) weights in the matmul entry points.

Reference value: the oracle's compositions (fp64 products of the bit-exact dequantized weights, fp32 RMSNorm / SiLU
in ggml order).  Bar per matmul: max_j |y - ref| <= 1e-3 * ||row of the product||_2; chained matmuls (an FFN behind a
projection, a down projection behind gate/up) pass the first one's error through, so those rows get 2e-3 of the
last product's norm plus 1e-3 of the first's, written at each assert."""
import numpy as np
import pytest

import inputs

from oracle.oracle import F32, F16, BF16, Q8_0, Q4_K, Q6_K, MXFP4

pytestmark = pytest.mark.gpu
T_ = {"q8_0": Q8_0, "q4_k": Q4_K, "mxfp4": MXFP4, "f32": F32, "f16": F16, "bf16": BF16}
EPS = 1e-6


def make(oracle, name, N, K, rng, sigma=0.05):
    """(type, raw bytes, N, K)"""
    v = (rng.standard_normal(N * K) * sigma).astype(np.float32)
    t = T_[name]
    if t == F32:
        raw = v.view(np.uint8).copy()
    elif t == F16:
        raw = v.astype(np.float16).view(np.uint8).copy()
    elif t == BF16:
        raw = (v.view(np.uint32) >> 16).astype(np.uint16).view(np.uint8).copy()
    else:
        raw = oracle.quantize(t, v)
    return (t, raw, N, K)


def qw(desc, device):
    import torch
    from tensorsharp_amd import QuantizedWeight
    t, raw, N, K = desc
    return QuantizedWeight(torch.from_numpy(raw).cuda() if device else raw, t, K, N)


def rownorm(m):
    return np.linalg.norm(np.asarray(m, dtype=np.float64), axis=1, keepdims=True)


def run(hip, device, fn, inout, *tensors_then_rest):
    """calls fn(inout, ...) with numpy arrays moved to the GPU for the device form; returns inout as numpy"""
    import torch
    if not device:
        fn(inout, *tensors_then_rest)
        hip.ClearHostBufferCache()
        return inout
    moved = [torch.from_numpy(a).cuda() if isinstance(a, np.ndarray) else a for a in (inout,) + tensors_then_rest]
    fn(*moved)
    torch.cuda.synchronize()
    return [m.cpu().numpy() if isinstance(m, torch.Tensor) else m for m in moved]


@pytest.mark.parametrize("name", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("M", [1, 5, 70])
@pytest.mark.parametrize("device", [False, True])
def test_dense_weights_in_addmm_quant(hip, oracle, name, M, device):
    import torch
    rng = np.random.default_rng(300 + M)
    N, K = 131, 520          # K % 64 != 0, N % 4 != 0: tails of the lane loop and the row groups
    w = make(oracle, name, N, K, rng)
    x = rng.standard_normal((M, K)).astype(np.float32)
    ref = oracle.matmul_any_f64(*w, x)
    q = qw(w, device)
    if device:
        res = torch.full((M, N), float("nan"), device="cuda")
        hip.AddmmQuantDevice(res, torch.from_numpy(x).cuda(), q.ptr, q.ggml_type, K, N, q.raw_bytes)
        torch.cuda.synchronize()
        got = res.cpu().numpy()
    else:
        got = np.full((M, N), np.nan, np.float32)
        hip.AddmmQuant(got, x, q.ptr, q.ggml_type, K, N, q.raw_bytes)
        hip.ClearHostBufferCache()
    # fp32 accumulation of exact products: far inside the matmul bar of 1e-3 * ||row||
    assert np.all(np.abs(got - ref) <= 1e-5 * rownorm(ref)), float(np.max(np.abs(got - ref) / rownorm(ref)))


@pytest.mark.parametrize("name", ["q8_0", "q4_k", "mxfp4"])
@pytest.mark.parametrize("M", [1, 3, 40])
@pytest.mark.parametrize("device", [False, True])
def test_outproj_ffn(hip, oracle, name, M, device):
    rng = np.random.default_rng(310 + M)
    A, H, F = 768, 512, 768        # attention width, hidden, FFN half width
    out_w = make(oracle, name, H, A, rng)
    gu = make(oracle, name, 2 * F, H, rng)
    dn = make(oracle, name, H, F, rng)
    x = rng.standard_normal((M, A)).astype(np.float32)
    resid = rng.standard_normal((M, H)).astype(np.float32)
    nw = rng.uniform(0.5, 1.5, H).astype(np.float32)
    ref, mm1, mm2 = oracle.outproj_ffn(resid, x, out_w, nw, EPS, gu, dn, F)
    fn = lambda r, i, n: hip.FusedOutProjFFN(r, i, qw(out_w, device), n, EPS, qw(gu, device), qw(dn, device), F)
    got = run(hip, device, fn, resid.copy(), x, nw)
    got = got[0] if device else got
    tol = 1e-3 * rownorm(mm1) + 2e-3 * rownorm(mm2)
    assert np.all(np.abs(got - ref) <= tol), (name, M, device, float(np.max(np.abs(got - ref) / tol)))


@pytest.mark.parametrize("name,router", [("q8_0", "f32"), ("q4_k", "f16"), ("mxfp4", "bf16"), ("q4_k", "q8_0")])
@pytest.mark.parametrize("M", [1, 6])
@pytest.mark.parametrize("device", [False, True])
def test_outproj_norm_router(hip, oracle, name, router, M, device):
    rng = np.random.default_rng(320 + M)
    A, H, E = 512, 768, 128
    out_w = make(oracle, name, H, A, rng)
    rw = make(oracle, router, E, H, rng, 0.2)
    x = rng.standard_normal((M, A)).astype(np.float32)
    resid = rng.standard_normal((M, H)).astype(np.float32)
    nw = rng.uniform(0.5, 1.5, H).astype(np.float32)
    res_ref, normed_ref, logits_ref, mm1 = oracle.outproj_norm_router(resid, x, out_w, nw, EPS, rw)
    normed = np.full((M, H), np.nan, np.float32)
    logits = np.full((M, E), np.nan, np.float32)
    fn = lambda r, i, n, no, lo: hip.FusedOutProjNormRouter(r, i, qw(out_w, device), n, EPS, no, qw(rw, device), lo)
    out = run(hip, device, fn, resid.copy(), x, nw, normed, logits)
    got_res, got_normed, got_logits = (out[0], out[3], out[4]) if device else (out, normed, logits)
    tol = 1e-3 * rownorm(mm1)
    assert np.all(np.abs(got_res - res_ref) <= tol), (name, M, float(np.max(np.abs(got_res - res_ref) / tol)))
    # the norm divides by the RMS of the row (about 1 here) and scales by norm weights <= 1.5
    rms = np.sqrt((res_ref ** 2).mean(axis=1, keepdims=True))
    assert np.all(np.abs(got_normed - normed_ref) <= 2.0 * tol / rms), float(np.max(np.abs(got_normed - normed_ref)))
    tol_l = 1e-3 * rownorm(logits_ref) + np.abs(oracle.weight_rows(*rw[:2], E, H)).sum(axis=1)[None, :] * np.max(2.0 * tol / rms)
    assert np.all(np.abs(got_logits - logits_ref) <= tol_l), float(np.max(np.abs(got_logits - logits_ref) / tol_l))


def experts(oracle, name, n, H, I, N, rng, gated, down_name=None):
    return [dict(gate=make(oracle, name, I, H, rng) if gated else None, up=make(oracle, name, I, H, rng),
                 down=make(oracle, down_name or name, N, I, rng)) for _ in range(n)]


def set_tol(oracle, parts, weights):
    # per expert: 2e-3 of its down product (gate/up errors pass through the activation), scaled by |route weight|
    return sum(2e-3 * abs(float(w)) * rownorm(p) for p, w in zip(parts, weights))


@pytest.mark.parametrize("name", ["q8_0", "q4_k"])
@pytest.mark.parametrize("n,M", [(1, 1), (6, 1), (16, 1), (5, 4)])
@pytest.mark.parametrize("device", [False, True])
def test_experts_relu_squared(hip, oracle, name, n, M, device):
    rng = np.random.default_rng(330 + n + M)
    H, I = 512, 768 if name == "q4_k" else 352
    ex = experts(oracle, name, n, H, I, H, rng, gated=False)
    w = rng.uniform(0.05, 0.6, n).astype(np.float32)
    x = rng.standard_normal((M, H)).astype(np.float32)
    ref, parts = oracle.expert_set(x, ex, w)
    fn = lambda r, i: hip.MoEExpertsForward(r, i, [qw(e["up"], device) for e in ex], [qw(e["down"], device) for e in ex], w)
    got = run(hip, device, fn, np.full((M, H), np.nan, np.float32), x)
    got = got[0] if device else got
    tol = set_tol(oracle, parts, w)
    assert np.all(np.abs(got - ref) <= tol), (name, n, M, device, float(np.max(np.abs(got - ref) / tol)))


@pytest.mark.parametrize("name,down", [("q8_0", None), ("q4_k", None), ("mxfp4", None), ("q4_k", "q8_0")])
@pytest.mark.parametrize("n,M", [(1, 1), (8, 1), (16, 1), (17, 1), (32, 1), (3, 5), (17, 3), (32, 2)])
@pytest.mark.parametrize("device", [False, True])
def test_experts_swiglu_forward(hip, oracle, name, down, n, M, device):
    rng = np.random.default_rng(340 + n + M)
    H, I = 512, 256
    ex = experts(oracle, name, n, H, I, H, rng, gated=True, down_name=down)
    w = rng.uniform(0.05, 0.6, n).astype(np.float32)
    x = rng.standard_normal((M, H)).astype(np.float32)
    ref, parts = oracle.expert_set(x, ex, w)
    fn = lambda r, i: hip.MoEExpertsSwiGLUForward(r, i, [qw(e["gate"], device) for e in ex], [qw(e["up"], device) for e in ex],
                                                  [qw(e["down"], device) for e in ex], w)
    got = run(hip, device, fn, np.full((M, H), np.nan, np.float32), x)
    got = got[0] if device else got
    tol = set_tol(oracle, parts, w)
    assert np.all(np.abs(got - ref) <= tol), (name, n, M, device, float(np.max(np.abs(got - ref) / tol)))


def make_blocks(name, N, K, rng):
    """(type, raw bytes, N, K) of valid random blocks for the formats whose quantizer the oracle does not restate"""
    import torch
    from oracle.oracle import MORE_TYPES
    from tensorsharp_amd import synth
    if name == "q6_k":
        g = torch.Generator()
        g.manual_seed(int(rng.integers(1 << 30)))
        return (Q6_K, synth.quantize_q6_k_simple(torch.randn((N, K), generator=g) * 0.05).numpy().reshape(-1), N, K)
    return (MORE_TYPES[name], inputs.random_blocks(name, N, K, rng), N, K)


@pytest.mark.parametrize("name", ["q4_0", "q4_1", "q5_0", "q5_1", "iq4_nl", "q5_k", "q6_k"])
@pytest.mark.parametrize("n", [1, 6])
def test_experts_swiglu_single_row_other_gemv_formats(hip, oracle, name, n):
    # one row: the down projection of each expert is a GEMV that forms silu(gate) * up while it stages its activations,
    # compiled per format
    rng = np.random.default_rng(350 + n)
    H, I = 512, 256
    ex = [dict(gate=make_blocks(name, I, H, rng), up=make_blocks(name, I, H, rng), down=make_blocks(name, H, I, rng)) for _ in range(n)]
    w = rng.uniform(0.05, 0.6, n).astype(np.float32)
    x = rng.standard_normal((1, H)).astype(np.float32)
    ref, parts = oracle.expert_set(x, ex, w)
    fn = lambda r, i: hip.MoEExpertsSwiGLUForward(r, i, [qw(e["gate"], True) for e in ex], [qw(e["up"], True) for e in ex],
                                                  [qw(e["down"], True) for e in ex], w)
    got = run(hip, True, fn, np.full((1, H), np.nan, np.float32), x)[0]
    tol = set_tol(oracle, parts, w)
    assert np.all(np.abs(got - ref) <= tol), (name, n, float(np.max(np.abs(got - ref) / tol)))


@pytest.mark.parametrize("up,down,n,M", [("q4_k", "q4_k", 3, 40), ("mxfp4", "mxfp4", 5, 33), ("q8_0", "q8_0", 2, 170),
                                         ("q4_k", "q8_0", 2, 200), ("q8_0", "mxfp4", 6, 7), ("q5_1", "q6_k", 4, 36),
                                         ("mxfp4", "mxfp4", 2, 170)])
@pytest.mark.parametrize("gated", [True, False])
def test_expert_sets_of_many_rows_run_as_tile_table_launches(hip, oracle, up, down, n, M, gated):
    """More than one row with block-format weights: every linear of the set is one tile-table GEMM over the experts'
    pointers (32-row tiles up to 160 rows, then 128-row tiles; M = 40 / 170 / 200 need two tiles per expert, the last one
    partial).  A shared expert of another type in the same set (two launches for that linear) is covered by
    test_experts_swiglu_residual_with_shared_expert."""
    rng = np.random.default_rng(360 + n + M)
    H, I = 512, 256
    mk = lambda nm, N, K: make(oracle, nm, N, K, rng) if nm in T_ else make_blocks(nm, N, K, rng)
    ex = [dict(gate=mk(up, I, H) if gated else None, up=mk(up, I, H), down=mk(down, H, I)) for e in range(n)]
    w = rng.uniform(0.05, 0.6, n).astype(np.float32)
    x = rng.standard_normal((M, H)).astype(np.float32)
    ref, parts = oracle.expert_set(x, ex, w)
    if gated:
        fn = lambda r, i: hip.MoEExpertsSwiGLUForward(r, i, [qw(e["gate"], True) for e in ex], [qw(e["up"], True) for e in ex],
                                                      [qw(e["down"], True) for e in ex], w)
    else:
        fn = lambda r, i: hip.MoEExpertsForward(r, i, [qw(e["up"], True) for e in ex], [qw(e["down"], True) for e in ex], w)
    got = run(hip, True, fn, np.full((M, H), np.nan, np.float32), x)[0]
    tol = set_tol(oracle, parts, w)
    assert np.all(np.abs(got - ref) <= tol), (up, down, n, M, gated, float(np.max(np.abs(got - ref) / tol)))


@pytest.mark.parametrize("shared", [None, "same", "wider", "other_type"])
@pytest.mark.parametrize("n,M", [(8, 1), (32, 1), (4, 3)])
@pytest.mark.parametrize("device", [False, True])
def test_experts_swiglu_residual_with_shared_expert(hip, oracle, shared, n, M, device):
    rng = np.random.default_rng(350 + n + M)
    H, I = 512, 256
    ex = experts(oracle, "q4_k", n, H, I, H, rng, gated=True)
    w = rng.uniform(0.02, 0.3, n).astype(np.float32)
    x = rng.standard_normal((M, H)).astype(np.float32)
    resid = rng.standard_normal((M, H)).astype(np.float32)
    all_ex, all_w, sh = list(ex), list(w), None
    scalar = 0.37
    if shared is not None:
        si = 512 if shared == "wider" else I
        sname = "q8_0" if shared == "other_type" else "q4_k"
        s = experts(oracle, sname, 1, H, si, H, rng, gated=True)[0]
        all_ex.append(s)
        all_w.append(scalar)
        sh = (qw(s["gate"], device), qw(s["up"], device), qw(s["down"], device))
    ref, parts = oracle.expert_set(x, all_ex, all_w, base=resid)
    fn = lambda r, i: hip.MoEExpertsSwiGLUResidual(r, i, [qw(e["gate"], device) for e in ex], [qw(e["up"], device) for e in ex],
                                                   [qw(e["down"], device) for e in ex], w, shared=sh, shared_scalar=scalar)
    got = run(hip, device, fn, resid.copy(), x)
    got = got[0] if device else got
    tol = set_tol(oracle, parts, all_w)
    assert np.all(np.abs(got - ref) <= tol), (shared, n, M, device, float(np.max(np.abs(got - ref) / tol)))


def test_expert_set_argument_errors(hip, oracle):
    rng = np.random.default_rng(360)
    H, I = 64, 64
    ex = experts(oracle, "q8_0", 1, H, I, H, rng, gated=True)
    x = np.zeros((1, H), np.float32)
    out = np.zeros((1, H), np.float32)
    g, u, d = qw(ex[0]["gate"], False), qw(ex[0]["up"], False), qw(ex[0]["down"], False)
    with pytest.raises(RuntimeError, match="num_experts must be 1..16"):
        hip.MoEExpertsForward(out, x, [u] * 17, [d] * 17, [0.1] * 17)
    # the gated forward takes up to 32 experts like the bridge (ggml_ops_fused.cpp:1795-1799); only the squared-ReLU form stops at 16
    with pytest.raises(RuntimeError, match="num_experts must be 1..32"):
        hip.MoEExpertsSwiGLUForward(out, x, [g] * 33, [u] * 33, [d] * 33, [0.1] * 33)
    with pytest.raises(RuntimeError, match="num_experts must be 1..32"):
        hip.MoEExpertsSwiGLUResidual(out, x, [g] * 33, [u] * 33, [d] * 33, [0.1] * 33)
    with pytest.raises(RuntimeError, match="weight shapes do not match"):
        hip.MoEExpertsSwiGLUForward(np.zeros((1, H + 32), np.float32), x, [g], [u], [d], [1.0])
    with pytest.raises(RuntimeError, match="shape mismatch"):
        hip.FusedOutProjFFN(np.zeros((2, H), np.float32), x, u, np.ones(H, np.float32), EPS, g, d, 32)
    hip.ClearHostBufferCache()


@pytest.mark.parametrize("slots", [1, 4])
@pytest.mark.parametrize("device", [False, True])
def test_mul_mat_id_f32_experts(hip, oracle, slots, device):
    import torch
    rng = np.random.default_rng(370 + slots)
    E, rows, K, T, k = 6, 130, 200, 5, 4
    w = (rng.standard_normal((E, rows, K)) * 0.1).astype(np.float32)
    x = rng.standard_normal((T, slots, K)).astype(np.float32)
    ids = rng.integers(0, E, (T, k)).astype(np.int32)
    ref = oracle.mul_mat_id(w, x, ids)
    if device:
        out = torch.full((T, k, rows), float("nan"), device="cuda")
        hip.MulMatId(out, torch.from_numpy(w).cuda(), torch.from_numpy(x).cuda(), torch.from_numpy(ids).cuda())
        torch.cuda.synchronize()
        got = out.cpu().numpy()
    else:
        got = np.full((T, k, rows), np.nan, np.float32)
        hip.MulMatId(got, w, x, ids)
        # F32 ids are truncated like the bridge's read_i32_values; a padded (strided) weight stack is packed on upload
        got_f = np.full((T, k, rows), np.nan, np.float32)
        wide = np.zeros((E, rows + 3, K + 5), np.float32)
        wide[:, :rows, :K] = w
        hip.MulMatId(got_f, wide[:, :rows, :K], x, ids.astype(np.float32) + 0.4)
        assert np.array_equal(got_f, got)
        with pytest.raises(RuntimeError, match="expert id out of range"):
            hip.MulMatId(got_f, w, x, np.full((T, k), E, np.int32))
        with pytest.raises(RuntimeError, match="share the inner dimension"):
            hip.MulMatId(got_f, w, x[:, :, :K - 8], ids)
    # fp32 accumulation of exact fp32 products
    assert np.all(np.abs(got - ref) <= 1e-5 * np.linalg.norm(ref, axis=2, keepdims=True))


def test_mul_mat_id_device_more_than_65535_pairs(hip, oracle):
    """The device form cuts (token, slot) pairs into launches like the host form: a prefill of 16 500 tokens x 4 slots."""
    import torch
    rng = np.random.default_rng(380)
    E, rows, K, T, k = 5, 12, 24, 16_500, 4
    assert T * k > 65535
    w = (rng.standard_normal((E, rows, K)) * 0.1).astype(np.float32)
    x = rng.standard_normal((T, 1, K)).astype(np.float32)
    ids = rng.integers(0, E, (T, k)).astype(np.int32)
    out = torch.full((T, k, rows), float("nan"), device="cuda")
    hip.MulMatId(out, torch.from_numpy(w).cuda(), torch.from_numpy(x).cuda(), torch.from_numpy(ids).cuda())
    torch.cuda.synchronize()
    ref = np.einsum("tsrk,tk->tsr", w.astype(np.float64)[ids], x[:, 0].astype(np.float64))
    assert np.all(np.abs(out.cpu().numpy() - ref) <= 1e-5 * np.linalg.norm(ref, axis=2, keepdims=True))


def test_device_forms_refuse_strided_views(hip, oracle):
    """The device entry points index operands in place, so an input whose inner stride is not 1 and an output whose rows
    overlap are refused with the message of the plain device matmul (the host forms pack such views instead)."""
    import ctypes as C
    import torch
    from tensorsharp_amd import hip_native as N
    rng = np.random.default_rng(390)
    H, I, M = 64, 64, 3
    ex = experts(oracle, "q8_0", 1, H, I, H, rng, gated=True)[0]
    g, u, d = (qw(ex[n], True) for n in ("gate", "up", "down"))
    x = torch.zeros((M, 2 * H), device="cuda")
    out = torch.zeros((M, H), device="cuda")
    nw = torch.ones(H, device="cuda")
    strided_x = N.TensorView2D(x.data_ptr(), M, H, 2 * H, 2, x.numel() * 4)            # every second element
    good_x = N.TensorView2D(x.data_ptr(), M, H, 2 * H, 1, x.numel() * 4)
    good_out = N.TensorView2D(out.data_ptr(), M, H, H, 1, out.numel() * 4)
    overlap_out = N.TensorView2D(out.data_ptr(), M, H, H // 2, 1, out.numel() * 4)     # rows overlap
    lib = N.lib()
    wa = lambda q: (C.c_void_p(q.ptr), q.ggml_type, q.ne0, q.ne1, q.raw_bytes)
    ptrs = lambda q: (C.c_void_p * 1)(q.ptr)
    rw = (C.c_float * 1)(1.0)
    shape = lambda q: (q.ggml_type, q.ne0, q.ne1, q.raw_bytes)
    nwp = C.c_void_p(nw.data_ptr())
    calls = {
        "AddmmQuant": lambda o, i: lib.TSHip_AddmmQuantF32Device(o, i, *wa(u)),
        "FusedRmsNormMatMul": lambda o, i: lib.TSHip_FusedRmsNormMatMulQuantF32Device(o, i, nwp, H, 1e-6, *wa(u)),
        "FusedMatMulAdd": lambda o, i: lib.TSHip_FusedMatMulQuantAddF32Device(o, i, *wa(u)),
        "MoEExpertsForward": lambda o, i: lib.TSHip_MoEExpertsForwardF32Device(o, i, 1, ptrs(u), ptrs(d), *shape(u), *shape(d), rw),
        "MoEExpertsSwiGLUForward": lambda o, i: lib.TSHip_MoEExpertsSwiGLUForwardF32Device(o, i, 1, ptrs(g), ptrs(u), ptrs(d), *shape(g),
                                                                                     *shape(u), *shape(d), rw),
    }
    for name, call in calls.items():
        for o, i in ((good_out, strided_x), (overlap_out, good_x)):
            assert call(o, i) == 0, name
            assert "stride1 == 1" in N.get_last_error(), (name, N.get_last_error())
        assert call(good_out, good_x) == 1, (name, N.get_last_error())
    torch.cuda.synchronize()


@pytest.mark.parametrize("device", [False, True])
def test_add_id_bias_rows_by_expert(hip, oracle, device):
    """TSHip_AddIdF32: result[t, s, :] = src[t, s, :] + bias[ids[t, s], :], bit-equal to the definition (one fp32 add)."""
    import torch
    from oracle.oracle import add_id
    rng = np.random.default_rng(395)
    T, cols, rows, E = 7, 4, 300, 9
    src = rng.standard_normal((T, cols, rows)).astype(np.float32)
    bias = rng.standard_normal((E, rows)).astype(np.float32)
    ids = rng.integers(0, E, (T, cols)).astype(np.int32)
    want = add_id(src, bias, ids)
    if device:
        s = torch.from_numpy(src).cuda()
        out = torch.full_like(s, float("nan"))
        hip.AddId(out, s, torch.from_numpy(bias).cuda(), torch.from_numpy(ids).cuda())
        hip.AddId(s, s, torch.from_numpy(bias).cuda(), torch.from_numpy(ids).cuda())       # in place
        torch.cuda.synchronize()
        assert np.array_equal(out.cpu().numpy().view(np.uint32), want.view(np.uint32))
        assert np.array_equal(s.cpu().numpy().view(np.uint32), want.view(np.uint32))
    else:
        out = np.full_like(src, np.nan)
        hip.AddId(out, src, bias, ids)
        assert np.array_equal(out.view(np.uint32), want.view(np.uint32))
        # F32 ids are truncated like the bridge's read_i32_values; padded (strided) views are packed
        wide = np.zeros((T, cols + 1, rows + 5), np.float32)
        wide[:, :cols, :rows] = src
        out2 = np.full_like(src, np.nan)
        hip.AddId(out2, wide[:, :cols, :rows], bias, ids.astype(np.float32) + 0.3)
        assert np.array_equal(out2.view(np.uint32), want.view(np.uint32))
        with pytest.raises(RuntimeError, match="expert id out of range"):
            hip.AddId(out2, src, bias, np.full((T, cols), E, np.int32))
        with pytest.raises(RuntimeError, match="same shape"):
            hip.AddId(out2[:, :, :rows - 4], src, bias, ids)
        with pytest.raises(RuntimeError, match="bias shape"):
            hip.AddId(out2, src, bias[:, :rows - 4], ids)
