"""GPU parity: the bridge's fused wrappers around the quantized matmul (ggml_ops_fused.cpp:21-640) through the
C ABI, host-pointer and device forms, decode (GEMV) and prefill (GEMM) row counts.

Reference value: oracle RMSNorm / SiLU restatements (fp32, ggml order) around the fp64 product with the bit-exact
dequantized weights.  Bar: max_j |y - ref| <= 1e-3 * ||matmul part of the row||_2 (the residual that is added
is exact and must not loosen the bound)."""
import numpy as np
import pytest

from oracle.oracle import Q8_0, Q4_K, MXFP4

pytestmark = pytest.mark.gpu
T_ = {"q8_0": Q8_0, "q4_k": Q4_K, "mxfp4": MXFP4}
EPS = 1e-6


def make(oracle, name, N, K, rng, sigma=0.03):
    return oracle.quantize(T_[name], (rng.standard_normal(N * K) * sigma).astype(np.float32))


def bound_ok(got, ref, mm):
    tol = 1e-3 * np.linalg.norm(mm.astype(np.float64), axis=1, keepdims=True)
    return np.all(np.abs(got.astype(np.float64) - ref) <= tol + 1e-30), float(np.max(np.abs(got - ref) / (tol + 1e-30)))


def qweights(name, arrs, device):
    import torch
    from tensorsharp_amd import QuantizedWeight
    out = []
    for wq, K, N in arrs:
        out.append(QuantizedWeight(torch.from_numpy(wq).cuda() if device else wq, T_[name], K, N))
    return out


@pytest.mark.parametrize("name", ["q8_0", "q4_k", "mxfp4"])
@pytest.mark.parametrize("M", [1, 3, 9, 40])
@pytest.mark.parametrize("device", [False, True])
def test_rms_norm_matmul(hip, oracle, name, M, device):
    import torch
    rng = np.random.default_rng(91 + M)
    N, K = 384, 1024
    wq = make(oracle, name, N, K, rng)
    x = (rng.standard_normal((M, K)) * 3).astype(np.float32)
    nw = rng.uniform(0.5, 1.5, K).astype(np.float32)
    xn = oracle.rms_norm_mul(x, nw, EPS)
    ref = oracle.matmul_f64(T_[name], wq, N, K, xn)
    (qw,) = qweights(name, [(wq, K, N)], device)
    if device:
        res = torch.empty((M, N), device="cuda")
        hip.FusedRmsNormMatMulQuant(res, torch.from_numpy(x).cuda(), torch.from_numpy(nw).cuda(), EPS, qw)
        torch.cuda.synchronize()
        got = res.cpu().numpy()
    else:
        got = np.full((M, N), np.nan, dtype=np.float32)
        hip.FusedRmsNormMatMulQuant(got, x, nw, EPS, qw)
        hip.ClearHostBufferCache()
    ok, worst = bound_ok(got, ref, ref)
    assert ok, (name, M, device, worst)


@pytest.mark.parametrize("name", ["q4_0", "q4_1", "q5_0", "q5_1", "iq4_nl", "q5_k", "q6_k"])
@pytest.mark.parametrize("M", [1, 3])
def test_rms_norm_matmul_decode_every_other_gemv_format(hip, oracle, name, M):
    # one launch per row with RMSNorm(x) * w formed while the activations are staged: each block format stages them in
    # its own unpack order (random valid blocks; the three headline formats are covered above)
    import torch
    from oracle.oracle import MORE_TYPES
    from tensorsharp_amd import QuantizedWeight, synth
    t = MORE_TYPES[name]
    rng = np.random.default_rng(17 + M)
    N, K = 392, 1024
    w = synth.random_weight(t, N, K, torch.device("cuda"), seed=31, sigma=0.03)
    x = (rng.standard_normal((M, K)) * 3).astype(np.float32)
    nw = rng.uniform(0.5, 1.5, K).astype(np.float32)
    ref = oracle.matmul_f64(t, w.cpu().numpy(), N, K, oracle.rms_norm_mul(x, nw, EPS))
    res = torch.empty((M, N), device="cuda")
    hip.FusedRmsNormMatMulQuant(res, torch.from_numpy(x).cuda(), torch.from_numpy(nw).cuda(), EPS, QuantizedWeight(w, t, K, N))
    torch.cuda.synchronize()
    ok, worst = bound_ok(res.cpu().numpy(), ref, ref)
    assert ok, (name, M, worst)


@pytest.mark.parametrize("name", ["q8_0", "q4_k", "mxfp4"])
@pytest.mark.parametrize("M", [1, 2, 70, 300])
@pytest.mark.parametrize("device", [False, True])
def test_matmul_add_in_place(hip, oracle, name, M, device):
    import torch
    rng = np.random.default_rng(93 + M)
    N, K = 320, 768
    wq = make(oracle, name, N, K, rng)
    x = rng.standard_normal((M, K)).astype(np.float32)
    resid = (rng.standard_normal((M, N)) * 5).astype(np.float32)
    mm = oracle.matmul_f64(T_[name], wq, N, K, x)
    ref = resid.astype(np.float64) + mm
    (qw,) = qweights(name, [(wq, K, N)], device)
    if device:
        r = torch.from_numpy(resid.copy()).cuda()
        hip.FusedMatMulQuantAdd(r, torch.from_numpy(x).cuda(), qw)
        torch.cuda.synchronize()
        got = r.cpu().numpy()
    else:
        got = resid.copy()
        hip.FusedMatMulQuantAdd(got, x, qw)
        hip.ClearHostBufferCache()
    ok, worst = bound_ok(got, ref, mm)
    assert ok, (name, M, device, worst)


@pytest.mark.parametrize("name", ["q8_0", "q4_k", "mxfp4"])
@pytest.mark.parametrize("M", [1, 3, 9, 48])
@pytest.mark.parametrize("device", [False, True])
def test_ffn_swiglu(hip, oracle, name, M, device):
    import torch
    rng = np.random.default_rng(95 + M)
    H, F = 512, 768
    gu = make(oracle, name, 2 * F, H, rng, 0.05)
    dn = make(oracle, name, H, F, rng, 0.05)
    x = (rng.standard_normal((M, H)) * 2).astype(np.float32)
    resid = rng.standard_normal((M, H)).astype(np.float32)
    nw = rng.uniform(0.5, 1.5, H).astype(np.float32)
    xn = oracle.rms_norm_mul(x, nw, EPS)
    g = oracle.matmul_f64(T_[name], gu, 2 * F, H, xn).astype(np.float32)
    act = oracle.silu_mul(g)
    mm = oracle.matmul_f64(T_[name], dn, H, F, act)
    ref = resid.astype(np.float64) + mm
    qgu, qdn = qweights(name, [(gu, H, 2 * F), (dn, F, H)], device)
    if device:
        r = torch.from_numpy(resid.copy()).cuda()
        hip.FusedFFNSwiGLUQuant(r, torch.from_numpy(x).cuda(), torch.from_numpy(nw).cuda(), EPS, qgu, qdn, F)
        torch.cuda.synchronize()
        got = r.cpu().numpy()
    else:
        got = resid.copy()
        hip.FusedFFNSwiGLUQuant(got, x, nw, EPS, qgu, qdn, F)
        hip.ClearHostBufferCache()
    # two chained fp16-operand matmuls: the first one's error passes through SiLU and the second matmul
    tol = 2e-3 * np.linalg.norm(mm, axis=1, keepdims=True)
    assert np.all(np.abs(got - ref) <= tol), (name, M, device, float(np.max(np.abs(got - ref) / tol)))


def test_fused_argument_errors(hip, oracle):
    from tensorsharp_amd import QuantizedWeight
    rng = np.random.default_rng(97)
    wq = make(oracle, "q8_0", 64, 128, rng)
    qw = QuantizedWeight(wq, Q8_0, 128, 64)
    x = np.zeros((2, 128), np.float32)
    with pytest.raises(RuntimeError, match="Size mismatch"):
        hip.FusedMatMulQuantAdd(np.zeros((3, 64), np.float32), x, qw)
    with pytest.raises(RuntimeError, match="Size mismatch"):
        hip.FusedRmsNormMatMulQuant(np.zeros((2, 64), np.float32), x, np.ones(100, np.float32), EPS, qw)
    with pytest.raises(RuntimeError, match="gate_up.ne1 != 2\\*half_dim"):
        hip.FusedFFNSwiGLUQuant(np.zeros((2, 128), np.float32), x, np.ones(128, np.float32), EPS, qw, qw, 48)
    hip.ClearHostBufferCache()


@pytest.mark.parametrize("name", ["q4_k", "q8_0"])
def test_rms_norm_matmul_row_longer_than_one_staging_pass(hip, oracle, name):
    # K above what the decode kernel stages in one pass: RMSNorm runs as a kernel of its own
    import torch
    rng = np.random.default_rng(99)
    N, K, M = 64, 16384 + 512, 2
    wq = make(oracle, name, N, K, rng)
    x = rng.standard_normal((M, K)).astype(np.float32)
    nw = rng.uniform(0.5, 1.5, K).astype(np.float32)
    ref = oracle.matmul_f64(T_[name], wq, N, K, oracle.rms_norm_mul(x, nw, EPS))
    (qw,) = qweights(name, [(wq, K, N)], True)
    res = torch.empty((M, N), device="cuda")
    hip.FusedRmsNormMatMulQuant(res, torch.from_numpy(x).cuda(), torch.from_numpy(nw).cuda(), EPS, qw)
    torch.cuda.synchronize()
    ok, worst = bound_ok(res.cpu().numpy(), ref, ref)
    assert ok, (name, worst)


@pytest.mark.parametrize("M", [1, 40])
def test_ffn_swiglu_q4_k_gate_up_q6_k_down(hip, oracle, M):
    # the mix of a Q4_K_M file: gate/up in Q4_K, down in Q6_K (its GEMV at M = 1 with silu(gate) * up formed in the staging)
    import torch
    from oracle.oracle import Q6_K
    from tensorsharp_amd import QuantizedWeight, synth
    rng = np.random.default_rng(97 + M)
    H, F = 512, 768
    gu = make(oracle, "q4_k", 2 * F, H, rng, 0.05)
    g = torch.Generator()
    g.manual_seed(9)
    dn = synth.quantize_q6_k_simple(torch.randn((H, F), generator=g) * 0.05).numpy()
    x = (rng.standard_normal((M, H)) * 2).astype(np.float32)
    resid = rng.standard_normal((M, H)).astype(np.float32)
    nw = rng.uniform(0.5, 1.5, H).astype(np.float32)
    xn = oracle.rms_norm_mul(x, nw, EPS)
    act = oracle.silu_mul(oracle.matmul_f64(Q4_K, gu, 2 * F, H, xn).astype(np.float32))
    mm = oracle.matmul_f64(Q6_K, dn, H, F, act)
    ref = resid.astype(np.float64) + mm
    r = torch.from_numpy(resid.copy()).cuda()
    hip.FusedFFNSwiGLUQuant(r, torch.from_numpy(x).cuda(), torch.from_numpy(nw).cuda(), EPS,
                            QuantizedWeight(torch.from_numpy(gu).cuda(), Q4_K, H, 2 * F),
                            QuantizedWeight(torch.from_numpy(dn).cuda(), Q6_K, F, H), F)
    torch.cuda.synchronize()
    tol = 2e-3 * np.linalg.norm(mm, axis=1, keepdims=True)
    got = r.cpu().numpy()
    assert np.all(np.abs(got - ref) <= tol), (M, float(np.max(np.abs(got - ref) / tol)))


@pytest.mark.parametrize("adjacent", [True, False])
def test_gate_up_fused_at_load_feeds_the_ffn(hip, oracle, adjacent):
    # ModelBase.FuseGateUpWeights (ModelBase.cs:768-802): gate and up become one [2F x H] weight - a view when the two
    # tensors are adjacent in the mapping, a copy otherwise - and the fused FFN on it equals the FFN of the two halves
    from tensorsharp_amd import QuantizedWeight, FuseGateUpWeights
    rng = np.random.default_rng(101)
    H, F, M = 512, 768, 3
    gate = make(oracle, "q4_k", F, H, rng, 0.05)
    up = make(oracle, "q4_k", F, H, rng, 0.05)
    dn = make(oracle, "q4_k", H, F, rng, 0.05)
    owner = object()
    mapping = np.concatenate([gate, np.zeros(0 if adjacent else 144, np.uint8), up])
    weights = {"blk.0.ffn_gate.weight": QuantizedWeight.CreateExternalView(mapping[:gate.size], Q4_K, H, F, owner),
               "blk.0.ffn_up.weight": QuantizedWeight.CreateExternalView(mapping[mapping.size - up.size:], Q4_K, H, F, owner)}
    assert FuseGateUpWeights(weights, 1) == 1
    gu = weights["blk.0.ffn_gate_up.weight"]
    assert (gu.ptr == mapping.ctypes.data) == adjacent and gu.ne1 == 2 * F
    x = (rng.standard_normal((M, H)) * 2).astype(np.float32)
    resid = rng.standard_normal((M, H)).astype(np.float32)
    nw = rng.uniform(0.5, 1.5, H).astype(np.float32)
    xn = oracle.rms_norm_mul(x, nw, EPS)
    g = oracle.matmul_f64(Q4_K, gate, F, H, xn).astype(np.float32)
    u = oracle.matmul_f64(Q4_K, up, F, H, xn).astype(np.float32)
    mm = oracle.matmul_f64(Q4_K, dn, H, F, oracle.silu_mul(np.concatenate([g, u], axis=1)))
    got = resid.copy()
    hip.FusedFFNSwiGLUQuant(got, x, nw, EPS, gu, QuantizedWeight(dn, Q4_K, F, H), F)
    hip.ClearHostBufferCache()
    tol = 2e-3 * np.linalg.norm(mm, axis=1, keepdims=True)
    assert np.all(np.abs(got - (resid + mm)) <= tol)


@pytest.mark.parametrize("gu_type", ["q4_0", "q4_1", "q5_0", "q5_1", "iq4_nl", "q5_k", "q6_k", "q8_0", "mxfp4"])
@pytest.mark.parametrize("M", [1, 2])
def test_ffn_decode_paired_store_every_gemv_format(hip, oracle, gu_type, M):
    # decode FFN: the gate_up launch computes gate row j and up row j in one wavefront (rows F apart in the stacked
    # weight) and stores silu(gate) * up; every format with a GEMV kernel has its own row-group geometry
    # (2 rows x 32 lanes or 4 rows x 16 lanes), so each is run once, with a Q8_0 down projection
    import torch
    from oracle.oracle import Q4_0, Q4_1, Q5_K, Q6_K, MORE_TYPES
    from tensorsharp_amd import QuantizedWeight, synth
    types = {"q4_0": Q4_0, "q4_1": Q4_1, "q5_k": Q5_K, "q6_k": Q6_K, "q8_0": Q8_0, "mxfp4": MXFP4}
    t = types.get(gu_type) or MORE_TYPES[gu_type]
    rng = np.random.default_rng(103 + M)
    H, F = 512, 1024 if t in (Q5_K, Q6_K) else 1056      # 1056 = 33 blocks: an odd number of row groups
    dev = torch.device("cuda")
    gu_d = synth.random_weight(t, 2 * F, H, dev, seed=11, sigma=0.05)
    gu = gu_d.cpu().numpy()
    dn = make(oracle, "q8_0", H, F, rng, 0.05)
    x = (rng.standard_normal((M, H)) * 2).astype(np.float32)
    resid = rng.standard_normal((M, H)).astype(np.float32)
    nw = rng.uniform(0.5, 1.5, H).astype(np.float32)
    xn = oracle.rms_norm_mul(x, nw, EPS)
    act = oracle.silu_mul(oracle.matmul_f64(t, gu, 2 * F, H, xn).astype(np.float32))
    mm = oracle.matmul_f64(Q8_0, dn, H, F, act)
    r = torch.from_numpy(resid.copy()).cuda()
    hip.FusedFFNSwiGLUQuant(r, torch.from_numpy(x).cuda(), torch.from_numpy(nw).cuda(), EPS, QuantizedWeight(gu_d, t, H, 2 * F),
                            QuantizedWeight(torch.from_numpy(dn).cuda(), Q8_0, F, H), F)
    torch.cuda.synchronize()
    tol = 2e-3 * np.linalg.norm(mm, axis=1, keepdims=True)
    assert np.all(np.abs(r.cpu().numpy() - (resid + mm)) <= tol), (gu_type, M)
