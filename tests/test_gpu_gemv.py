"""GPU parity: decode GEMV through the C ABI against the oracle.

Bar: max_j |y[m,j] - ref[m,j]| / ||ref[m,:]||_2 <= 1e-3 per output row, ref = fp64 product of the
bit-exact dequantised weights with the fp32 activations.  The stricter max|delta|/rms(ref row)
is asserted too, at 1e-4 for the fp32 Q8_0 path and 5e-3 for the fp16-activation 4-bit paths.
"""
import numpy as np
import pytest

import inputs
from oracle.oracle import Q8_0, Q4_K, MXFP4

pytestmark = pytest.mark.gpu
T = {"q8_0": Q8_0, "q4_k": Q4_K, "mxfp4": MXFP4}
RMS_TOL = {"q8_0": 1e-4, "q4_k": 5e-3, "mxfp4": 5e-3}


def check(name, y, ref):
    e1, e2 = inputs.row_l2_err(y, ref), inputs.rms_err(y, ref)
    assert e1 <= 1e-3, (name, e1)
    assert e2 <= RMS_TOL[name], (name, e2)
    return e1, e2


def run_device(hip, t, wq, N, K, x):
    import torch
    from tensorsharp_amd import QuantizedWeight
    qw = QuantizedWeight(torch.from_numpy(wq).cuda(), t, K, N)
    y = hip.LinearForward(torch.from_numpy(x).cuda(), qw)
    torch.cuda.synchronize()
    return y.cpu().numpy()


@pytest.mark.parametrize("cfg,tname", [("CFG1", "ffn_up"), ("CFG2", "wq"), ("CFG2", "wk"), ("CFG2", "gate"),
                                        ("CFG2", "down"), ("CFG4", "gate_up"), ("CFG4", "down")])
def test_baseline_shapes(hip, oracle, cfg, tname):
    fmt, N, K = getattr(inputs, cfg)[tname]
    tag = f"{cfg.lower()}.{tname}"
    wq = oracle.quantize(T[fmt], inputs.weights(tag, N * K))
    x = inputs.activations(tag, 1, K)
    ref = oracle.matmul_f64(T[fmt], wq, N, K, x)
    y = run_device(hip, T[fmt], wq, N, K, x)
    e = check(fmt, y, ref)
    print(tag, "row-L2 err %.2e rms err %.2e" % e)


@pytest.mark.parametrize("name", ["q8_0", "q4_k", "mxfp4"])
@pytest.mark.parametrize("N,K", [(1, 256), (3, 512), (5, 768), (7, 1024), (130, 2560), (257, 4096), (1001, 2816)])
def test_ragged_shapes(hip, oracle, name, N, K):
    if name == "q4_k" and K % 256:
        pytest.skip("K must be a multiple of 256 for Q4_K")
    rng = np.random.default_rng(N * 7919 + K)
    wq = oracle.quantize(T[name], (rng.standard_normal(N * K) * 0.02).astype(np.float32))
    x = rng.standard_normal((1, K)).astype(np.float32)
    check(name, run_device(hip, T[name], wq, N, K, x), oracle.matmul_f64(T[name], wq, N, K, x))


@pytest.mark.parametrize("name", ["q8_0", "q4_k", "mxfp4"])
def test_activation_ranges_and_linearity(hip, oracle, name):
    rng = np.random.default_rng(31)
    N, K = 300, 2048
    wq = oracle.quantize(T[name], (rng.standard_normal(N * K) * 0.02).astype(np.float32))
    x = rng.standard_normal((1, K)).astype(np.float32)
    base = run_device(hip, T[name], wq, N, K, x)
    for s in (1e-20, 1e-6, 3e4, 1e12):       # outside fp16 range both ways: handled by the power-of-two pre-scale
        xs = (x * np.float32(s)).astype(np.float32)
        y = run_device(hip, T[name], wq, N, K, xs)
        check(name, y, oracle.matmul_f64(T[name], wq, N, K, xs))
    two = run_device(hip, T[name], wq, N, K, (2 * x).astype(np.float32))
    assert np.array_equal(two, 2 * base)      # scaling by a power of two is exact
    zero = run_device(hip, T[name], wq, N, K, np.zeros((1, K), np.float32))
    assert np.all(zero == 0)
    # sparse activations with one large outlier
    xo = np.zeros((1, K), np.float32)
    xo[0, 17], xo[0, K - 1] = 1000.0, -0.001
    check(name, run_device(hip, T[name], wq, N, K, xo), oracle.matmul_f64(T[name], wq, N, K, xo))


@pytest.mark.parametrize("name", ["q8_0", "mxfp4"])
def test_unaligned_sub_weight_views(hip, oracle, name):
    """Expert-style views: a weight that starts at an arbitrary block offset inside a bigger
    allocation (17-byte and 34-byte blocks land on every byte / 2-byte alignment)."""
    import torch
    from tensorsharp_amd import QuantizedWeight
    rng = np.random.default_rng(33)
    N, K = 64, 1120                              # 35 blocks per row: odd row stride
    rows_before = (1, 2, 3)
    total = max(rows_before) + N
    wq = oracle.quantize(T[name], (rng.standard_normal(total * K) * 0.02).astype(np.float32))
    dev = torch.from_numpy(wq).cuda()
    rs = oracle.row_size(T[name], K)
    x = rng.standard_normal((1, K)).astype(np.float32)
    xd = torch.from_numpy(x).cuda()
    for rb in rows_before:
        view = dev[rb * rs: (rb + N) * rs]
        y = hip.LinearForward(xd, QuantizedWeight(view, T[name], K, N))
        torch.cuda.synchronize()
        ref = oracle.matmul_f64(T[name], wq[rb * rs:(rb + N) * rs], N, K, x)
        check(name, y.cpu().numpy(), ref)


def host_case_weight(oracle, name, N, K, rng):
    """(ggml type, raw blocks) of a random weight in any format with a GEMV kernel."""
    from oracle.oracle import Q6_K, MORE_TYPES
    if name in T:
        return T[name], oracle.quantize(T[name], (rng.standard_normal(N * K) * 0.02).astype(np.float32))
    if name == "q6_k":
        return Q6_K, q6k_weight(N, K, 35)
    return MORE_TYPES[name], inputs.random_blocks(name, N, K, rng)


@pytest.mark.parametrize("name", ["q8_0", "q4_k", "mxfp4", "q6_k", "q5_k", "q4_0", "q4_1", "q5_0", "q5_1", "iq4_nl"])
def test_host_entry_points(hip, oracle, name):
    """Drop-in path: host pointers, strided activation view, preload key, batch form."""
    rng = np.random.default_rng(35)
    N, K, M = 96, 1024, 3
    t, wq = host_case_weight(oracle, name, N, K, rng)
    T_ = dict(T)
    T_[name] = t
    big = rng.standard_normal((M, K + 40)).astype(np.float32)
    x = big[:, 8:8 + K]                               # row stride K+40, stride1 == 1
    ref = oracle.matmul_f64(T_[name], wq, N, K, np.ascontiguousarray(x))
    out = np.full((M, N + 5), np.nan, dtype=np.float32)
    res = out[:, :N]                                  # strided result view
    hip.AddmmQuant(res, x, wq.ctypes.data, T_[name], K, N, wq.size)
    check(name if name in RMS_TOL else "q4_k", res, ref)
    assert np.all(np.isnan(out[:, N:]))               # nothing outside the view was written
    # column-strided activations are packed by the shim
    xt = np.asfortranarray(np.ascontiguousarray(x))
    res2 = np.empty((M, N), dtype=np.float32)
    hip.AddmmQuant(res2, xt, wq.ctypes.data, T_[name], K, N, wq.size)
    assert np.array_equal(res2, res)
    # preload under an opaque key, then drop the host bytes
    key = 0x7000_0000_1234
    scratch = wq.copy()
    hip.PreloadQuantizedWeight(key, scratch.ctypes.data, T_[name], K, N, scratch.size)
    scratch[:] = 0
    res3 = np.empty((M, N), dtype=np.float32)
    hip.AddmmQuant(res3, np.ascontiguousarray(x), key, T_[name], K, N, wq.size)
    assert np.array_equal(res3, res)
    hip.InvalidateHostBuffer(key)
    # batch form == per-row single calls on sub-weights
    rs = oracle.row_size(T_[name], K)
    n_sub = N // 3
    offs = [0, n_sub * rs, 2 * n_sub * rs]
    resb = np.empty((M, n_sub), dtype=np.float32)
    hip.AddmmQuantBatch(resb, np.ascontiguousarray(x), wq.ctypes.data, T_[name], K, wq.size, offs, [n_sub] * 3)
    for b in range(3):
        assert np.array_equal(resb[b], res[b, b * n_sub:(b + 1) * n_sub])
    hip.ClearHostBufferCache()


def test_error_paths(hip, oracle):
    """The failures the bridge reports (ggml_ops_matmul.cpp:303-329) come back as 0 + message."""
    from tensorsharp_amd import hip_native as N
    rng = np.random.default_rng(37)
    Nn, K = 8, 256
    wq = oracle.quantize(Q4_K, (rng.standard_normal(Nn * K) * 0.02).astype(np.float32))
    x = np.zeros((2, K), np.float32)
    y = np.zeros((2, Nn), np.float32)

    def call(result, m1, w, t, ne0, ne1, rb):
        with pytest.raises(RuntimeError) as ei:
            hip.AddmmQuant(result, m1, w, t, ne0, ne1, rb)
        return str(ei.value)

    assert "Invalid quantized weight descriptor" in call(y, x, 0, Q4_K, K, Nn, wq.size)
    assert "m1.dim0 != result.dim0" in call(y[:1], x, wq.ctypes.data, Q4_K, K, Nn, wq.size)
    assert "quantized weight dims don't match" in call(y, x, wq.ctypes.data, Q4_K, K, Nn + 1, wq.size)
    assert "quantized weight dims don't match" in call(y, x[:, :128], wq.ctypes.data, Q4_K, K, Nn, wq.size)
    assert "Unsupported weight type" in call(y, x, wq.ctypes.data, 10, K, Nn, wq.size)      # Q2_K
    assert "too small" in call(y, x, wq.ctypes.data, Q4_K, K, Nn, wq.size - 144)
    x32 = np.zeros((2, 32), np.float32)
    assert "multiple of the block size" in call(y, x32, wq.ctypes.data, Q4_K, 32, Nn, wq.size)
    # a failed call leaves the message readable until the next call on this thread, success clears it
    hip.AddmmQuant(y, x, wq.ctypes.data, Q4_K, K, Nn, wq.size)
    assert N.get_last_error() == ""
    hip.ClearHostBufferCache()


@pytest.mark.parametrize("name", ["q8_0", "q4_k", "mxfp4"])
def test_grouped_launch_equals_single_launches(hip, oracle, name):
    """TSHip_AddmmQuantGroupF32Device: several independent decode GEMVs in one launch."""
    import torch
    from tensorsharp_amd import QuantizedWeight
    rng = np.random.default_rng(41)
    shapes = [(96, 1024), (33, 2048), (700, 512), (1, 256), (260, 3072), (64, 1024), (17, 768)]
    if name == "q4_k":
        shapes = [(n, k) for n, k in shapes if k % 256 == 0]
    ws, xs, ys, refs = [], [], [], []
    for n, k in shapes:
        wq = oracle.quantize(T[name], (rng.standard_normal(n * k) * 0.02).astype(np.float32))
        x = rng.standard_normal((1, k)).astype(np.float32)
        refs.append(oracle.matmul_f64(T[name], wq, n, k, x))
        ws.append(QuantizedWeight(torch.from_numpy(wq).cuda(), T[name], k, n))
        xs.append(torch.from_numpy(x).cuda())
        ys.append(torch.full((1, n), float("nan"), device="cuda"))
    hip.UseCurrentStream()
    pack = hip.PrepareGroup(ys, xs, ws)
    hip.AddmmQuantGroupDevice(pack)
    torch.cuda.synchronize()
    for y, ref, w, x in zip(ys, refs, ws, xs):
        check(name, y.cpu().numpy(), ref)
        single = hip.LinearForward(x, w)
        torch.cuda.synchronize()
        assert inputs.row_l2_err(y.cpu().numpy(), single.cpu().numpy()) < 1e-5


def test_grouped_full_layer(hip, oracle):
    """configs[1] at full size: the seven Q4_K projections of one layer in one launch."""
    import torch
    from tensorsharp_amd import QuantizedWeight
    ws, xs, ys, refs = [], [], [], []
    for tname, (fmt, n, k) in inputs.CFG2.items():
        tag = f"cfg2.{tname}"
        wq = oracle.quantize(T[fmt], inputs.weights(tag, n * k))
        x = inputs.activations(tag, 1, k)
        refs.append(oracle.matmul_f64(T[fmt], wq, n, k, x))
        ws.append(QuantizedWeight(torch.from_numpy(wq).cuda(), T[fmt], k, n))
        xs.append(torch.from_numpy(x).cuda())
        ys.append(torch.empty((1, n), device="cuda"))
    hip.UseCurrentStream()
    hip.AddmmQuantGroupDevice(hip.PrepareGroup(ys, xs, ws))
    torch.cuda.synchronize()
    for y, ref in zip(ys, refs):
        check("q4_k", y.cpu().numpy(), ref)


@pytest.mark.parametrize("name,N,K", [("q4_k", 1001, 14336), ("q8_0", 515, 8192 + 32), ("mxfp4", 2880, 5760), ("q4_k", 6, 8192),
                                      ("q8_0", 4096, 4096 + 64)])
def test_few_rows_long_k_split_over_wavefronts(hip, oracle, name, N, K):
    # few rows, long K: four wavefronts share a row group and each takes a quarter of its steps; also as y = add + W x
    import torch
    from tensorsharp_amd import QuantizedWeight
    rng = np.random.default_rng(N + K)
    wq = oracle.quantize(T[name], (rng.standard_normal(N * K) * 0.02).astype(np.float32))
    x = rng.standard_normal((1, K)).astype(np.float32)
    ref = oracle.matmul_f64(T[name], wq, N, K, x)
    check(name, run_device(hip, T[name], wq, N, K, x), ref)
    resid = rng.standard_normal((1, N)).astype(np.float32)
    r = torch.from_numpy(resid.copy()).cuda()
    hip.FusedMatMulQuantAdd(r, torch.from_numpy(x).cuda(), QuantizedWeight(torch.from_numpy(wq).cuda(), T[name], K, N))
    torch.cuda.synchronize()
    got = r.cpu().numpy().astype(np.float64) - resid
    assert np.max(np.abs(got - ref)) <= 1e-3 * np.linalg.norm(ref) + 1e-6 * np.max(np.abs(resid)), name


# ---- Q6_K (output matrix and some projections of Q4_K_M files): 210-byte blocks, 2-byte aligned ----
def q6k_weight(N, K, seed, std=0.02):
    import torch
    from tensorsharp_amd import synth
    g = torch.Generator().manual_seed(seed)
    return synth.quantize_q6_k_simple(torch.randn((N, K), generator=g) * std).numpy()


@pytest.mark.parametrize("N,K", [(1, 256), (3, 512), (7, 1024), (130, 2560), (257, 4096), (1001, 2816), (4096, 14336), (6, 8192)])
def test_q6_k_shapes(hip, oracle, N, K):
    from oracle.oracle import Q6_K
    wq = q6k_weight(N, K, N * 31 + K)
    rng = np.random.default_rng(N + K)
    x = rng.standard_normal((1, K)).astype(np.float32)
    ref = oracle.matmul_f64(Q6_K, wq, N, K, x)
    check("q4_k", run_device(hip, Q6_K, wq, N, K, x), ref)
    for s in (1e-20, 3e4):
        xs = (x * np.float32(s)).astype(np.float32)
        check("q4_k", run_device(hip, Q6_K, wq, N, K, xs), oracle.matmul_f64(Q6_K, wq, N, K, xs))
    assert np.all(run_device(hip, Q6_K, wq, N, K, np.zeros((1, K), np.float32)) == 0)


def test_q6_k_extreme_quants_and_scales(hip, oracle):
    # every 6-bit value and both signs of the int8 scales, in random order
    from oracle.oracle import Q6_K
    rng = np.random.default_rng(77)
    N, K = 64, 1024
    nb = N * K // 256
    raw = rng.integers(0, 256, size=(nb, 210), dtype=np.uint8)
    raw[:, 208:210] = rng.uniform(1e-4, 4e-4, nb).astype(np.float16).view(np.uint8).reshape(nb, 2)
    raw[0, 192:208] = np.array([-128, 127, -1, 1, 0, 64, -64, 5] * 2, dtype=np.int8).view(np.uint8)
    wq = raw.reshape(-1)
    x = rng.standard_normal((1, K)).astype(np.float32)
    check("q4_k", run_device(hip, Q6_K, wq, N, K, x), oracle.matmul_f64(Q6_K, wq, N, K, x))


def test_q6_k_views_two_bytes_off_and_grouped(hip, oracle):
    # a weight that starts one row into an allocation (105 blocks per row: rows alternate between byte 0 and byte 2 of
    # a dword), alone and as members of a grouped launch
    import torch
    from tensorsharp_amd import QuantizedWeight
    from oracle.oracle import Q6_K
    N, K = 48, 256 * 5
    wq = q6k_weight(N + 3, K, 5)
    rb = (K // 256) * 210
    dev = torch.from_numpy(wq).cuda()
    rng = np.random.default_rng(6)
    x = rng.standard_normal((1, K)).astype(np.float32)
    xd = torch.from_numpy(x).cuda()
    ws, ys, refs = [], [], []
    for skip in (1, 2, 3):
        view = dev[skip * rb:(skip + N) * rb]
        refs.append(oracle.matmul_f64(Q6_K, wq[skip * rb:(skip + N) * rb], N, K, x))
        ws.append(QuantizedWeight(view, Q6_K, K, N))
        y = hip.LinearForward(xd, ws[-1])
        torch.cuda.synchronize()
        check("q4_k", y.cpu().numpy(), refs[-1])
        ys.append(torch.full((1, N), float("nan"), device="cuda"))
    hip.UseCurrentStream()
    hip.AddmmQuantGroupDevice(hip.PrepareGroup(ys, [xd] * 3, ws))
    torch.cuda.synchronize()
    for y, ref in zip(ys, refs):
        check("q4_k", y.cpu().numpy(), ref)


# ---- Q5_K: Q4_K with a fifth bit per weight (176-byte blocks) ----
@pytest.mark.parametrize("N,K", [(1, 256), (5, 768), (130, 2560), (257, 4096), (4096, 14336), (6, 8192)])
def test_q5_k_shapes(hip, oracle, N, K):
    from oracle.oracle import Q5_K
    rng = np.random.default_rng(N * 13 + K)
    wq = inputs.random_blocks("q5_k", N, K, rng)
    x = rng.standard_normal((1, K)).astype(np.float32)
    check("q4_k", run_device(hip, Q5_K, wq, N, K, x), oracle.matmul_f64(Q5_K, wq, N, K, x))
    xs = (x * np.float32(1e-20)).astype(np.float32)
    check("q4_k", run_device(hip, Q5_K, wq, N, K, xs), oracle.matmul_f64(Q5_K, wq, N, K, xs))
    assert np.all(run_device(hip, Q5_K, wq, N, K, np.zeros((1, K), np.float32)) == 0)


# ---- Q4_0 / Q4_1 / Q5_0 / Q5_1 / IQ4_NL: 18- to 24-byte blocks of 32 weights ----
LEGACY = ["q4_0", "q4_1", "q5_0", "q5_1", "iq4_nl"]


@pytest.mark.parametrize("name", LEGACY)
@pytest.mark.parametrize("N,K", [(1, 32), (3, 96), (7, 1056), (130, 2560), (257, 4096), (1001, 2880), (4096, 14336)])
def test_q4_legacy_shapes(hip, oracle, name, N, K):
    from oracle.oracle import MORE_TYPES
    t = MORE_TYPES[name]
    rng = np.random.default_rng(N * 17 + K)
    wq = inputs.random_blocks(name, N, K, rng)
    x = rng.standard_normal((1, K)).astype(np.float32)
    check("q4_k", run_device(hip, t, wq, N, K, x), oracle.matmul_f64(t, wq, N, K, x))
    xs = (x * np.float32(3e4)).astype(np.float32)
    check("q4_k", run_device(hip, t, wq, N, K, xs), oracle.matmul_f64(t, wq, N, K, xs))
    assert np.all(run_device(hip, t, wq, N, K, np.zeros((1, K), np.float32)) == 0)


@pytest.mark.parametrize("name", LEGACY)
def test_q4_legacy_views_at_odd_rows(hip, oracle, name):
    # 35 blocks per row: rows of the 18- and 22-byte blocks alternate between byte 0 and byte 2 of a dword; views that
    # start rows into a tensor
    import torch
    from tensorsharp_amd import QuantizedWeight
    from oracle.oracle import MORE_TYPES
    t = MORE_TYPES[name]
    rng = np.random.default_rng(44)
    N, K = 64, 1120
    wq = inputs.random_blocks(name, N + 3, K, rng)
    rs = oracle.row_size(t, K)
    dev = torch.from_numpy(wq).cuda()
    x = rng.standard_normal((1, K)).astype(np.float32)
    xd = torch.from_numpy(x).cuda()
    for rb in (1, 2, 3):
        y = hip.LinearForward(xd, QuantizedWeight(dev[rb * rs:(rb + N) * rs], t, K, N))
        torch.cuda.synchronize()
        check("q4_k", y.cpu().numpy(), oracle.matmul_f64(t, wq[rb * rs:(rb + N) * rs], N, K, x))


@pytest.mark.parametrize("name", LEGACY)
def test_legacy_formats_element_by_element(hip, oracle, name):
    """A one-hot activation picks one weight: every element position of a block (nibble halves, fifth bits, table entries)
    must come out as the dequantizer gives it, blocks with all-zero and all-one quant bits included."""
    from oracle.oracle import MORE_TYPES
    t = MORE_TYPES[name]
    rng = np.random.default_rng(4400)
    N, K = 6, 64
    wq = inputs.random_blocks(name, N, K, rng).reshape(N * 2, -1)
    hdr = wq.shape[1] - 16
    wq[0, hdr:] = 0xff                       # every nibble 15
    wq[1, hdr:] = 0x00
    if name in ("q5_0", "q5_1"):
        wq[0, hdr - 4:hdr] = 0xff            # every fifth bit set
        wq[1, hdr - 4:hdr] = 0x00
        wq[2, hdr - 4:hdr] = [0x01, 0x80, 0x00, 0x10]     # single bits: elements 0, 15, 28
    wq = wq.reshape(-1)
    w = oracle.dequantize(t, wq, N * K).reshape(N, K)
    for k in range(K):
        x = np.zeros((1, K), np.float32)
        x[0, k] = 1.5
        y = run_device(hip, t, wq, N, K, x)
        assert np.allclose(y[0], 1.5 * w[:, k], rtol=2e-6, atol=1e-9), (name, k, y[0], 1.5 * w[:, k])


@pytest.mark.parametrize("name,N,K", [("q4_k", 4096, 4096), ("q4_k", 9000, 1024), ("mxfp4", 2880, 2880), ("mxfp4", 20000, 512),
                                      ("q8_0", 1000, 2560), ("q6_k", 700, 1024), ("q5_k", 700, 1024), ("q4_0", 900, 1024),
                                      ("q4_1", 900, 1024), ("q5_0", 900, 1024), ("q5_1", 900, 1024), ("iq4_nl", 900, 1024)])
def test_timeline_build_same_results_and_ordered_stamps(hip, oracle, name, N, K):
    """TSHip_SetGemvTimeline selects a build of the kernel that stamps s_memrealtime per wavefront (the eager build for the
    first and third case, which fit one row group per wavefront; the streaming build otherwise).  Its results are the
    normal build's bit for bit, and every wavefront left entry <= staged <= exit (first step done in between where it had a
    row group)."""
    import ctypes as C
    import torch
    from tensorsharp_amd import QuantizedWeight, hip_native as Nat, synth
    from oracle.oracle import MORE_TYPES, Q6_K
    t = {"q4_k": Q4_K, "mxfp4": MXFP4, "q8_0": Q8_0, "q6_k": Q6_K}.get(name) or MORE_TYPES[name]
    dev = torch.device("cuda:0")
    w = synth.random_weight(t, N, K, dev, seed=91)
    qw = QuantizedWeight(w, t, K, N)
    x = torch.randn((1, K), device=dev, generator=torch.Generator(device=dev).manual_seed(5))
    want = hip.LinearForward(x, qw)
    torch.cuda.synchronize()
    waves = 8 * 4 * 256 + 64                       # at most four workgroups of eight wavefronts per CU
    buf = torch.zeros((waves, 8), dtype=torch.int64, device=dev)
    Nat.check_result(Nat.lib().TSHip_SetGemvTimeline(C.c_void_p(buf.data_ptr()), waves * 64), "timeline")
    try:
        got = hip.LinearForward(x, qw)
        torch.cuda.synchronize()
    finally:
        Nat.check_result(Nat.lib().TSHip_SetGemvTimeline(None, 0), "timeline")
    assert torch.equal(got.view(torch.int32), want.view(torch.int32))
    a = buf.cpu().numpy()
    ran = a[a[:, 4] != 0]
    assert ran.shape[0] >= 8 and ran.shape[0] % 8 == 0, ran.shape
    entry, staged, first, exit_ = ran[:, 0], ran[:, 2], ran[:, 3], ran[:, 4]
    worked = first != 0                            # wavefronts without a row group never finish a step
    assert worked.any()
    assert np.all(entry <= staged) and np.all(staged <= exit_)
    assert np.all(staged[worked] <= first[worked]) and np.all(first[worked] <= exit_[worked])
    assert (exit_.max() - entry.min()) * 10 < 5_000_000        # 10 ns ticks: the launch took less than 5 ms
    # and a later launch without the buffer leaves nothing behind
    buf.zero_()
    hip.LinearForward(x, qw)
    torch.cuda.synchronize()
    assert int(buf.abs().sum().item()) == 0


@pytest.mark.parametrize("name,shapes", [("q4_k", [(4096, 4096), (1024, 4096)]), ("q4_k", [(9000, 1024), (300, 1024), (5000, 2048)]),
                                         ("mxfp4", [(2880, 2880), (2880, 2880)]), ("mxfp4", [(20000, 512), (64, 512)]),
                                         ("q8_0", [(1000, 2560), (3000, 512)]), ("q6_k", [(700, 1024), (900, 512)]),
                                         ("q5_k", [(700, 1024), (900, 512)]), ("q4_0", [(900, 1024), (700, 512)]),
                                         ("q4_1", [(900, 1024), (700, 512)]), ("q5_0", [(900, 1024), (700, 512)]),
                                         ("q5_1", [(900, 1024), (700, 512)]), ("iq4_nl", [(900, 1024), (700, 512)])])
def test_timeline_build_of_a_grouped_launch(hip, oracle, name, shapes):
    """Several matrices in one launch with the timeline buffer set (the first and third case fit one row group per
    wavefront and take the eager build): same bits as the normal build, and the stamps name every problem of the launch."""
    import ctypes as C
    import torch
    from tensorsharp_amd import QuantizedWeight, hip_native as Nat, synth
    from oracle.oracle import MORE_TYPES, Q6_K
    t = {"q4_k": Q4_K, "mxfp4": MXFP4, "q8_0": Q8_0, "q6_k": Q6_K}.get(name) or MORE_TYPES[name]
    dev = torch.device("cuda:0")
    ws = [QuantizedWeight(synth.random_weight(t, n, k, dev, seed=91 + i), t, k, n) for i, (n, k) in enumerate(shapes)]
    g = torch.Generator(device=dev).manual_seed(5)
    xs = [torch.randn((1, k), device=dev, generator=g) for _, k in shapes]
    want = [torch.empty((1, n), device=dev) for n, _ in shapes]
    got = [torch.empty((1, n), device=dev) for n, _ in shapes]
    hip.AddmmQuantGroupDevice(hip.PrepareGroup(want, xs, ws))
    torch.cuda.synchronize()
    waves = 8 * 4 * 256 + 64
    buf = torch.zeros((waves, 8), dtype=torch.int64, device=dev)
    Nat.check_result(Nat.lib().TSHip_SetGemvTimeline(C.c_void_p(buf.data_ptr()), waves * 64), "timeline")
    try:
        hip.AddmmQuantGroupDevice(hip.PrepareGroup(got, xs, ws))
        torch.cuda.synchronize()
    finally:
        Nat.check_result(Nat.lib().TSHip_SetGemvTimeline(None, 0), "timeline")
    for a, b in zip(got, want):
        assert torch.equal(a.view(torch.int32), b.view(torch.int32))
    a = buf.cpu().numpy()
    ran = a[a[:, 4] != 0]
    assert ran.shape[0] >= 8 * len(shapes) and ran.shape[0] % 8 == 0, ran.shape
    assert np.all(ran[:, 0] <= ran[:, 2]) and np.all(ran[:, 2] <= ran[:, 4])
    problems = set(int(v) for v in (ran[:, 5] >> 8) & 0xff)
    assert problems == set(range(len(shapes))), problems

