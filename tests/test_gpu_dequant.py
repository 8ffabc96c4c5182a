"""GPU parity: dequantization through the C ABI is bit-exact with the oracle."""
import numpy as np
import pytest

import inputs
from oracle.oracle import Q8_0, Q4_K, MXFP4

pytestmark = pytest.mark.gpu
T = {"q8_0": Q8_0, "q4_k": Q4_K, "mxfp4": MXFP4}
BB = {"q8_0": 34, "q4_k": 144, "mxfp4": 17}


def bits_equal(a, b):
    a = np.asarray(a, dtype=np.float32).view(np.uint32)
    b = np.asarray(b, dtype=np.float32).view(np.uint32)
    nan = (b & 0x7FFFFFFF) > 0x7F800000
    return np.array_equal(a[~nan], b[~nan]) and np.all(((a[nan] & 0x7FFFFFFF) > 0x7F800000))


def test_reference_unit_test_vectors(hip, golden):
    for name in ("q8_0", "q4_k"):
        y = hip.DequantizeToFloat32(T[name], golden[f"ref_tests_{name}_raw"], 32 if name == "q8_0" else 256)
        np.testing.assert_array_equal(y[golden[f"ref_tests_{name}_expect_idx"]], golden[f"ref_tests_{name}_expect_val"])


def test_golden_blocks(hip, golden):
    for name, t in T.items():
        q = golden[f"blocks_{name}_q"]
        want = golden[f"blocks_{name}_deq"]
        assert bits_equal(hip.DequantizeToFloat32(t, q, want.size), want), name


def test_all_fp16_scales_q8_0(hip, oracle):
    codes = np.arange(65536, dtype=np.uint16)
    raw = np.zeros((65536, 34), dtype=np.uint8)
    raw[:, 0], raw[:, 1] = codes & 0xFF, codes >> 8
    raw[:, 2:] = ((np.arange(32)[None, :] * 37 + codes[:, None] * 11) % 256).astype(np.uint8)
    raw = raw.reshape(-1)
    assert bits_equal(hip.DequantizeToFloat32(Q8_0, raw, 65536 * 32), oracle.dequantize(Q8_0, raw))


def test_all_e8m0_codes_mxfp4(hip, oracle):
    raw = np.zeros((256, 16, 17), dtype=np.uint8)
    raw[:, :, 0] = np.arange(256, dtype=np.uint8)[:, None]
    raw[:, :, 1:] = np.arange(256, dtype=np.uint8).reshape(16, 16)[None]
    raw = raw.reshape(-1)
    assert bits_equal(hip.DequantizeToFloat32(MXFP4, raw, 256 * 16 * 32), oracle.dequantize(MXFP4, raw))


@pytest.mark.parametrize("name", ["q8_0", "q4_k", "mxfp4"])
def test_random_bytes_host_and_device_entry(hip, oracle, name):
    import torch
    rng = np.random.default_rng(21)
    raw = rng.integers(0, 256, size=BB[name] * 20000, dtype=np.uint8)
    want = oracle.dequantize(T[name], raw)
    assert bits_equal(hip.DequantizeToFloat32(T[name], raw, want.size), want)
    dev = torch.from_numpy(raw).cuda()
    out = hip.DequantizeToFloat32Device(T[name], dev, want.size)
    torch.cuda.synchronize()
    assert bits_equal(out.cpu().numpy(), want)


def test_q4_k_every_scale_code_and_unaligned_blocks(hip, oracle):
    # every 6-bit scale / min code in every sub-block position and every nibble; then the same blocks at a device
    # address that is not 16-byte aligned (the dequantizer has a kernel for aligned blocks and one for the rest)
    import torch
    rng = np.random.default_rng(77)
    raw = rng.integers(0, 256, size=(4096, 144), dtype=np.uint8)
    codes = np.arange(4096)
    raw[:, 0:2] = np.array([0x00, 0x3C], dtype=np.uint8)            # d = 1.0
    raw[:, 2:4] = np.array([0x00, 0x38], dtype=np.uint8)            # dmin = 0.5
    for j in range(8):                                              # sub-block j: scale = code % 64, min = code // 64 (rotated per j)
        sc, mn = (codes + 7 * j) % 64, ((codes // 64) + 5 * j) % 64
        if j < 4:
            raw[:, 4 + j] = (raw[:, 4 + j] & 0xC0) | sc
            raw[:, 8 + j] = (raw[:, 8 + j] & 0xC0) | mn
        else:
            raw[:, 8 + j] = (sc & 15) | ((mn & 15) << 4)
            raw[:, j] = (raw[:, j] & 0x3F) | ((sc >> 4) << 6)
            raw[:, 4 + j] = (raw[:, 4 + j] & 0x3F) | ((mn >> 4) << 6)
    raw = raw.reshape(-1)
    want = oracle.dequantize(Q4_K, raw)
    dev = torch.from_numpy(raw).cuda()
    out = hip.DequantizeToFloat32Device(Q4_K, dev, want.size)
    torch.cuda.synchronize()
    assert bits_equal(out.cpu().numpy(), want)
    shifted = torch.empty(raw.size + 16, dtype=torch.uint8, device="cuda")
    for off in (2, 4, 9):
        shifted[off:off + raw.size] = dev
        out = hip.DequantizeToFloat32Device(Q4_K, shifted[off:off + raw.size], want.size)
        torch.cuda.synchronize()
        assert bits_equal(out.cpu().numpy(), want), off


@pytest.mark.parametrize("name", ["q8_0", "mxfp4", "q4_k"])
def test_destination_not_16_byte_aligned(hip, oracle, name):
    import torch
    rng = np.random.default_rng(79)
    raw = rng.integers(0, 256, size=BB[name] * 3000, dtype=np.uint8)
    want = oracle.dequantize(T[name], raw)
    buf = torch.zeros(want.size + 8, dtype=torch.float32, device="cuda")
    for off in (1, 3):
        hip.DequantizeToFloat32Device(T[name], torch.from_numpy(raw).cuda(), want.size, dst=buf[off:off + want.size])
        torch.cuda.synchronize()
        assert bits_equal(buf[off:off + want.size].cpu().numpy(), want), (name, off)


def test_full_size_weight(hip, oracle):
    # cfg 2 gate projection, 58.7 M weights, reference-quantized
    fmt, N, K = inputs.CFG2["gate"]
    q = oracle.quantize(T[fmt], inputs.weights("cfg2.gate", N * K))
    assert bits_equal(hip.DequantizeToFloat32(T[fmt], q, N * K), oracle.dequantize(T[fmt], q))


def test_codes(hip):
    from tensorsharp_amd import hip_native as N
    lib = N.lib()
    buf = np.zeros(144, dtype=np.uint8)
    out = np.zeros(256, dtype=np.float32)
    assert lib.TSHip_DequantizeToF32(Q4_K, None, 256, out.ctypes.data) == -1
    assert lib.TSHip_DequantizeToF32(Q4_K, buf.ctypes.data, 255, out.ctypes.data) == -1
    assert lib.TSHip_DequantizeToF32(10, buf.ctypes.data, 256, out.ctypes.data) == -2     # Q2_K: no dequantizer here
    assert lib.TSHip_DequantizeToF32(Q4_K, buf.ctypes.data, 0, out.ctypes.data) == 0
    src = np.arange(8, dtype=np.float32)
    dst = np.zeros(8, dtype=np.float32)
    assert lib.TSHip_DequantizeToF32(0, src.ctypes.data, 8, dst.ctypes.data) == 0 and np.array_equal(src, dst)


# ---- the other block formats the managed code reads (ManagedQuantizedOps.cs:40-59) ----------------------------
from oracle.oracle import MORE_TYPES, BLOCK  # noqa: E402
import os  # noqa: E402


@pytest.fixture(scope="module")
def formats():
    return np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "formats.npz"))


@pytest.mark.parametrize("name", sorted(MORE_TYPES))
def test_more_formats_reference_known_answers(hip, formats, name):
    # bytes and floats written by the reference's own quantizers / dequantizers (tests/golden/make_golden_formats.py)
    t = MORE_TYPES[name]
    for q, want in ((formats[f"{name}_q"], formats[f"{name}_deq"]), (formats[f"{name}_rq"], formats[f"{name}_rdeq"])):
        assert bits_equal(hip.DequantizeToFloat32(t, q, want.size), want), name


@pytest.mark.parametrize("name", sorted(MORE_TYPES))
def test_more_formats_random_bytes_and_row_gather(hip, oracle, name):
    import torch
    t = MORE_TYPES[name]
    bs, bb = BLOCK[t]
    rng = np.random.default_rng(23 + t)
    K = 512
    rows = 300
    raw = rng.integers(0, 256, size=rows * (K // bs) * bb, dtype=np.uint8)
    want = oracle.dequantize(t, raw)
    dev = torch.from_numpy(raw).cuda()
    out = hip.DequantizeToFloat32Device(t, dev, want.size)
    torch.cuda.synchronize()
    assert bits_equal(out.cpu().numpy(), want)
    # embedding gather of the same rows
    idx = np.array([299, 0, 17, 150, 17], dtype=np.int32)
    res = np.full((idx.size, K), 7.0, dtype=np.float32)
    hip.GetRowsQuant(res, raw.ctypes.data, t, K, rows, raw.size, idx)
    w = want.reshape(rows, K)
    for i, r in enumerate(idx):
        assert bits_equal(res[i], w[r]), (name, i)
    hip.ClearHostBufferCache()


def test_q8_1_dequant_gather_and_matmul(hip, oracle):
    # Q8_1 has no reference-written known answers (ggml has no dequantizer for it); the oracle's restatement is pinned by
    # its closed form over every scale code.  Here: bit-exact dequantization and row gather, and the matmul (dequantized
    # slices through the dense kernel) against the fp64 product at the matmul bar 1e-3 * ||row||.
    import torch
    from oracle.oracle import Q8_1
    rng = np.random.default_rng(61)
    K, rows = 512, 300
    raw = rng.integers(0, 256, size=rows * (K // 32) * 36, dtype=np.uint8)
    want = oracle.dequantize(Q8_1, raw)
    assert bits_equal(hip.DequantizeToFloat32(Q8_1, raw, want.size), want)
    out = hip.DequantizeToFloat32Device(Q8_1, torch.from_numpy(raw).cuda(), want.size)
    torch.cuda.synchronize()
    assert bits_equal(out.cpu().numpy(), want)
    idx = np.array([299, 0, 17, 150, 17], dtype=np.int32)
    res = np.full((idx.size, K), 7.0, dtype=np.float32)
    hip.GetRowsQuant(res, raw.ctypes.data, Q8_1, K, rows, raw.size, idx)
    for i, r in enumerate(idx):
        assert bits_equal(res[i], want.reshape(rows, K)[r]), i
    hip.ClearHostBufferCache()
    # finite scales for the product
    blocks = raw.reshape(-1, 36).copy()
    blocks[:, 0:2] = rng.uniform(1e-3, 4e-3, blocks.shape[0]).astype(np.float16).view(np.uint8).reshape(-1, 2)
    w = blocks.reshape(-1)
    for M in (1, 7):
        x = rng.standard_normal((M, K)).astype(np.float32)
        ref = oracle.matmul_f64(Q8_1, w, rows, K, x)
        got = np.full((M, rows), np.nan, np.float32)
        hip.AddmmQuant(got, x, w.ctypes.data, Q8_1, K, rows, w.size)
        hip.ClearHostBufferCache()
        assert np.all(np.abs(got - ref) <= 1e-3 * np.linalg.norm(ref, axis=1, keepdims=True))
