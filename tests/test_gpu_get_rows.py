"""GPU parity: embedding gather (GetRowsQuant) through the C ABI.  Bit-exact: a gathered row equals the
oracle's dequantization of that row.  The first test restates the reference's own regression test
(TensorSharp.GGML.Native/tests/get_rows_quant_test.cpp:98-210)."""
import ctypes as C

import numpy as np
import pytest

from oracle.oracle import Q8_0, Q4_K, MXFP4

pytestmark = pytest.mark.gpu
T_ = {"q8_0": Q8_0, "q4_k": Q4_K, "mxfp4": MXFP4}
ROW = {"q8_0": lambda k: 34 * k // 32, "q4_k": lambda k: 144 * k // 256, "mxfp4": lambda k: 17 * k // 32}


def unaligned_f32(n, like=None):
    """n floats at an address that is 4-byte but not 32-byte aligned (make_unaligned_ptr of the reference test)."""
    raw = np.zeros(n * 4 + 64, dtype=np.uint8)
    off = 0
    while (raw.ctypes.data + off) % 32 == 0 or (raw.ctypes.data + off) % 4 != 0:
        off += 1
    v = raw[off:off + n * 4].view(np.float32)
    if like is not None:
        v[:] = like.ravel()
    return v


def test_reference_regression_cases_f32_source(hip):
    rows, cols = 32, 64
    src = (np.arange(rows, dtype=np.float32)[:, None] * 1000 + np.arange(cols, dtype=np.float32)[None, :])
    idx = np.array([5, 1], dtype=np.int32)
    expect = src[idx]
    for label, res, s in (("aligned", np.zeros((2, cols), np.float32), src.copy()),
                          ("unaligned result", unaligned_f32(2 * cols).reshape(2, cols), src.copy()),
                          ("unaligned source", np.zeros((2, cols), np.float32), unaligned_f32(rows * cols, src).reshape(rows, cols)),
                          ("both unaligned", unaligned_f32(2 * cols).reshape(2, cols), unaligned_f32(rows * cols, src).reshape(rows, cols))):
        hip.GetRowsQuant(res, s.ctypes.data, 0, cols, rows, rows * cols * 4, idx)
        assert np.array_equal(res, expect), label
        hip.InvalidateHostBuffer(s.ctypes.data)
    hip.ClearHostBufferCache()


@pytest.mark.parametrize("name", ["q8_0", "q4_k", "mxfp4"])
def test_gather_is_bit_exact_host_and_device(hip, oracle, name):
    import torch
    from tensorsharp_amd import QuantizedWeight
    rng = np.random.default_rng(71)
    N, K = 700, 768
    t = T_[name]
    wq = oracle.quantize(t, (rng.standard_normal(N * K) * 0.05).astype(np.float32))
    deq = oracle.dequantize(t, wq, N * K).reshape(N, K)
    idx = np.array([699, 0, 5, 5, 123, 698, 1, 350], dtype=np.int32)
    out = np.full((len(idx), K), np.nan, dtype=np.float32)
    hip.GetRowsQuant(out, wq.ctypes.data, t, K, N, wq.size, idx)
    assert np.array_equal(out.view(np.uint32), deq[idx].view(np.uint32))
    hip.ClearHostBufferCache()
    # device form, strided result rows, an out-of-range index -> zero row
    qw = QuantizedWeight(torch.from_numpy(wq).cuda(), t, K, N)
    idx2 = np.array([3, -1, 699, N, 42], dtype=np.int32)
    res = torch.full((len(idx2), K + 16), 7.0, device="cuda")[:, :K]
    hip.GetRowsQuantDevice(res, qw, torch.from_numpy(idx2).cuda())
    torch.cuda.synchronize()
    got = res.cpu().numpy()
    for i, r in enumerate(idx2):
        want = deq[r] if 0 <= r < N else np.zeros(K, np.float32)
        assert np.array_equal(got[i].view(np.uint32), want.view(np.uint32)), (name, i, r)


def test_argument_errors(hip, oracle):
    wq = oracle.quantize(Q8_0, np.ones(4 * 64, dtype=np.float32))
    out = np.zeros((2, 64), dtype=np.float32)
    with pytest.raises(RuntimeError, match="Index out of range"):
        hip.GetRowsQuant(out, wq.ctypes.data, Q8_0, 64, 4, wq.size, np.array([0, 4], dtype=np.int32))
    with pytest.raises(RuntimeError, match="Shape mismatch"):
        hip.GetRowsQuant(out, wq.ctypes.data, Q8_0, 64, 4, wq.size, np.array([0, 1, 2], dtype=np.int32))
    with pytest.raises(RuntimeError, match="Unsupported source type"):
        hip.GetRowsQuant(out, wq.ctypes.data, 14, 64, 4, wq.size, np.array([0, 1], dtype=np.int32))
    with pytest.raises(ValueError):
        hip.GetRowsQuant(np.zeros((2, 64)), wq.ctypes.data, Q8_0, 64, 4, wq.size, np.array([0, 1], dtype=np.int32))
    hip.ClearHostBufferCache()
