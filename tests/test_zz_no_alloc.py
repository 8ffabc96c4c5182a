"""GPU: the entry point that allocates nothing (TSHip_AddmmQuantF32DeviceNoAlloc) against TSHip_AddmmQuantF32Device.

Both run the same kernels; the only difference is where the scratch (converted activations, sums of K chunks) lives:
a static device array instead of the library's grow-only buffers.  Results must be identical bit for bit, and within
the matmul bar (row-L2 <= 1e-3) of the fp64 oracle.  Two calls in a row share the static array, the second one smaller.
"""
import numpy as np
import pytest

import inputs
from oracle.oracle import Q8_0, Q4_K, MXFP4

pytestmark = pytest.mark.gpu


def _both(hip, t, wq, N, K, x):
    import torch
    w = torch.from_numpy(wq).cuda()
    xd = torch.from_numpy(np.ascontiguousarray(x)).cuda()
    M = x.shape[0]
    y_ref = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    y_new = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    hip.UseCurrentStream()
    hip.AddmmQuantDevice(y_ref, xd, w.data_ptr(), t, K, N, wq.size)
    hip.AddmmQuantDeviceNoAlloc(y_new, xd, w.data_ptr(), t, K, N, wq.size)
    torch.cuda.synchronize()
    return y_ref.cpu().numpy(), y_new.cpu().numpy()


@pytest.mark.parametrize("t", [Q4_K, Q8_0, MXFP4])
def test_two_calls_in_a_row_second_smaller(hip, oracle, t):
    rng = np.random.default_rng(7100 + t)
    # first: 300 rows on the 128-row tiles with a long K (K chunks in use for the 4-bit formats); second: 40 rows
    # (register-resident kernel) of a shorter K, whose scratch overlaps the first call's
    for (M, N, K) in [(300, 512, 8192), (40, 200, 1024)]:
        wq = oracle.quantize(t, (rng.standard_normal(N * K) * 0.02).astype(np.float32))
        x = rng.standard_normal((M, K)).astype(np.float32)
        y_ref, y_new = _both(hip, t, wq, N, K, x)
        assert np.array_equal(y_ref.view(np.uint32), y_new.view(np.uint32)), (t, M, N, K)
        ref = oracle.matmul_f64(t, wq, N, K, x)
        assert inputs.row_l2_err(y_new, ref) <= 1e-3


def test_decode_row_and_long_k_chunks(hip, oracle):
    rng = np.random.default_rng(7200)
    # M = 1 takes the GEMV (no scratch at all); M = 16 with K = 16384 needs K chunks in the register-resident kernel
    for (M, N, K) in [(1, 384, 2048), (16, 96, 16384), (1, 64, 256)]:
        wq = oracle.quantize(Q4_K, (rng.standard_normal(N * K) * 0.02).astype(np.float32))
        x = rng.standard_normal((M, K)).astype(np.float32)
        y_ref, y_new = _both(hip, Q4_K, wq, N, K, x)
        assert np.array_equal(y_ref.view(np.uint32), y_new.view(np.uint32)), (M, N, K)
        assert inputs.row_l2_err(y_new, oracle.matmul_f64(Q4_K, wq, N, K, x)) <= 1e-3


def test_rejects_sizes_beyond_the_static_scratch(hip):
    import torch
    from tensorsharp_amd import hip_native
    # 20000 rows x 4096: 164 MB of converted activations > 64 MiB
    M, N, K = 20000, 256, 4096
    w = torch.zeros(N * (K // 256) * 144, dtype=torch.uint8, device="cuda")
    x = torch.zeros((M, K), dtype=torch.float32, device="cuda")
    y = torch.zeros((M, N), dtype=torch.float32, device="cuda")
    with pytest.raises(RuntimeError, match="exceed the static scratch buffer"):
        hip.AddmmQuantDeviceNoAlloc(y, x, w.data_ptr(), Q4_K, K, N, w.numel())
    assert "scratch" in hip_native.get_last_error()
