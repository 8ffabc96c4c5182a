"""GPU: contracts of the C-ABI boundary that are not about one kernel's arithmetic - operands beyond the kernels'
32-bit addressing (cut by rows inside the call, as the bridge does: ggml_ops_matmul.cpp:331-367), two host threads on
two streams, the weight cache's hit rules (ggml_ops_core.cpp:604-640), expert ids that are not in the table."""
import threading

import numpy as np
import pytest

import inputs
from oracle.oracle import Q8_0, Q4_K, MXFP4

pytestmark = pytest.mark.gpu


def _q8_rows_on_device(torch, N, K, seed):
    """Valid random Q8_0 rows made on the device (a 2 GiB tensor is not made on the host): d = 2^-8, int8 quants."""
    g = torch.Generator(device="cuda").manual_seed(seed)
    nb = N * (K // 32)
    raw = torch.randint(0, 256, (nb, 34), dtype=torch.uint8, device="cuda", generator=g)
    raw[:, 0] = 0x00
    raw[:, 1] = 0x1c          # fp16 0x1c00 = 2^-8
    return raw.reshape(-1)


def test_weight_of_more_than_2_gib_is_cut_by_rows(hip, oracle):
    """A Q8_0 LM head of 250 000 x 8192 (2.18 GB): one decode row and a small batch, checked on rows either side of
    the cut (and at both ends) against the fp64 oracle on exactly those weight rows."""
    import torch
    from tensorsharp_amd import QuantizedWeight
    N, K = 250_000, 8192
    rs = 34 * (K // 32)
    assert N * rs > 2**31
    w = _q8_rows_on_device(torch, N, K, 5)
    qw = QuantizedWeight(w, Q8_0, K, N)
    rng = np.random.default_rng(8100)
    cut = ((2**31 - 65) // rs) // 256 * 256                   # first row of the second slice
    rows = np.array([0, 1, cut - 1, cut, cut + 1, N - 2, N - 1, 123_457])
    sub = w.reshape(N, rs)[torch.from_numpy(rows).cuda()].cpu().numpy().reshape(-1)
    for M in (1, 8):
        x = rng.standard_normal((M, K)).astype(np.float32)
        y = hip.LinearForward(torch.from_numpy(x).cuda(), qw)
        torch.cuda.synchronize()
        got = y[:, torch.from_numpy(rows).cuda()].cpu().numpy()
        ref = oracle.matmul_f64(Q8_0, sub, len(rows), K, x)
        # the bar is relative to the whole output row's norm; the sampled columns' norm is smaller, so this is stricter
        assert inputs.row_l2_err(got, ref) <= 1e-3, (M, inputs.row_l2_err(got, ref))
        assert bool(torch.isfinite(y).all())
    del w, qw, y
    torch.cuda.empty_cache()


def test_two_host_threads_on_two_streams(hip, oracle):
    """Each thread selects its own stream (TSHip_SetStream is per thread) and runs prefill matmuls whose scratch is the
    stream's own; results must equal the serial ones bit for bit."""
    import torch
    from tensorsharp_amd import QuantizedWeight
    rng = np.random.default_rng(8200)
    jobs = []
    for i, (t, M, N, K) in enumerate([(Q4_K, 200, 512, 2048), (Q8_0, 96, 768, 1024)]):
        wq = oracle.quantize(t, (rng.standard_normal(N * K) * 0.02).astype(np.float32))
        x = rng.standard_normal((M, K)).astype(np.float32)
        qw = QuantizedWeight(torch.from_numpy(wq).cuda(), t, K, N)
        xd = torch.from_numpy(x).cuda()
        serial = hip.LinearForward(xd, qw)
        torch.cuda.synchronize()
        jobs.append((qw, xd, serial.clone(), oracle.matmul_f64(t, wq, N, K, x)))
    results = [None, None]
    errors = []

    def worker(i):
        try:
            qw, xd, _, _ = jobs[i]
            st = torch.cuda.Stream()
            with torch.cuda.stream(st):
                for _ in range(20):
                    y = hip.LinearForward(xd, qw)
            st.synchronize()
            results[i] = y
        except Exception as e:      # noqa: BLE001 - reported below
            errors.append(e)

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(2)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    assert not errors, errors
    for i in range(2):
        _, _, serial, ref = jobs[i]
        assert torch.equal(results[i], serial), i
        assert inputs.row_l2_err(results[i].cpu().numpy(), ref) <= 1e-3


def test_host_address_reused_for_another_size_is_uploaded_again(hip, oracle):
    """The same host address first holds a 256-row weight, then a 128-row one with other bytes: a cache hit on
    'enough bytes' would run the second call on the first tensor's rows."""
    rng = np.random.default_rng(8300)
    K = 512
    big = oracle.quantize(Q8_0, (rng.standard_normal(256 * K) * 0.02).astype(np.float32))
    small = oracle.quantize(Q8_0, (rng.standard_normal(128 * K) * 0.02).astype(np.float32))
    buf = np.empty_like(big)
    x = rng.standard_normal((2, K)).astype(np.float32)
    buf[:] = big
    out = np.empty((2, 256), dtype=np.float32)
    hip.AddmmQuant(out, x, buf.ctypes.data, Q8_0, K, 256, buf.size)
    assert inputs.row_l2_err(out, oracle.matmul_f64(Q8_0, big, 256, K, x)) <= 1e-3
    buf[:small.size] = small
    out2 = np.empty((2, 128), dtype=np.float32)
    hip.AddmmQuant(out2, x, buf.ctypes.data, Q8_0, K, 128, small.size)
    assert inputs.row_l2_err(out2, oracle.matmul_f64(Q8_0, small, 128, K, x)) <= 1e-3
    hip.ClearHostBufferCache()


def test_sync_of_a_pointer_that_was_never_uploaded_is_a_no_op(hip):
    """ModelBase.SyncTensorHostCache (ModelBase.cs:1859-1865) calls it on arbitrary tensors."""
    a = np.arange(16, dtype=np.float32)
    hip.SyncHostBuffer(a)
    assert np.array_equal(a, np.arange(16, dtype=np.float32))


def test_batch_on_a_preloaded_stack_uses_the_device_copy(hip, oracle):
    """AddmmQuantBatch with m2_data = a preload key whose host bytes are gone (ModelBase.cs:690-697 releases them)."""
    rng = np.random.default_rng(8400)
    K, rows = 256, [64, 32, 96]
    parts = [oracle.quantize(Q4_K, (rng.standard_normal(n * K) * 0.02).astype(np.float32)) for n in rows]
    stack = np.concatenate(parts)
    offs = np.concatenate([[0], np.cumsum([p.size for p in parts])[:-1]])
    key = 0x7E57_0000_1000                      # an opaque key: not readable memory
    hip.PreloadQuantizedWeight(key, stack.ctypes.data, Q4_K, K, sum(rows), stack.size)
    x = rng.standard_normal((3, K)).astype(np.float32)
    out = np.zeros((3, max(rows)), dtype=np.float32)
    hip.AddmmQuantBatch(out, x, key, Q4_K, K, stack.size, offs, rows)
    for b, n in enumerate(rows):
        ref = oracle.matmul_f64(Q4_K, parts[b], n, K, x[b:b + 1])
        assert inputs.row_l2_err(out[b:b + 1, :n], ref) <= 1e-3
    hip.InvalidateHostBuffer(key)


@pytest.mark.parametrize("T", [1, 2, 40])
def test_expert_id_outside_the_table_contributes_nothing(hip, oracle, T):
    """ids are read on the device; one that names no expert must neither fault nor contribute (decode path: T * k <= 8,
    grouped path beyond)."""
    import torch
    rng = np.random.default_rng(8500 + T)
    E, H, F, k = 8, 256, 512, 4
    t = MXFP4
    gu = oracle.quantize(t, (rng.standard_normal(E * 2 * F * H) * 0.05).astype(np.float32))
    dn = oracle.quantize(t, (rng.standard_normal(E * H * F) * 0.05).astype(np.float32))
    gb = (rng.standard_normal((E, 2 * F)) * 0.1).astype(np.float32)
    db = (rng.standard_normal((E, H)) * 0.1).astype(np.float32)
    hidden = rng.standard_normal((T, H)).astype(np.float32)
    ids, wts = oracle.moe_route(rng.standard_normal((T, E)).astype(np.float32), k)
    bad = ids.copy()
    bad[0, 1] = -1
    bad[T - 1, 3] = E + 1000
    # reference: the same call with the bad assignments' weights zeroed and their ids replaced by a valid expert
    good, w0 = bad.copy(), wts.copy()
    for (r, s) in ((0, 1), (T - 1, 3)):
        good[r, s] = 0
        w0[r, s] = 0.0
    ref = oracle.moe_forward(t, gu, gb, dn, db, E, H, F, hidden, good, w0)
    c = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    out = hip.MoEExpertsGptOssForward(c(hidden), c(bad.astype(np.int32)), c(wts), c(gu), c(gb), c(dn), c(db), t, E, H, F)
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    assert np.all(np.isfinite(got))
    assert inputs.row_l2_err(got, ref) <= 1e-3, inputs.row_l2_err(got, ref)


def test_device_gather_of_more_than_65535_indices(hip, oracle):
    import torch
    from tensorsharp_amd import QuantizedWeight
    rng = np.random.default_rng(8600)
    N, K, n = 300, 64, 70_000
    wq = oracle.quantize(Q8_0, (rng.standard_normal(N * K) * 0.02).astype(np.float32))
    idx = rng.integers(0, N, n).astype(np.int32)
    out = torch.empty((n, K), dtype=torch.float32, device="cuda")
    hip.GetRowsQuantDevice(out, QuantizedWeight(torch.from_numpy(wq).cuda(), Q8_0, K, N), torch.from_numpy(idx).cuda())
    torch.cuda.synchronize()
    deq = oracle.dequantize(Q8_0, wq).reshape(N, K)
    assert np.array_equal(out.cpu().numpy().view(np.uint32), deq[idx].view(np.uint32))
