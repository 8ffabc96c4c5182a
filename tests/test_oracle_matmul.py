"""Matmul semantics of the oracle: exact (fp64), managed order, ggml (int8 activation) order."""
import numpy as np
import pytest

import inputs
from oracle.oracle import Q8_0, Q4_K, MXFP4

T = {"q8_0": Q8_0, "q4_k": Q4_K, "mxfp4": MXFP4}


def test_reference_dot_vectors(oracle, golden):
    # ManagedQuantizedOpsTests.cs:113-147 (Q8_0, M=2, K=32) and :149-194 (Q4_K, M=3, K=256):
    # DotRowBatch == naive fp32 dot of the dequantised row, to 5 decimals
    for name, raw_key, K in (("q8_0", "ref_tests_q8_0_raw", 32), ("q4_k", "ref_tests_q4_k_dot_raw", 256)):
        raw = golden[raw_key]
        x = golden[f"ref_tests_{name}_dot_x"]
        deq = oracle.dequantize(T[name], raw)
        naive = np.zeros(x.shape[0], dtype=np.float32)
        for m in range(x.shape[0]):
            s = np.float32(0)
            for i in range(K):
                s = np.float32(s + np.float32(deq[i] * x[m, i]))
            naive[m] = s
        for vw in (4, 8, 16):
            got = oracle.matmul_managed(T[name], raw, 1, K, x, vec_width=vw)[:, 0]
            np.testing.assert_allclose(got, naive, atol=5e-6, rtol=0)
        exact = oracle.matmul_f64(T[name], raw, 1, K, x)[:, 0]
        np.testing.assert_allclose(exact, naive, atol=5e-6, rtol=0)
    # closed form for the Q8_0 vector: row = 0.5*{2,-4,7}, x0 = i/8 -> 0*1 + 0.125*-2 + 0.25*3.5
    raw = golden["ref_tests_q8_0_raw"]
    x = golden["ref_tests_q8_0_dot_x"]
    y = oracle.matmul_f64(Q8_0, raw, 1, 32, x)[:, 0]
    assert y[0] == pytest.approx(0.625, abs=1e-12)
    assert y[1] == pytest.approx(1.0 * 1.0 - 2.0 * (1 - 0.03125) + 3.5 * (1 - 0.0625), abs=1e-12)


@pytest.mark.parametrize("name", ["q8_0", "q4_k", "mxfp4"])
def test_exact_matmul_is_dense_gemm_on_dequantized_weights(oracle, name):
    rng = np.random.default_rng(9)
    N, K, M = 40, 768, 5
    w = oracle.quantize(T[name], (rng.standard_normal(N * K) * 0.02).astype(np.float32))
    x = rng.standard_normal((M, K)).astype(np.float32)
    dense = oracle.dequantize(T[name], w).reshape(N, K).astype(np.float64)
    want = x.astype(np.float64) @ dense.T
    got = oracle.matmul_f64(T[name], w, N, K, x)
    np.testing.assert_allclose(got, want, rtol=1e-12, atol=1e-12)
    # managed fp32 order stays within fp32 rounding of it; GEMM row m == GEMV of row m
    man = oracle.matmul_managed(T[name], w, N, K, x)
    assert inputs.row_l2_err(man, want) < 1e-6
    for m in range(M):
        one = oracle.matmul_managed(T[name], w, N, K, x[m:m + 1])
        assert np.array_equal(one[0], man[m])
    # linearity in x and zero input
    got2 = oracle.matmul_f64(T[name], w, N, K, 2 * x)
    np.testing.assert_allclose(got2, 2 * got, rtol=1e-12, atol=1e-12)
    assert np.all(oracle.matmul_f64(T[name], w, N, K, np.zeros((1, K), np.float32)) == 0)


def test_ggml_order_golden_known_answers(oracle, golden):
    # ggml_mul_mat output of the reference's CPU backend, stored with its inputs
    for name, t in T.items():
        wq, x, want = golden[f"mm_{name}_wq"], golden[f"mm_{name}_x"], golden[f"mm_{name}_y_ggml"]
        M, N = want.shape
        K = x.shape[1]
        got = oracle.matmul_ggml(t, wq, N, K, x)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), name
        # and both sit within the int8-activation error of the exact product
        exact = oracle.matmul_f64(t, wq, N, K, x)
        assert inputs.row_l2_err(got, exact) < 5e-3


def test_ggml_order_matches_reference_build(oracle, reference):
    rng = np.random.default_rng(10)
    for name, t in T.items():
        N, K, M = 96, 1024, 4
        w = oracle.quantize(t, (rng.standard_normal(N * K) * 0.02).astype(np.float32))
        x = rng.standard_normal((M, K)).astype(np.float32)
        assert np.array_equal(oracle.matmul_ggml(t, w, N, K, x), reference.mul_mat(t, w, N, K, x, threads=2)), name


def test_argument_checks(oracle):
    import ctypes as C
    w = np.zeros(34 * 4, dtype=np.uint8)
    x = np.zeros((1, 64), dtype=np.float32)
    out = np.zeros((1, 2), dtype=np.float64)
    f = oracle.lib.tso_matmul_f64
    f32p, f64p = C.POINTER(C.c_float), C.POINTER(C.c_double)
    ok = f(8, C.c_void_p(w.ctypes.data), 2, 64, x.ctypes.data_as(f32p), 1, 64, out.ctypes.data_as(f64p))
    assert ok == 0
    assert f(8, C.c_void_p(w.ctypes.data), 2, 48, x.ctypes.data_as(f32p), 1, 64, out.ctypes.data_as(f64p)) == -1
    assert f(8, C.c_void_p(w.ctypes.data), 2, 64, x.ctypes.data_as(f32p), 1, 32, out.ctypes.data_as(f64p)) == -1
    assert f(77, C.c_void_p(w.ctypes.data), 2, 64, x.ctypes.data_as(f32p), 1, 64, out.ctypes.data_as(f64p)) == -2
