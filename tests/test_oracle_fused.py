"""Pins the oracle's RMSNorm and SiLU restatements (ggml-cpu/ops.cpp:3646-3695, vec.h:958-960) against what the
mathematics fixes: fp64 closed forms, invariants and special cases."""
import numpy as np


def test_rms_norm_closed_form_and_invariants(oracle):
    rng = np.random.default_rng(81)
    x = (rng.standard_normal((5, 2560)) * rng.uniform(0.01, 30, (5, 1))).astype(np.float32)
    w = rng.uniform(0.5, 1.5, 2560).astype(np.float32)
    eps = 1e-6
    got = oracle.rms_norm_mul(x, w, eps)
    x64 = x.astype(np.float64)
    ref = x64 / np.sqrt((x64 * x64).mean(axis=1, keepdims=True) + eps) * w
    assert np.max(np.abs(got - ref) / (np.abs(ref) + 1e-30)) < 4e-7            # a few fp32 roundings
    # unit RMS before the weight; scale invariance x -> c x (eps negligible); a constant row maps to +-w
    g1 = oracle.rms_norm_mul(x, np.ones_like(w), 0.0)
    assert np.allclose(np.sqrt((g1.astype(np.float64) ** 2).mean(axis=1)), 1.0, atol=1e-6)
    assert np.allclose(oracle.rms_norm_mul(x * 8.0, w, 0.0), oracle.rms_norm_mul(x, w, 0.0), rtol=1e-6)   # power of two: exact scaling
    c = np.full((1, 64), -3.0, dtype=np.float32)
    assert np.allclose(oracle.rms_norm_mul(c, w[:64], 0.0), -w[:64], rtol=2e-7)
    # eps dominates a zero row: output exactly zero, no NaN
    z = oracle.rms_norm_mul(np.zeros((1, 64), np.float32), w[:64], 1e-5)
    assert np.all(z == 0)
    # a dropped eps or a mean over the wrong count would fail this one
    t = np.array([[3.0, 4.0]], dtype=np.float32)
    assert np.allclose(oracle.rms_norm_mul(t, np.ones(2, np.float32), 0.5), t / np.sqrt(12.5 + 0.5), rtol=2e-7)


def test_silu_mul_closed_form_and_identities(oracle):
    rng = np.random.default_rng(83)
    gu = (rng.standard_normal((4, 512)) * 4).astype(np.float32)
    got = oracle.silu_mul(gu)
    g, u = gu[:, :256].astype(np.float64), gu[:, 256:].astype(np.float64)
    ref = g / (1.0 + np.exp(-g)) * u
    assert np.max(np.abs(got - ref)) <= 4e-7 * np.max(np.abs(ref))
    # silu(x) - silu(-x) = x ; silu(0) = 0 ; the gate is the FIRST half (swapping halves changes the result)
    x = np.linspace(-20, 20, 101, dtype=np.float32)
    one = np.ones_like(x)
    a = oracle.silu_mul(np.concatenate([x, one])[None, :])[0]
    b = oracle.silu_mul(np.concatenate([-x, one])[None, :])[0]
    assert np.allclose(a - b, x, atol=2e-6)
    assert oracle.silu_mul(np.array([[0.0, 5.0]], np.float32))[0, 0] == 0.0
    assert np.isclose(oracle.silu_mul(np.array([[2.0, 3.0]], np.float32))[0, 0], 2 / (1 + np.exp(-2.0)) * 3, rtol=1e-6)
