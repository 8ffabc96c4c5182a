"""Quantizers of the oracle (restating ggml-quants.c:199-222, :260-305, :622-701, :1280-1350)."""
import hashlib

import numpy as np
import pytest

import inputs
from oracle.oracle import Q8_0, Q4_K, MXFP4

T = {"q8_0": Q8_0, "q4_k": Q4_K, "mxfp4": MXFP4}
MXFP4_TABLE = np.array([0, 1, 2, 3, 4, 6, 8, 12, 0, -1, -2, -3, -4, -6, -8, -12], dtype=np.float32)


def test_golden_blocks_byte_exact(oracle, golden):
    # bytes produced by the reference's own quantizer on the same fp32 inputs
    for name, t in T.items():
        q = oracle.quantize(t, golden[f"blocks_{name}_x"])
        assert np.array_equal(q, golden[f"blocks_{name}_q"]), name


def test_q8_k_activation_blocks(oracle, golden):
    assert np.array_equal(oracle.quantize_q8_K(golden["q8k_x"]), golden["q8k_q"])


def test_q8_0_closed_form(oracle):
    rng = np.random.default_rng(5)
    x = (rng.standard_normal(32 * 500) * 0.02).astype(np.float32)
    q = oracle.quantize(Q8_0, x).reshape(-1, 34)
    xb = x.reshape(-1, 32)
    amax = np.max(np.abs(xb), axis=1)
    d = (amax / np.float32(127)).astype(np.float32)
    assert np.array_equal(q[:, :2].copy().view(np.float16)[:, 0], d.astype(np.float16))
    inv = np.where(d != 0, np.float32(1) / d, np.float32(0)).astype(np.float32)
    scaled = (xb * inv[:, None]).astype(np.float32)
    want = np.where(scaled >= 0, np.floor(scaled + np.float32(0.5)), np.ceil(scaled - np.float32(0.5)))  # half away
    assert np.array_equal(q[:, 2:].view(np.int8), want.astype(np.int8))
    # |x - deq| <= d/2 (+ fp16 rounding of d)
    deq = oracle.dequantize(Q8_0, q.reshape(-1)).reshape(-1, 32)
    assert np.all(np.abs(deq - xb) <= (d[:, None] * 0.5 + amax[:, None] * 1e-3 + 1e-12))


def test_mxfp4_brute_force(oracle):
    rng = np.random.default_rng(6)
    x = (rng.standard_normal(32 * 400) * 0.02).astype(np.float32)
    x[:32] = 0
    q = oracle.quantize(MXFP4, x).reshape(-1, 17)
    xb = x.reshape(-1, 32)
    amax = np.max(np.abs(xb), axis=1)
    e = np.where(amax > 0, np.floor(np.log2(np.maximum(amax, 1e-38).astype(np.float64))) - 2 + 127, 0).astype(np.int64)
    assert np.array_equal(q[:, 0].astype(np.int64), e)
    d = (2.0 ** (e - 128.0)).astype(np.float32)
    cand = MXFP4_TABLE[None, None, :] * d[:, None, None]
    err = np.abs(cand - xb[:, :, None]).astype(np.float32)
    best = np.argmin(err, axis=2)          # first minimum wins, like the reference loop
    lo, hi = q[:, 1:] & 0x0F, q[:, 1:] >> 4
    assert np.array_equal(lo, best[:, :16])
    assert np.array_equal(hi, best[:, 16:])


def test_q4_k_invariants(oracle):
    rng = np.random.default_rng(7)
    x = (rng.standard_normal(256 * 300) * 0.02).astype(np.float32)
    q = oracle.quantize(Q4_K, x)
    deq = oracle.dequantize(Q4_K, q)
    rms = np.sqrt(np.mean((deq - x) ** 2)) / 0.02
    assert 0.05 < rms < 0.09          # measured 0.071 for the reference quantizer on N(0, 0.02)
    # re-quantising the dequantised values reproduces the same values (fixed point of the grid)
    deq2 = oracle.dequantize(Q4_K, oracle.quantize(Q4_K, deq))
    assert np.sqrt(np.mean((deq2 - deq) ** 2)) / 0.02 < 0.02
    # constant block: scale 0 -> all quants 0, value carried by the min
    c = np.full(256, -0.37, dtype=np.float32)
    dc = oracle.dequantize(Q4_K, oracle.quantize(Q4_K, c))
    assert np.allclose(dc, -0.37, rtol=2e-3)


def test_matches_reference_build(oracle, reference):
    rng = np.random.default_rng(8)
    for name, t in T.items():
        x = (rng.standard_normal(256 * 2000) * 0.02).astype(np.float32)
        x[1000:1256] *= 50
        assert np.array_equal(oracle.quantize(t, x), reference.quantize(t, x)), name
    xa = rng.standard_normal(256 * 50).astype(np.float32)
    assert np.array_equal(oracle.quantize_q8_K(xa), reference.quantize_q8_K(xa))


ALL_BASELINE_WEIGHTS = [(c, t) for c in ("cfg1", "cfg2", "cfg3", "cfg4", "cfg5") for t in getattr(inputs, c.upper())]


@pytest.mark.parametrize("cfg_name,tname", ALL_BASELINE_WEIGHTS)
def test_baseline_weight_digests(oracle, golden, cfg_name, tname):
    """SHA-256 of the reference-quantized bytes of the seeded BASELINE weights, every config at its full shape (the
    digests were written from the reference's own quantizers by tests/golden/make_golden.py): the oracle's quantizers
    produce the same bytes, so the GPU tests below them run on reference-quantized weights."""
    fmt, N, K = getattr(inputs, cfg_name.upper())[tname]
    tag = f"{cfg_name}.{tname}"
    q = oracle.quantize(T[fmt], inputs.weights(tag, N * K))
    got = np.frombuffer(hashlib.sha256(q.tobytes()).digest(), dtype=np.uint8)
    assert np.array_equal(got, golden[f"sha_{tag}"])
