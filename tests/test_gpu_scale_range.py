"""GPU parity: matmul over block scales far from those of a trained model.

The reference dequantizes in fp32 and is exact for every scale (ManagedQuantizedOps.cs:411-427 Q8_0, :447-479 Q4_K,
:579-598 MXFP4 with E8M0ToFp32Half :678-682).  Here the single-row kernels (GEMV) apply block scales in fp32 and are
held to the same: every E8M0 code, fp16 scales from the smallest subnormal to the largest finite value.  The matrix-core
kernels with fp16 operands hold a weight as fp16(weight * 2^10): exact from the smallest scale up to a per-format limit
(Q8_0 |d| < 0.5, Q4_K |d|, |dmin| <= 2^-4, MXFP4 codes 94 .. 130: weights of magnitude 32 and more are outside), and a
column that holds a scale beyond it must come back as NaN, never as a wrong number.  MXFP4 launches on the block-scaled
matrix instruction (128- and 256-row tiles) take every code but 255.

Reference value: fp64 product of the bit-exact dequantized weights (tso_matmul_f64).  Bars: the path's own
max_j |y - ref| / ||ref row||_2 <= 1e-3, and per column |y_j - ref_j| <= 1e-3 ||w_j||_2 ||x||_2, which a column of
small scale next to columns of large scale does not pass by being negligible.
"""
import numpy as np
import pytest

import inputs
from oracle.oracle import Q8_0, Q4_K, MXFP4

pytestmark = pytest.mark.gpu


def f16_bytes(v):
    return np.asarray(v, dtype=np.float16).view(np.uint8).reshape(-1, 2)


def mxfp4_rows(N, K, codes, rng):
    """codes: [N, K / 32] E8M0 bytes; random E2M1 nibbles"""
    nb = N * (K // 32)
    raw = rng.integers(0, 256, size=(nb, 17), dtype=np.uint8)
    raw[:, 0] = np.asarray(codes, dtype=np.uint8).reshape(-1)
    return raw.reshape(-1)


def q8_0_rows(N, K, d, rng):
    """d: [N, K / 32] scales (rounded to fp16); random int8 quants"""
    nb = N * (K // 32)
    raw = rng.integers(0, 256, size=(nb, 34), dtype=np.uint8)
    raw[:, 0:2] = f16_bytes(np.asarray(d).reshape(-1))
    return raw.reshape(-1)


def q4_k_rows(N, K, d, dmin, rng):
    """d, dmin: [N, K / 256]; random 6-bit scales / mins and nibbles"""
    nb = N * (K // 256)
    raw = rng.integers(0, 256, size=(nb, 144), dtype=np.uint8)
    raw[:, 0:2] = f16_bytes(np.asarray(d).reshape(-1))
    raw[:, 2:4] = f16_bytes(np.asarray(dmin).reshape(-1))
    return raw.reshape(-1)


def run(hip, t, raw, N, K, x):
    import torch
    from tensorsharp_amd import QuantizedWeight
    y = hip.LinearForward(torch.from_numpy(np.ascontiguousarray(x)).cuda(), QuantizedWeight(torch.from_numpy(raw).cuda(), t, K, N))
    torch.cuda.synchronize()
    return y.cpu().numpy()


def check_columns(oracle, t, raw, N, K, x, y, tag):
    ref = oracle.matmul_f64(t, raw, N, K, x)
    assert np.all(np.isfinite(ref)), tag
    assert np.all(np.isfinite(y)), (tag, "non-finite columns", np.flatnonzero(~np.isfinite(y).all(axis=0))[:8])
    assert inputs.row_l2_err(y, ref) <= 1e-3, (tag, inputs.row_l2_err(y, ref))
    w = oracle.dequantize(t, raw, N * K).reshape(N, K).astype(np.float64)
    bound = 1e-3 * np.linalg.norm(x.astype(np.float64), axis=1)[:, None] * np.linalg.norm(w, axis=1)[None, :]
    worst = float(np.max(np.abs(y - ref) / np.maximum(bound, 1e-300)))
    assert worst <= 1.0, (tag, "per-column error / bound", worst)


# rows that reach: the GEMV, the 32-row register-resident kernel, 128-row tiles, 256-row tiles
ROWS = [1, 3, 8, 100, 160, 300]


@pytest.mark.parametrize("M", ROWS)
def test_mxfp4_codes_per_row(hip, oracle, M):
    """Every weight row has its own block exponent.  Single rows: codes 20 .. 250 (below, fp32 results are subnormal in
    the reference too).  Matrix-core kernels with fp16 operands: the whole window 94 .. 130."""
    rng = np.random.default_rng(9100 + M)
    N, K = 512, 1024
    lo, hi = (20, 250) if M <= 3 else (94, 130)
    row_code = rng.integers(lo, hi + 1, N)
    row_code[:4] = [lo, hi, lo + 1, hi - 1]
    codes = np.repeat(row_code[:, None], K // 32, axis=1)
    raw = mxfp4_rows(N, K, codes, rng)
    x = (rng.standard_normal((M, K)) * (2.0 ** -12 if M <= 3 else 1.0)).astype(np.float32)
    check_columns(oracle, MXFP4, raw, N, K, x, run(hip, MXFP4, raw, N, K, x), ("mxfp4", M))


@pytest.mark.parametrize("M", ROWS)
def test_mxfp4_codes_per_block(hip, oracle, M):
    """Exponents differ from block to block inside a row (window of the fp16 operands; single rows: 60 .. 190)."""
    rng = np.random.default_rng(9200 + M)
    N, K = 384, 2048
    lo, hi = (60, 190) if M <= 3 else (94, 130)
    codes = rng.integers(lo, hi + 1, (N, K // 32))
    raw = mxfp4_rows(N, K, codes, rng)
    x = rng.standard_normal((M, K)).astype(np.float32)
    check_columns(oracle, MXFP4, raw, N, K, x, run(hip, MXFP4, raw, N, K, x), ("mxfp4", M))


@pytest.mark.parametrize("M,N", [(600, 2048), (2048, 8192)])
def test_mxfp4_block_scaled_tiles_take_every_code_but_255(hip, oracle, M, N):
    """Plain launches of 128-row (600 x 2048) and 256-row (2048 x 8192) tiles run on the block-scaled instruction: the
    hardware applies the E8M0 exponent, so codes 20 .. 230 are all exact (activations scaled so that fp32 results stay
    finite and normal)."""
    rng = np.random.default_rng(9300 + M)
    K = 1024
    row_code = rng.integers(20, 231, N)
    codes = np.repeat(row_code[:, None], K // 32, axis=1)
    raw = mxfp4_rows(N, K, codes, rng)
    x = (rng.standard_normal((M, K)) * 2.0 ** -8).astype(np.float32)
    rows = np.arange(0, M, 37)
    y = run(hip, MXFP4, raw, N, K, x)
    check_columns(oracle, MXFP4, raw, N, K, x[rows], y[rows], ("mxfp4 block-scaled", M))


@pytest.mark.parametrize("M", ROWS)
def test_q8_0_scales_from_smallest_subnormal_up(hip, oracle, M):
    """fp16 d from 2^-24 (the smallest subnormal) to just under 0.5 per row (a quant of -128 times 0.5 * 2^10 would leave
    fp16), both signs; single rows up to 60000."""
    rng = np.random.default_rng(9400 + M)
    N, K = 512, 1024
    top = 60000.0 if M <= 3 else 0.4997
    d_row = np.exp2(rng.uniform(-24, np.log2(top), N)) * rng.choice([-1.0, 1.0], N)
    d_row[:4] = [2.0 ** -24, top, -(2.0 ** -24), 3 * 2.0 ** -24]
    raw = q8_0_rows(N, K, np.repeat(d_row[:, None], K // 32, axis=1), rng)
    x = (rng.standard_normal((M, K)) * (2.0 ** -6 if M <= 3 else 1.0)).astype(np.float32)
    check_columns(oracle, Q8_0, raw, N, K, x, run(hip, Q8_0, raw, N, K, x), ("q8_0", M))


@pytest.mark.parametrize("M", ROWS)
def test_q8_0_scales_per_block(hip, oracle, M):
    rng = np.random.default_rng(9500 + M)
    N, K = 320, 2048
    d = np.exp2(rng.uniform(-24, -1.01, (N, K // 32)))
    raw = q8_0_rows(N, K, d, rng)
    x = rng.standard_normal((M, K)).astype(np.float32)
    check_columns(oracle, Q8_0, raw, N, K, x, run(hip, Q8_0, raw, N, K, x), ("q8_0", M))


@pytest.mark.parametrize("M", ROWS)
def test_q4_k_scales_from_smallest_subnormal_up(hip, oracle, M):
    """fp16 d and dmin from 2^-24 to 2^-4 per row (single rows: up to 1000), random 6-bit scales and mins."""
    rng = np.random.default_rng(9600 + M)
    N, K = 512, 1024
    top = 1000.0 if M <= 3 else 2.0 ** -4
    d_row = np.exp2(rng.uniform(-24, np.log2(top), N))
    m_row = np.exp2(rng.uniform(-24, np.log2(top), N))
    d_row[:3], m_row[:3] = [2.0 ** -24, top, 2.0 ** -24], [2.0 ** -24, top, top]
    raw = q4_k_rows(N, K, np.repeat(d_row[:, None], K // 256, axis=1), np.repeat(m_row[:, None], K // 256, axis=1), rng)
    x = (rng.standard_normal((M, K)) * (2.0 ** -6 if M <= 3 else 1.0)).astype(np.float32)
    check_columns(oracle, Q4_K, raw, N, K, x, run(hip, Q4_K, raw, N, K, x), ("q4_k", M))


@pytest.mark.parametrize("name", ["mxfp4", "q8_0", "q4_k"])
@pytest.mark.parametrize("M", [8, 100, 160, 300])
def test_scale_beyond_the_fp16_operands_gives_nan_not_a_wrong_number(hip, oracle, name, M):
    """One block of a few columns holds a scale the fp16 operands cannot carry: exactly those columns are NaN (on every
    row), all others meet the bar."""
    rng = np.random.default_rng(9700 + M)
    N, K = 640, 1024
    bad_cols = [0, 31, 32, 257, 639]
    if name == "mxfp4":
        t = MXFP4
        codes = np.full((N, K // 32), 118)
        for i, c in enumerate(bad_cols):
            codes[c, (7 * i) % (K // 32)] = [140, 93, 200, 3, 131][i]
        raw = mxfp4_rows(N, K, codes, rng)
    elif name == "q8_0":
        t = Q8_0
        d = np.full((N, K // 32), 1e-3)
        for i, c in enumerate(bad_cols):
            d[c, (7 * i) % (K // 32)] = [0.6, 8.0, 60000.0, -0.75, 0.5005][i]
        raw = q8_0_rows(N, K, d, rng)
    else:
        t = Q4_K
        d = np.full((N, K // 256), 1e-3)
        dmin = np.full((N, K // 256), 1e-3)
        for i, c in enumerate(bad_cols):
            (d if i % 2 == 0 else dmin)[c, i % (K // 256)] = [0.07, 0.5, 100.0, 0.0626, 30000.0][i]
        raw = q4_k_rows(N, K, d, dmin, rng)
    x = rng.standard_normal((M, K)).astype(np.float32)
    y = run(hip, t, raw, N, K, x)
    assert np.all(np.isnan(y[:, bad_cols])), (name, M, np.isnan(y[:, bad_cols]).mean(axis=0))
    good = np.setdiff1d(np.arange(N), bad_cols)
    ref = oracle.matmul_f64(t, raw, N, K, x)
    assert np.all(np.isfinite(y[:, good]))
    assert inputs.row_l2_err(y[:, good], ref[:, good]) <= 1e-3


def test_single_rows_take_every_mxfp4_code(hip, oracle):
    """GEMV with code 255 (2^127 in ggml's table, ggml-impl.h:471-489; finite in fp32 only for the table values 0 and
    +-1, so that row holds no others), code 251 (the largest whose every value is finite) and codes 0 and 1 (subnormal
    patterns)."""
    rng = np.random.default_rng(9800)
    N, K = 256, 512
    codes = np.full((N, K // 32), 127)
    codes[0, :] = 255
    codes[1, :] = 251
    codes[2, :] = 0
    codes[3, :] = 1
    raw = mxfp4_rows(N, K, codes, rng).reshape(-1, 17)
    nib = np.array([0, 1, 9], np.uint8)[rng.integers(0, 3, (K // 32, 16, 2))]
    raw[:K // 32, 1:] = nib[:, :, 0] | (nib[:, :, 1] << 4)
    raw = raw.reshape(-1)
    x = np.zeros((1, K), np.float32)
    x[0, ::32] = 2.0 ** -20                     # one activation per block keeps 12 * 2^127 * x finite
    y = run(hip, MXFP4, raw, N, K, x)
    ref = oracle.matmul_f64(MXFP4, raw, N, K, x)
    big = [0, 1]
    assert np.all(np.isfinite(y[:, big]))
    assert np.allclose(y[:, big], ref[:, big], rtol=1e-6, atol=0.0)
    rest = np.arange(4, N)
    assert np.allclose(y[:, rest], ref[:, rest], rtol=1e-5, atol=1e-12)
    # codes 0 and 1: results are fp32 subnormals (2^-128 * 12 * 2^-20 * 16 blocks); exact to the subnormal grid
    assert np.all(np.abs(y[:, [2, 3]] - ref[:, [2, 3]]) <= 2.0 ** -148)


@pytest.mark.parametrize("T", [1, 40])
def test_moe_expert_stage_with_spread_exponents(hip, oracle, T):
    """The GPT-OSS expert stage with block exponents 100 .. 126 per weight row: one token (expert-indirect GEMV) and a
    batch (block-scaled expert tiles)."""
    import torch
    rng = np.random.default_rng(9900 + T)
    E, k, H, F = 8, 2, 512, 256
    def stack(rows, cols):
        codes = np.repeat(rng.integers(100, 127, E * rows)[:, None], cols // 32, axis=1)
        return mxfp4_rows(E * rows, cols, codes, rng)
    gu_w, dn_w = stack(2 * F, H), stack(H, F)
    gu_scale = 2.0 ** -6
    hidden = (rng.standard_normal((T, H)) * gu_scale).astype(np.float32)
    gu_b = (rng.standard_normal((E, 2 * F)) * 0.1).astype(np.float32)
    dn_b = (rng.standard_normal((E, H)) * 0.1).astype(np.float32)
    ids = np.stack([rng.permutation(E)[:k] for _ in range(T)]).astype(np.int32)
    wts = rng.uniform(0.2, 0.8, (T, k)).astype(np.float32)
    ref = oracle.moe_forward(MXFP4, gu_w, gu_b, dn_w, dn_b, E, H, F, hidden, ids, wts)
    out = hip.MoEExpertsGptOssForward(torch.from_numpy(hidden).cuda(), torch.from_numpy(ids).cuda(), torch.from_numpy(wts).cuda(),
                                      torch.from_numpy(gu_w).cuda(), torch.from_numpy(gu_b).cuda(), torch.from_numpy(dn_w).cuda(),
                                      torch.from_numpy(dn_b).cuda(), MXFP4, E, H, F)
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    assert np.all(np.isfinite(got))
    assert inputs.row_l2_err(got, ref) <= 1e-3, inputs.row_l2_err(got, ref)
