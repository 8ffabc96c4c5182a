"""Scalar helpers of the oracle: fp16 <-> fp32 and E8M0, pinned by exhaustive enumeration
against numpy's IEEE binary16 and the closed form (reference: ggml-impl.h:378-425, :471-489)."""
import numpy as np


def test_fp16_to_fp32_all_codes(oracle):
    codes = np.arange(65536, dtype=np.uint16)
    mine = np.array([oracle.lib.tso_fp16_to_fp32(int(c)) for c in codes], dtype=np.float32)
    want = codes.view(np.float16).astype(np.float32)
    nan = np.isnan(want)
    assert np.array_equal(mine.view(np.uint32)[~nan], want.view(np.uint32)[~nan])
    assert np.all(np.isnan(mine[nan]))


def test_fp32_to_fp16_round_to_nearest_even(oracle):
    rng = np.random.default_rng(1)
    parts = [rng.standard_normal(50000).astype(np.float32) * np.float32(s)
             for s in (1e-8, 1e-6, 1e-4, 1e-2, 1, 100, 7e4)]
    halves = np.arange(65536, dtype=np.uint16).view(np.float16).astype(np.float32)
    halves = halves[~np.isnan(halves)]
    # every midpoint between adjacent halves (ties) and its neighbours
    pos = np.sort(halves[halves >= 0])
    mids = ((pos[:-1].astype(np.float64) + pos[1:].astype(np.float64)) / 2).astype(np.float32)
    mids = mids[np.isfinite(mids)]
    edge = np.array([65519.99, 65520, 65504, 65536, 1e9, -1e9, np.inf, -np.inf, 2.9802322e-8, 2.99e-8, 0.0, -0.0],
                    dtype=np.float32)
    xs = np.concatenate(parts + [halves, mids, np.nextafter(mids, np.float32(0)), np.nextafter(mids, np.float32(1e9)),
                                 -mids, edge])
    mine = np.array([oracle.lib.tso_fp32_to_fp16(float(v)) for v in xs], dtype=np.uint16)
    with np.errstate(over="ignore"):
        want = xs.astype(np.float16).view(np.uint16)
    assert np.array_equal(mine, want)
    assert oracle.lib.tso_fp32_to_fp16(float("nan")) & 0x7FFF == 0x7E00


def test_fp16_helpers_match_reference_build(oracle, reference):
    codes = np.arange(65536, dtype=np.uint16)
    a = np.array([oracle.lib.tso_fp16_to_fp32(int(c)) for c in codes], dtype=np.float32)
    b = np.array([reference.lib.ref_fp16_to_fp32(int(c)) for c in codes], dtype=np.float32)
    ok = ~np.isnan(b)
    assert np.array_equal(a.view(np.uint32)[ok], b.view(np.uint32)[ok])
    rng = np.random.default_rng(2)
    xs = np.concatenate([rng.standard_normal(40000).astype(np.float32) * np.float32(s) for s in (1e-7, 1e-3, 1, 3e4)])
    m = np.array([oracle.lib.tso_fp32_to_fp16(float(v)) for v in xs], dtype=np.uint16)
    r = np.array([reference.lib.ref_fp32_to_fp16(float(v)) for v in xs], dtype=np.uint16)
    assert np.array_equal(m, r)


def test_e8m0_half_scale_closed_form(oracle):
    for e in range(256):
        got = np.float32(oracle.lib.tso_e8m0_to_fp32_half(e))
        if e < 255:
            want = np.float32(2.0 ** (e - 128)) if e >= 2 else np.array([0x00200000 << e], dtype=np.uint32).view(np.float32)[0]
            assert got.view(np.uint32) == np.float32(want).view(np.uint32), e
        # 2^(e-128) exactly, including the two subnormal codes
        if e < 255:
            assert float(got) == 2.0 ** (e - 128)


def test_row_size_table(oracle):
    assert oracle.row_size(8, 2560) == 80 * 34
    assert oracle.row_size(12, 4096) == 16 * 144
    assert oracle.row_size(39, 2880) == 90 * 17
    assert oracle.row_size(12, 4000) == 0      # not a block multiple
    assert oracle.row_size(8, 0) == 0
    assert oracle.row_size(99, 256) == 0
