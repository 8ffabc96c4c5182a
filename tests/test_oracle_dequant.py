"""Dequantizers of the oracle (restating ManagedQuantizedOps.cs:411-427, :447-479, :579-598)."""
import numpy as np

from oracle.oracle import Q8_0, Q4_K, MXFP4

T = {"q8_0": Q8_0, "q4_k": Q4_K, "mxfp4": MXFP4}
MXFP4_TABLE = np.array([0, 1, 2, 3, 4, 6, 8, 12, 0, -1, -2, -3, -4, -6, -8, -12], dtype=np.float32)


def test_reference_unit_test_vectors(oracle, golden):
    # InferenceWeb.Tests/ManagedQuantizedOpsTests.cs:29-45 and :47-68
    for name in ("q8_0", "q4_k"):
        y = oracle.dequantize(T[name], golden[f"ref_tests_{name}_raw"])
        idx = golden[f"ref_tests_{name}_expect_idx"]
        np.testing.assert_array_equal(y[idx], golden[f"ref_tests_{name}_expect_val"])
        rest = np.ones(y.size, bool)
        rest[idx] = False
        if name == "q8_0":
            assert np.all(y[rest] == 0)


def test_golden_blocks_bit_exact(oracle, golden):
    for name, t in T.items():
        y = oracle.dequantize(t, golden[f"blocks_{name}_q"])
        want = golden[f"blocks_{name}_deq"]
        assert np.array_equal(y.view(np.uint32), want.view(np.uint32)), name


def test_q8_0_closed_form_all_scales(oracle):
    # every fp16 scale code x a sweep of int8 values: y = q * float(d), one exact fp32 product
    codes = np.arange(65536, dtype=np.uint16)
    raw = np.zeros((65536, 34), dtype=np.uint8)
    raw[:, 0] = codes & 0xFF
    raw[:, 1] = codes >> 8
    q = ((np.arange(32)[None, :] * 37 + codes[:, None] * 11) % 256).astype(np.uint8)
    raw[:, 2:] = q
    y = oracle.dequantize(Q8_0, raw.reshape(-1)).reshape(65536, 32)
    with np.errstate(invalid="ignore", over="ignore"):
        want = q.view(np.int8).astype(np.float32) * codes.view(np.float16).astype(np.float32)[:, None]
    ok = ~np.isnan(want)
    assert np.array_equal(y.view(np.uint32)[ok], want.view(np.uint32)[ok])


def _scale_min(j, p):
    if j < 4:
        return p[:, j] & 63, p[:, j + 4] & 63
    return (p[:, j + 4] & 0x0F) | ((p[:, j - 4] >> 6) << 4), (p[:, j + 4] >> 4) | ((p[:, j] >> 6) << 4)


def test_q4_k_closed_form_random_bytes(oracle):
    # independent numpy restatement: y = (d*sc)*q - (dmin*m), separately rounded fp32 ops
    rng = np.random.default_rng(3)
    nb = 4096
    raw = rng.integers(0, 256, size=(nb, 144), dtype=np.uint8)
    # keep d/dmin finite
    raw[:, 1] &= 0x7B
    raw[:, 3] &= 0x7B
    y = oracle.dequantize(Q4_K, raw.reshape(-1)).reshape(nb, 256)
    d = raw[:, 0:2].copy().view(np.float16).astype(np.float32)[:, 0]
    dmin = raw[:, 2:4].copy().view(np.float16).astype(np.float32)[:, 0]
    p = raw[:, 4:16].astype(np.uint32)
    qs = raw[:, 16:]
    want = np.empty((nb, 256), dtype=np.float32)
    for g in range(4):
        sc1, m1 = _scale_min(2 * g, p)
        sc2, m2 = _scale_min(2 * g + 1, p)
        d1 = (d * sc1.astype(np.float32)).astype(np.float32)[:, None]
        d2 = (d * sc2.astype(np.float32)).astype(np.float32)[:, None]
        o1 = (dmin * m1.astype(np.float32)).astype(np.float32)[:, None]
        o2 = (dmin * m2.astype(np.float32)).astype(np.float32)[:, None]
        lo = (qs[:, 32 * g:32 * g + 32] & 0x0F).astype(np.float32)
        hi = (qs[:, 32 * g:32 * g + 32] >> 4).astype(np.float32)
        want[:, 64 * g:64 * g + 32] = (d1 * lo).astype(np.float32) - o1
        want[:, 64 * g + 32:64 * g + 64] = (d2 * hi).astype(np.float32) - o2
    assert np.array_equal(y.view(np.uint32), want.view(np.uint32))


def test_mxfp4_closed_form_all_codes(oracle):
    # all 256 exponent codes x all 256 quant bytes: value = table[nibble] * 2^(e-128)
    raw = np.zeros((256, 16, 17), dtype=np.uint8)
    raw[:, :, 0] = np.arange(256, dtype=np.uint8)[:, None]
    raw[:, :, 1:] = np.arange(256, dtype=np.uint8).reshape(16, 16)[None]
    y = oracle.dequantize(MXFP4, raw.reshape(-1)).reshape(256, 16, 32)
    e = np.arange(256)
    bits = np.where(e < 2, 0x00200000 << np.minimum(e, 1), (np.maximum(e, 1) - 1) << 23).astype(np.uint32)
    d = bits.view(np.float32)[:, None, None]
    q = raw[:, :, 1:]
    want = np.concatenate([d * MXFP4_TABLE[q & 0x0F], d * MXFP4_TABLE[q >> 4]], axis=2).astype(np.float32)
    ok = ~np.isnan(want)
    assert np.array_equal(y.view(np.uint32)[ok], want.view(np.uint32)[ok])
    # spot value: e=127 -> d=0.5, nibble 7 -> 12*0.5
    blk = np.zeros(17, dtype=np.uint8)
    blk[0] = 127
    blk[1] = 0x97   # low nibble 7 -> +12, high nibble 9 -> -1
    v = oracle.dequantize(MXFP4, blk)
    assert v[0] == 6.0 and v[16] == -0.5


def test_matches_reference_build_on_random_bytes(oracle, reference):
    rng = np.random.default_rng(4)
    for name, t in T.items():
        bb = {"q8_0": 34, "q4_k": 144, "mxfp4": 17}[name]
        raw = rng.integers(0, 256, size=bb * 3000, dtype=np.uint8)
        a = oracle.dequantize(t, raw)
        b = reference.dequantize(t, raw)
        ok = ~np.isnan(b)
        assert np.array_equal(a.view(np.uint32)[ok], b.view(np.uint32)[ok]), name


def test_error_codes(oracle):
    import ctypes as C
    buf = np.zeros(64, dtype=np.uint8)
    out = np.zeros(64, dtype=np.float32)
    f32p = C.POINTER(C.c_float)
    assert oracle.lib.tso_dequantize(8, None, 32, out.ctypes.data_as(f32p)) == -1
    assert oracle.lib.tso_dequantize(77, C.c_void_p(buf.ctypes.data), 32, out.ctypes.data_as(f32p)) == -2
    assert oracle.lib.tso_dequantize(8, C.c_void_p(buf.ctypes.data), 33, out.ctypes.data_as(f32p)) == -1
    assert oracle.lib.tso_dequantize(8, C.c_void_p(buf.ctypes.data), 0, out.ctypes.data_as(f32p)) == 0


# ---- formats beyond the three matmul formats (ManagedQuantizedOps.cs:268-409, :481-577) -------------------
from oracle.oracle import MORE_TYPES, BLOCK, Q4_0, Q4_1, Q5_0, Q5_1, Q5_K, Q6_K, IQ4_NL, F16, BF16  # noqa: E402
import os  # noqa: E402
import pytest  # noqa: E402


@pytest.fixture(scope="module")
def formats():
    return np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "formats.npz"))


@pytest.mark.parametrize("name", sorted(MORE_TYPES))
def test_more_formats_match_the_reference_build(oracle, formats, name):
    # known answers written by the reference's own dequantizers (tests/golden/make_golden_formats.py)
    t = MORE_TYPES[name]
    for q, want in ((formats[f"{name}_q"], formats[f"{name}_deq"]), (formats[f"{name}_rq"], formats[f"{name}_rdeq"])):
        y = oracle.dequantize(t, q)
        assert np.array_equal(y.view(np.uint32), want.view(np.uint32)), name


def _f16(raw2):
    return np.ascontiguousarray(raw2).view(np.float16).astype(np.float64)[:, 0]


def test_q6_k_closed_form(oracle):
    # every value is d * scale * (q - 32) with an 11-bit d, an 8-bit scale and a 6-bit q: exact in fp32, so an
    # fp64 evaluation of the layout (ggml-common.h block_q6_K) must agree to the bit
    rng = np.random.default_rng(5)
    nb = 2048
    raw = rng.integers(0, 256, size=(nb, 210), dtype=np.uint8)
    raw[:, 209] &= 0x7B
    y = oracle.dequantize(Q6_K, raw.reshape(-1)).reshape(nb, 256)
    d = _f16(raw[:, 208:210])
    sc = raw[:, 192:208].view(np.int8).astype(np.float64)
    want = np.empty((nb, 256))
    for e in range(256):
        half, r = divmod(e, 128)
        grp, l = divmod(r, 32)
        qlb = raw[:, 64 * half + 32 * (grp & 1) + l]
        nib = (qlb >> 4) if grp >= 2 else (qlb & 0x0F)
        hi = (raw[:, 128 + 32 * half + l] >> (2 * grp)) & 3
        q = (nib | (hi << 4)).astype(np.float64) - 32
        want[:, e] = d * sc[:, 8 * half + 2 * grp + l // 16] * q
    assert np.array_equal(y.astype(np.float64), want)


def test_q5_k_closed_form(oracle):
    rng = np.random.default_rng(6)
    nb = 2048
    raw = rng.integers(0, 256, size=(nb, 176), dtype=np.uint8)
    raw[:, 1] &= 0x7B
    raw[:, 3] &= 0x7B
    y = oracle.dequantize(Q5_K, raw.reshape(-1)).reshape(nb, 256)
    d = _f16(raw[:, 0:2]).astype(np.float32)
    dmin = _f16(raw[:, 2:4]).astype(np.float32)
    p = raw[:, 4:16]
    want = np.empty((nb, 256), dtype=np.float32)
    for j in range(8):
        sc, mn = _scale_min(j, p)
        d1 = d * sc.astype(np.float32)
        m1 = dmin * mn.astype(np.float32)
        g, hi = divmod(j, 2)
        qb = raw[:, 48 + 32 * g:48 + 32 * g + 32]
        nib = (qb >> 4) if hi else (qb & 0x0F)
        bit = (raw[:, 16:48] >> j) & 1
        q = (nib + 16 * bit).astype(np.float32)
        want[:, 32 * j:32 * j + 32] = d1[:, None] * q - m1[:, None]
    assert np.array_equal(y.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("t,hdr,bias,has_min", [(Q4_0, 2, 8, False), (Q4_1, 4, 0, True), (Q5_0, 6, 16, False), (Q5_1, 8, 0, True)])
def test_legacy_32_blocks_closed_form(oracle, t, hdr, bias, has_min):
    rng = np.random.default_rng(7 + t)
    nb = 4096
    bb = BLOCK[t][1]
    raw = rng.integers(0, 256, size=(nb, bb), dtype=np.uint8)
    raw[:, 1] &= 0x7B
    if has_min:
        raw[:, 3] &= 0x7B
    y = oracle.dequantize(t, raw.reshape(-1)).reshape(nb, 32)
    d = _f16(raw[:, 0:2]).astype(np.float32)
    m = _f16(raw[:, 2:4]).astype(np.float32) if has_min else None
    qs = raw[:, hdr:hdr + 16]
    q = np.concatenate([qs & 0x0F, qs >> 4], axis=1).astype(np.int32)
    if t in (Q5_0, Q5_1):
        qh = raw[:, hdr - 4:hdr].copy().view(np.uint32)[:, 0]
        bits = (qh[:, None] >> np.arange(32)[None, :]) & 1
        q = q + 16 * bits.astype(np.int32)
    want = (q - bias).astype(np.float32) * d[:, None]
    if has_min:
        want = want + m[:, None]
    assert np.array_equal(y.view(np.uint32), want.astype(np.float32).view(np.uint32))


def test_iq4_nl_f16_bf16_closed_form(oracle):
    rng = np.random.default_rng(8)
    table = np.array([-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113], dtype=np.float32)
    raw = rng.integers(0, 256, size=(4096, 18), dtype=np.uint8)
    raw[:, 1] &= 0x7B
    y = oracle.dequantize(IQ4_NL, raw.reshape(-1)).reshape(-1, 32)
    d = _f16(raw[:, 0:2]).astype(np.float32)
    qs = raw[:, 2:]
    want = d[:, None] * table[np.concatenate([qs & 0x0F, qs >> 4], axis=1)]
    assert np.array_equal(y.view(np.uint32), want.view(np.uint32))
    # every fp16 / bf16 code
    codes = np.arange(65536, dtype=np.uint16)
    y = oracle.dequantize(F16, codes.view(np.uint8))
    want = codes.view(np.float16).astype(np.float32)
    ok = ~np.isnan(want)
    assert np.array_equal(y.view(np.uint32)[ok], want.view(np.uint32)[ok])
    y = oracle.dequantize(BF16, codes.view(np.uint8))
    assert np.array_equal(y.view(np.uint32), codes.astype(np.uint32) << 16)


def test_q8_1_closed_form_all_scales(oracle):
    # Q8_1 (ManagedQuantizedOps.cs:429-445): fp16 d at byte 0, the fp16 sum term at byte 2 is skipped, 32 int8 at byte 4.
    # ggml has no dequantizer for this activation format, so the pin is the closed form y = q * float(d) over every
    # scale code; filling the skipped bytes with a value that would change the result catches a wrong offset.
    from oracle.oracle import Q8_1
    codes = np.arange(65536, dtype=np.uint16)
    raw = np.zeros((65536, 36), dtype=np.uint8)
    raw[:, 0] = codes & 0xFF
    raw[:, 1] = codes >> 8
    raw[:, 2] = 0x55
    raw[:, 3] = 0x7B          # a large finite fp16 in the sum slot
    q = ((np.arange(32)[None, :] * 29 + codes[:, None] * 7) % 256).astype(np.uint8)
    raw[:, 4:] = q
    y = oracle.dequantize(Q8_1, raw.reshape(-1)).reshape(65536, 32)
    with np.errstate(invalid="ignore", over="ignore"):
        want = q.view(np.int8).astype(np.float32) * codes.view(np.float16).astype(np.float32)[:, None]
    ok = ~np.isnan(want)
    assert np.array_equal(y.view(np.uint32)[ok], want.view(np.uint32)[ok])
    assert oracle.row_size(Q8_1, 64) == 72
