"""GPU parity: prefill GEMM (M > 3) through the C ABI against the oracle.

Bar: max_j |y[m,j] - ref[m,j]| / ||ref[m,:]||_2 <= 1e-3 per output row, ref = fp64 product of the
bit-exact dequantised weights with the fp32 activations.  Operands are fp16 on the matrix cores
(fp32 accumulate), so the stricter max|delta|/rms(ref row) is held to 1e-2.
"""
import numpy as np
import pytest

import inputs
from oracle.oracle import Q8_0, Q4_K, MXFP4

pytestmark = pytest.mark.gpu
T = {"q8_0": Q8_0, "q4_k": Q4_K, "mxfp4": MXFP4}


def check(y, ref, tag=""):
    e1, e2 = inputs.row_l2_err(y, ref), inputs.rms_err(y, ref)
    assert e1 <= 1e-3, (tag, e1)
    assert e2 <= 1e-2, (tag, e2)
    return e1, e2


def run_device(hip, t, wq, N, K, x):
    import torch
    from tensorsharp_amd import QuantizedWeight
    y = hip.LinearForward(torch.from_numpy(np.ascontiguousarray(x)).cuda(), QuantizedWeight(torch.from_numpy(wq).cuda(), t, K, N))
    torch.cuda.synchronize()
    return y.cpu().numpy()


@pytest.mark.parametrize("name", ["q8_0", "q4_k", "mxfp4"])
@pytest.mark.parametrize("M,N,K", [(4, 128, 256), (64, 128, 512), (65, 130, 768), (128, 256, 1024), (200, 77, 2048),
                                   (7, 1000, 4096), (129, 384, 2560)])
def test_shapes(hip, oracle, name, M, N, K):
    if name == "q4_k" and K % 256:
        pytest.skip("K must be a multiple of 256 for Q4_K")
    rng = np.random.default_rng(M * 131 + N * 7 + K)
    wq = oracle.quantize(T[name], (rng.standard_normal(N * K) * 0.02).astype(np.float32))
    x = rng.standard_normal((M, K)).astype(np.float32)
    y = run_device(hip, T[name], wq, N, K, x)
    check(y, oracle.matmul_f64(T[name], wq, N, K, x), (name, M, N, K))


@pytest.mark.parametrize("name", ["q8_0", "mxfp4"])
def test_k_not_a_multiple_of_the_k_tile(hip, oracle, name):
    # K = 32 * odd: the last 64-wide k-tile holds one block only; rows are 2-byte / 1-byte aligned
    rng = np.random.default_rng(51)
    M, N, K = 33, 70, 32 * 45
    wq = oracle.quantize(T[name], (rng.standard_normal(N * K) * 0.02).astype(np.float32))
    x = rng.standard_normal((M, K)).astype(np.float32)
    check(run_device(hip, T[name], wq, N, K, x), oracle.matmul_f64(T[name], wq, N, K, x))


@pytest.mark.parametrize("name", ["q8_0", "q4_k", "mxfp4"])
def test_gemm_row_equals_gemv(hip, oracle, name):
    """The reference's own self-check (Gemma3Model.cs:601-622): batched rows vs single rows."""
    rng = np.random.default_rng(53)
    M, N, K = 16, 512, 1024
    wq = oracle.quantize(T[name], (rng.standard_normal(N * K) * 0.02).astype(np.float32))
    x = rng.standard_normal((M, K)).astype(np.float32)
    x[3] *= 1e4       # per-row scaling keeps every row inside fp16 range
    x[5] *= 1e-6
    x[7] = 0
    full = run_device(hip, T[name], wq, N, K, x)
    ref = oracle.matmul_f64(T[name], wq, N, K, x)
    check(full, ref)
    assert np.all(full[7] == 0)
    for m in (0, 3, 5):
        one = run_device(hip, T[name], wq, N, K, x[m:m + 1])
        assert inputs.row_l2_err(one, full[m:m + 1]) < 2e-4


def test_host_entry_prefill(hip, oracle):
    rng = np.random.default_rng(55)
    M, N, K = 40, 192, 512
    wq = oracle.quantize(Q4_K, (rng.standard_normal(N * K) * 0.02).astype(np.float32))
    x = rng.standard_normal((M, K)).astype(np.float32)
    out = np.empty((M, N), dtype=np.float32)
    hip.AddmmQuant(out, x, wq.ctypes.data, Q4_K, K, N, wq.size)
    check(out, oracle.matmul_f64(Q4_K, wq, N, K, x))
    hip.ClearHostBufferCache()


def sample_rows(M, always, count, seed):
    """`count` or more distinct rows of [0, M): the tile-boundary rows in `always` plus seeded random ones"""
    rng = np.random.default_rng(seed)
    rows = set(r for r in always if r < M)
    while len(rows) < count:
        rows.add(int(rng.integers(0, M)))
    return sorted(rows)


def test_config3_q4_k_prefill(hip, oracle):
    """BASELINE configs[2]: Q4_K, M=512, K=4096, N=14336.  The weight bytes are the reference quantizer's (the oracle's
    quantizer reproduces them: digest sha_cfg3.gate); 64 output rows are checked against the fp64 product."""
    fmt, N, K = inputs.CFG3["gate"]
    M = 512
    wq = oracle.quantize(T[fmt], inputs.weights("cfg3.gate", N * K))
    x = inputs.activations("cfg3.x", M, K)
    y = run_device(hip, T[fmt], wq, N, K, x)
    rows = sample_rows(M, [0, 1, 63, 64, 127, 128, 255, 256, 300, 511], 64, 3)
    ref = oracle.matmul_f64(T[fmt], wq, N, K, x[rows])
    e = check(y[rows], ref, "cfg3")
    print("cfg3 row-L2 err %.2e rms err %.2e over %d rows" % (e + (len(rows),)))
    assert np.all(np.isfinite(y))


@pytest.mark.parametrize("name,M", [("q4_k", 40), ("mxfp4", 64), ("q8_0", 9)])
def test_more_tiles_than_workgroups(hip, oracle, name, M):
    # few rows x very many columns: the persistent workgroups each walk over several tiles
    rng = np.random.default_rng(57 + M)
    N, K = 256 * 300 + 77, 256
    wq = oracle.quantize(T[name], (rng.standard_normal(N * K) * 0.02).astype(np.float32))
    x = rng.standard_normal((M, K)).astype(np.float32)
    y = run_device(hip, T[name], wq, N, K, x)
    check(y, oracle.matmul_f64(T[name], wq, N, K, x), (name, M))


@pytest.mark.parametrize("name", ["q8_0", "q4_k", "mxfp4"])
def test_tall_activations(hip, oracle, name):
    # M > 1024 takes the 256-row tiles; the last tile is ragged in both directions
    rng = np.random.default_rng(59)
    M, N, K = 1100, 300, 768
    wq = oracle.quantize(T[name], (rng.standard_normal(N * K) * 0.02).astype(np.float32))
    x = rng.standard_normal((M, K)).astype(np.float32)
    y = run_device(hip, T[name], wq, N, K, x)
    check(y, oracle.matmul_f64(T[name], wq, N, K, x), name)


@pytest.mark.parametrize("name,row_bytes", [("mxfp4", 17 * 3), ("q8_0", 34 * 3)])
@pytest.mark.parametrize("M", [8, 100])
def test_weight_view_at_odd_address(hip, oracle, name, row_bytes, M):
    # a sub-matrix that starts at row 1: its first byte is 1- or 2-byte aligned only
    import torch
    from tensorsharp_amd import QuantizedWeight
    rng = np.random.default_rng(61 + M)
    N, K = 301, 96
    wq = oracle.quantize(T[name], (rng.standard_normal(N * K) * 0.02).astype(np.float32))
    assert wq.size == N * row_bytes
    x = rng.standard_normal((M, K)).astype(np.float32)
    dev = torch.from_numpy(wq).cuda()
    sub = dev[row_bytes:]
    y = hip.LinearForward(torch.from_numpy(x).cuda(), QuantizedWeight(sub, T[name], K, N - 1))
    torch.cuda.synchronize()
    check(y.cpu().numpy(), oracle.matmul_f64(T[name], wq[row_bytes:], N - 1, K, x), (name, M))


@pytest.mark.parametrize("name,M,N,K", [
    ("mxfp4", 32, 5000, 2880),    # six k-tiles per wavefront, three raw buffers, half-filled last copy
    ("mxfp4", 17, 9001, 4096),    # eight k-tiles per wavefront, two raw buffers
    ("mxfp4", 5, 3000, 1024),     # two k-tiles per wavefront
    ("mxfp4", 31, 2000, 2048),    # four
    ("mxfp4", 9, 1500, 4160),     # K longer than one chunk of the register-resident kernel: two chunks, summed
    ("mxfp4", 30, 700, 8192 + 64),
    ("q4_k", 32, 9000, 2048),
    ("q4_k", 12, 14336, 4096),
    ("q4_k", 20, 1000, 4352),     # two chunks
    ("q4_k", 8, 4096, 14336),     # four chunks, few columns
    ("q4_k", 6, 333, 256),        # a single k-tile group: seven of the eight wavefronts have no K range
    ("q8_0", 32, 3000, 1024),
    ("q8_0", 11, 7000, 2048),
    ("q8_0", 25, 900, 2080),      # two chunks
    ("q8_0", 5, 300, 6176),       # four chunks, the last one a single block
    ("q8_0", 4, 40, 32),          # one block per row
])
def test_at_most_32_rows(hip, oracle, name, M, N, K):
    # M <= 32: the activations stay in registers and the wavefronts of a workgroup split K
    rng = np.random.default_rng(M * 17 + N + K)
    wq = oracle.quantize(T[name], (rng.standard_normal(N * K) * 0.02).astype(np.float32))
    x = rng.standard_normal((M, K)).astype(np.float32)
    y = run_device(hip, T[name], wq, N, K, x)
    check(y, oracle.matmul_f64(T[name], wq, N, K, x), (name, M, N, K))


# ---- Q6_K (the format Q4_K_M files use for the output matrix and some projections): matrix-core kernels only ----
def q6k_weight(N, K, seed):
    import torch
    from tensorsharp_amd import synth
    g = torch.Generator()
    g.manual_seed(seed)
    return synth.quantize_q6_k_simple(torch.randn((N, K), generator=g) * 0.02).numpy()


@pytest.mark.parametrize("M,N,K", [(1, 1000, 2048), (3, 333, 256), (4, 128, 256), (32, 3000, 2048), (17, 700, 4096),
                                   (1, 4096, 14336), (2, 600, 2304),
                                   (33, 130, 768), (64, 600, 1024), (65, 257, 2304), (128, 256, 1024), (200, 77, 2048),
                                   (1100, 300, 768)])
def test_q6_k_shapes(hip, oracle, M, N, K):
    from oracle.oracle import Q6_K
    rng = np.random.default_rng(M * 31 + N + K)
    wq = q6k_weight(N, K, M + N)
    x = rng.standard_normal((M, K)).astype(np.float32)
    y = run_device(hip, Q6_K, wq, N, K, x)
    check(y, oracle.matmul_f64(Q6_K, wq, N, K, x), ("q6_k", M, N, K))


@pytest.mark.parametrize("M", [2, 40, 150])
def test_q6_k_rows_two_bytes_off(hip, oracle, M):
    # K = 256 * odd and a view from row 1: rows start 2 bytes off a dword, and so does every second block
    import torch
    from tensorsharp_amd import QuantizedWeight
    from oracle.oracle import Q6_K
    rng = np.random.default_rng(73 + M)
    N, K = 200, 256 * 3
    wq = q6k_weight(N, K, 5)
    row_bytes = 210 * 3
    x = rng.standard_normal((M, K)).astype(np.float32)
    dev = torch.from_numpy(wq).cuda()
    y = hip.LinearForward(torch.from_numpy(x).cuda(), QuantizedWeight(dev[row_bytes:], Q6_K, K, N - 1))
    torch.cuda.synchronize()
    check(y.cpu().numpy(), oracle.matmul_f64(Q6_K, wq[row_bytes:], N - 1, K, x), ("q6_k view", M))


@pytest.mark.parametrize("name,M,N,K", [("mxfp4", 600, 300, 768), ("q4_k", 520, 1000, 1024), ("q8_0", 70, 500, 1088),
                                       ("mxfp4", 300, 17000, 512),
                                       # few tiles and a long K: K is cut into chunks whose sums a second kernel adds
                                       ("q8_0", 200, 300, 8192), ("q4_k", 600, 260, 8192), ("mxfp4", 1100, 300, 6144 + 64),
                                       # chunks of 12 and 16 k-tiles
                                       ("q4_k", 1024, 520, 2048), ("q8_0", 520, 600, 3072), ("q4_k", 700, 520, 3072)])
def test_128_row_tiles(hip, oracle, name, M, N, K):
    # row counts past the register-resident kernel's range: 128-row tiles, ragged last tile
    rng = np.random.default_rng(M + N + K)
    wq = oracle.quantize(T[name], (rng.standard_normal(N * K) * 0.02).astype(np.float32))
    x = rng.standard_normal((M, K)).astype(np.float32)
    y = run_device(hip, T[name], wq, N, K, x)
    check(y, oracle.matmul_f64(T[name], wq, N, K, x), (name, M, N, K))


# ---- plain MXFP4 launches of 128- / 256-row tiles: the block-scaled matrix instruction, activations as two MX fp6 terms ----
@pytest.mark.parametrize("M,N,K", [(300, 520, 32 * 33),      # odd block count: half of the last k-tile is past K
                                   (700, 1500, 2880),        # ragged last tile in both directions, 45 k-tiles
                                   (257, 300, 64),           # a single k-tile
                                   (1030, 264, 4096 + 32),
                                   (300, 264, 8192 + 64),    # rows beyond 8192: the 1024-thread conversion
                                   (384, 1500, 2880),        # few tiles: K chunks of 12 k-tiles, the last one of 9
                                   (640, 1100, 2880 - 32)])  # the same with half a k-tile at the end
def test_mxfp4_block_scaled_tiles(hip, oracle, M, N, K):
    rng = np.random.default_rng(M + 3 * N + K)
    wq = oracle.quantize(MXFP4, (rng.standard_normal(N * K) * 0.02).astype(np.float32))
    x = rng.standard_normal((M, K)).astype(np.float32)
    check(run_device(hip, MXFP4, wq, N, K, x), oracle.matmul_f64(MXFP4, wq, N, K, x), ("mx", M, N, K))


@pytest.mark.parametrize("M,N", [(600, 2100), (1024, 8448)])
def test_mxfp4_rows_longer_than_the_block_scaled_kernels_take(hip, oracle, M, N):
    # K > 32768: the activations stay fp16 and the launch runs the exchange-layout kernel (128-row tiles for the first
    # shape, 256-row tiles for the second), K cut into chunks
    rng = np.random.default_rng(900 + M)
    K = 32768 + 32 * 9
    wq = inputs.random_blocks("mxfp4", N, K, rng)
    x = rng.standard_normal((M, K)).astype(np.float32)
    y = run_device(hip, MXFP4, wq, N, K, x)
    rows = np.unique(np.concatenate([np.arange(0, M, 149), [M - 1]]))
    check(y[rows], oracle.matmul_f64(MXFP4, wq, N, K, x[rows]), ("mx long rows", M, N))


def test_mxfp4_block_scaled_256_row_tiles(hip, oracle):
    # more 128-row tiles than one round of workgroups: 256-row tiles; an odd block count and a ragged last column tile
    rng = np.random.default_rng(8)
    M, N, K = 1024, 8500, 32 * 35
    wq = inputs.random_blocks("mxfp4", N, K, rng)
    x = rng.standard_normal((M, K)).astype(np.float32)
    y = run_device(hip, MXFP4, wq, N, K, x)
    rows = np.unique(np.concatenate([np.arange(0, M, 41), [127, 128, 255, 256, 511, 767, 1023]]))
    check(y[rows], oracle.matmul_f64(MXFP4, wq, N, K, x[rows]), "mx 256-row tiles")


@pytest.mark.parametrize("K,M", [(256, 24), (1024, 24), (2048, 24), (2848, 17), (1024, 32), (3008, 31), (2880, 16)])
def test_mxfp4_block_scaled_register_resident_k_ranges(hip, oracle, K, M):
    """Small batch over a large weight with a short K: two, four and six k-tiles per wavefront of the register-resident
    kernel (K = 256 leaves most wavefronts without a k-tile; 2848 and 3008 end in half a k-tile).  Units of more than
    16 rows fetch their activations through LDS in two passes of 16 rows (17: a single row in the second pass),
    smaller ones load them directly."""
    import torch
    from tensorsharp_amd import QuantizedWeight
    rng = np.random.default_rng(K + M)
    N = (64 << 20) // K + 40
    wq = inputs.random_blocks("mxfp4", N, K, rng)
    x = rng.standard_normal((M, K)).astype(np.float32)
    y = hip.LinearForward(torch.from_numpy(x).cuda(), QuantizedWeight(torch.from_numpy(wq).cuda(), MXFP4, K, N))
    torch.cuda.synchronize()
    y = y.cpu().numpy()
    cols = np.unique(np.concatenate([[0, 31, 32, N - 1], rng.integers(0, N, 300)]))
    rb = K // 32 * 17
    sub = np.concatenate([wq[c * rb:(c + 1) * rb] for c in cols])
    check(y[:, cols], oracle.matmul_f64(MXFP4, sub, len(cols), K, x), ("mx register-resident", K))


def test_mxfp4_block_scaled_dynamic_range(hip, oracle):
    """Every 32-element block of the activations has its own magnitude (2^-40 .. 2^40), some blocks and rows are zero,
    single outliers sit in otherwise small blocks: the block exponents are absolute, so nothing saturates or vanishes."""
    rng = np.random.default_rng(5)
    M, N, K = 300, 260, 1024
    wq = oracle.quantize(MXFP4, (rng.standard_normal(N * K) * 0.02).astype(np.float32))
    x = rng.standard_normal((M, K)).astype(np.float32)
    mag = np.exp2(rng.integers(-40, 41, size=(M, K // 32))).astype(np.float32)
    x = (x.reshape(M, K // 32, 32) * mag[:, :, None]).reshape(M, K)
    x[:, 64:96] = 0.0
    x[7, :] = 0.0
    x[np.arange(M), rng.integers(0, K, size=M)] *= 1000.0
    y = run_device(hip, MXFP4, wq, N, K, x)
    assert np.isfinite(y).all()
    assert (y[7] == 0).all()
    check(y, oracle.matmul_f64(MXFP4, wq, N, K, x), "mx dynamic range")


def test_mxfp4_block_scaled_non_finite_rows(hip, oracle):
    """An inf or a NaN in a row makes that row of the result non-finite (its block's scale byte becomes NaN) and
    leaves the other rows alone."""
    rng = np.random.default_rng(6)
    M, N, K = 260, 256, 512
    wq = oracle.quantize(MXFP4, (rng.standard_normal(N * K) * 0.02).astype(np.float32))
    x = rng.standard_normal((M, K)).astype(np.float32)
    ref = oracle.matmul_f64(MXFP4, wq, N, K, x)
    x[3, 100] = np.inf
    x[200, 5] = np.nan
    y = run_device(hip, MXFP4, wq, N, K, x)
    assert not np.isfinite(y[3]).any() and not np.isfinite(y[200]).any()
    keep = np.ones(M, bool)
    keep[[3, 200]] = False
    check(y[keep], ref[keep], "mx rows beside non-finite ones")


@pytest.mark.parametrize("M", [9, 40])
def test_mxfp4_block_scaled_small_batch_large_weight(hip, oracle, M):
    """A small batch over a weight of 64 M elements or more takes the register-resident kernel on the block-scaled
    instruction (32-row units); two K chunks at this K.  Random valid blocks; the oracle checks 300 sampled columns."""
    import torch
    from tensorsharp_amd import QuantizedWeight
    rng = np.random.default_rng(M)
    N, K = 21000, 3200
    wq = inputs.random_blocks("mxfp4", N, K, rng)
    x = rng.standard_normal((M, K)).astype(np.float32)
    y = hip.LinearForward(torch.from_numpy(x).cuda(), QuantizedWeight(torch.from_numpy(wq).cuda(), MXFP4, K, N))
    torch.cuda.synchronize()
    y = y.cpu().numpy()
    cols = np.unique(np.concatenate([[0, 31, 32, N - 1], rng.integers(0, N, 300)]))
    rb = K // 32 * 17
    sub = np.concatenate([wq[c * rb:(c + 1) * rb] for c in cols])
    ref = oracle.matmul_f64(MXFP4, sub, len(cols), K, x)
    # the row norm of the full result scales the bound: a column subset has a smaller norm, which only tightens it
    check(y[:, cols], ref, ("mx small batch", M))


@pytest.mark.parametrize("M", [40, 48, 90, 130])
def test_mxfp4_block_scaled_small_batch_48_row_units(hip, oracle, M):
    """With K in one chunk (K <= 3072) a small batch over a large weight runs in 48-row units where they are at most two
    thirds as many as 32-row units (40, 48, 90 and 130 rows: 1, 1, 2 and 3 units instead of 2, 2, 3 and 5; the last unit
    of 130 holds 34 rows).  N is not a multiple of 32 and K not of 64."""
    import torch
    from tensorsharp_amd import QuantizedWeight
    rng = np.random.default_rng(100 + M)
    N, K = 24010, 2848
    wq = inputs.random_blocks("mxfp4", N, K, rng)
    x = rng.standard_normal((M, K)).astype(np.float32)
    y = hip.LinearForward(torch.from_numpy(x).cuda(), QuantizedWeight(torch.from_numpy(wq).cuda(), MXFP4, K, N))
    torch.cuda.synchronize()
    y = y.cpu().numpy()
    cols = np.unique(np.concatenate([[0, 15, 16, 31, 32, N - 1, N - 10], rng.integers(0, N, 300)]))
    rb = K // 32 * 17
    sub = np.concatenate([wq[c * rb:(c + 1) * rb] for c in cols])
    ref = oracle.matmul_f64(MXFP4, sub, len(cols), K, x)
    check(y[:, cols], ref, ("mx 48-row units", M))


def test_q6_k_128_row_tiles(hip, oracle):
    from oracle.oracle import Q6_K
    rng = np.random.default_rng(77)
    M, N, K = 300, 520, 1024
    wq = q6k_weight(N, K, 11)
    x = rng.standard_normal((M, K)).astype(np.float32)
    check(run_device(hip, Q6_K, wq, N, K, x), oracle.matmul_f64(Q6_K, wq, N, K, x), "q6_k 300")


# ---- the remaining block formats of the managed code (ManagedQuantizedOps.cs:40-59): matrix-core kernels only ----
@pytest.mark.parametrize("name", ["q4_0", "q4_1", "q5_0", "q5_1", "iq4_nl", "q5_k"])
@pytest.mark.parametrize("M,N,K", [(1, 700, 1024), (5, 130, 256), (32, 2000, 2304), (40, 300, 4352), (300, 520, 768),
                                   (1100, 260, 512)])
def test_more_formats_matmul(hip, oracle, name, M, N, K):
    from oracle.oracle import MORE_TYPES
    t = MORE_TYPES[name]
    rng = np.random.default_rng(M * 7 + N + K + t)
    wq = inputs.random_blocks(name, N, K, rng)
    x = rng.standard_normal((M, K)).astype(np.float32)
    y = run_device(hip, t, wq, N, K, x)
    check(y, oracle.matmul_f64(t, wq, N, K, x), (name, M, N, K))


@pytest.mark.parametrize("name", ["q4_0", "q4_1", "q5_0", "q5_1", "iq4_nl", "q5_k", "mxfp4"])
def test_256_row_tiles_of_the_other_formats(hip, oracle, name):
    # 1024 x 8448: more 128-row tiles than one round of workgroups, so the launcher takes 256-row tiles
    from oracle.oracle import MORE_TYPES
    M, N, K = 1024, 8448, 512
    t = MORE_TYPES[name] if name in MORE_TYPES else T[name]
    rng = np.random.default_rng(N + t)
    wq = inputs.random_blocks(name, N, K, rng) if name in MORE_TYPES else oracle.quantize(t, (rng.standard_normal(N * K) * 0.02).astype(np.float32))
    x = rng.standard_normal((M, K)).astype(np.float32)
    y = run_device(hip, t, wq, N, K, x)
    rows = np.unique(np.concatenate([np.arange(0, M, 37), [255, 256, 511, 767, 1023]]))
    check(y[rows], oracle.matmul_f64(t, wq, N, K, x[rows]), (name, M, N, K))


@pytest.mark.parametrize("name", ["q4_0", "q4_1", "q5_0", "q5_1", "iq4_nl"])
def test_small_batch_k_range_of_four_tiles(hip, oracle, name):
    # K = 1536: 24 k-tiles over eight wavefronts -> the register-resident kernel built for four k-tiles per wavefront
    from oracle.oracle import MORE_TYPES
    M, N, K = 16, 300, 1536
    t = MORE_TYPES[name]
    rng = np.random.default_rng(K + t)
    wq = inputs.random_blocks(name, N, K, rng)
    x = rng.standard_normal((M, K)).astype(np.float32)
    y = run_device(hip, t, wq, N, K, x)
    check(y, oracle.matmul_f64(t, wq, N, K, x), (name, M, N, K))


@pytest.mark.parametrize("name,row_bytes", [("q4_0", 18 * 3), ("q5_0", 22 * 3), ("q5_1", 24 * 5)])
def test_more_formats_rows_two_bytes_off(hip, oracle, name, row_bytes):
    import torch
    from tensorsharp_amd import QuantizedWeight
    from oracle.oracle import MORE_TYPES
    t = MORE_TYPES[name]
    rng = np.random.default_rng(91)
    K = 96 if name != "q5_1" else 160
    N = 150
    wq = inputs.random_blocks(name, N, K, rng)
    assert wq.size == N * row_bytes
    x = rng.standard_normal((12, K)).astype(np.float32)
    dev = torch.from_numpy(wq).cuda()
    y = hip.LinearForward(torch.from_numpy(x).cuda(), QuantizedWeight(dev[row_bytes:], t, K, N - 1))
    torch.cuda.synchronize()
    check(y.cpu().numpy(), oracle.matmul_f64(t, wq[row_bytes:], N - 1, K, x), (name, "view"))


@pytest.mark.parametrize("tname", ["up_q8", "up_q4", "down_q8", "down_q4"])
def test_config5_full_size(hip, oracle, tname):
    """BASELINE configs[4] at its full size: M = 2048, the up shape and the transposed down shape, Q8_0 and Q4_K.
    The weights are the seeded N(0, 0.02) values quantized as the reference quantizes them (the oracle's quantizers
    reproduce the reference's bytes for exactly these tensors: digests sha_cfg5.*).  Checked: 64 output rows against the
    oracle's fp64 product, a GEMM row against the decode GEMV of the same row (two different kernels), exact
    linearity under a power-of-two scaling of the activations, and finiteness of every output."""
    import torch
    from tensorsharp_amd import QuantizedWeight
    name, N, K = inputs.CFG5[tname]
    M = 2048
    dev = torch.device("cuda:0")
    wq = oracle.quantize(T[name], inputs.weights("cfg5." + tname, N * K))
    w = QuantizedWeight(torch.from_numpy(wq).to(dev), T[name], K, N)
    x_host = inputs.activations("cfg5.x." + tname, M, K)
    x = torch.from_numpy(x_host).to(dev)
    y = hip.LinearForward(x, w)
    torch.cuda.synchronize()
    assert bool(torch.isfinite(y).all())
    rows = sample_rows(M, [0, 127, 128, 255, 256, 1023, 1024, 2047], 64, 5)
    ref = oracle.matmul_f64(T[name], wq, N, K, x_host[rows])
    e = check(y[rows].cpu().numpy(), ref, (name, N, K))
    print("cfg5 %s %dx%dx%d row-L2 err %.2e rms err %.2e over %d rows" % ((name, M, N, K) + e + (len(rows),)))
    # the decode kernel on one of the rows
    r = rows[len(rows) // 2]
    y1 = hip.LinearForward(x[r:r + 1].contiguous(), w)
    check(y1.cpu().numpy(), ref[len(rows) // 2:len(rows) // 2 + 1], (name, "gemv row"))
    # activations times 4: every row's power-of-two scale absorbs the factor, so the results are exactly 4 y
    y4 = hip.LinearForward(x * 4.0, w)
    torch.cuda.synchronize()
    assert torch.equal(y4, y * 4.0)


@pytest.mark.parametrize("name", ["q4_k", "q8_0", "mxfp4", "q5_k", "q6_k", "q4_1"])
@pytest.mark.parametrize("M,N,K", [(200, 32, 1024), (9, 63, 2048), (4, 1, 512)])
def test_narrow_results_are_formed_from_exact_weights(hip, oracle, name, M, N, K):
    """Fewer than 64 result columns with more than three rows: the row norm the 1e-3 bound is taken against is that of a
    few numbers, and the rounded scale products of fp16 operands (Q4_K: every result 7.5e-4 of the results' magnitude off,
    one sigma) would come within reach of it.  Such calls multiply by an exact fp32 copy of the small weight instead, and
    agree with the fp64 reference to fp32 rounding."""
    import torch
    from oracle.oracle import MORE_TYPES, Q6_K
    from tensorsharp_amd import QuantizedWeight, synth
    t = T.get(name) or MORE_TYPES.get(name) or Q6_K
    rng = np.random.default_rng(M + N + K)
    w = synth.random_weight(t, N, K, torch.device("cuda"), seed=7, sigma=0.03)
    x = (rng.standard_normal((M, K)) * 2).astype(np.float32)
    ref = oracle.matmul_f64(t, w.cpu().numpy(), N, K, x)
    y = hip.LinearForward(torch.from_numpy(x).cuda(), QuantizedWeight(w, t, K, N))
    torch.cuda.synchronize()
    err = inputs.row_l2_err(y.cpu().numpy(), ref)         # fp16 operands would leave 1e-4 ... 1e-3 here
    assert err <= 1e-5, (name, M, N, K, err)
