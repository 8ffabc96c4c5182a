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


# ---- compositions: out-projection + FFN / router, weighted expert sets -----------------------------------------
def _f32w(mat):
    """(type, raw, N, K) of a dense F32 weight"""
    from oracle.oracle import F32
    m = np.ascontiguousarray(mat, dtype=np.float32)
    return (F32, m.view(np.uint8).reshape(-1), m.shape[0], m.shape[1])


def test_expert_ffn_closed_forms_pin_the_roles_of_gate_up_down(oracle):
    rng = np.random.default_rng(85)
    H = 32
    x = (rng.standard_normal((3, H)) * 2).astype(np.float32)
    eye = np.eye(H, dtype=np.float32)
    x64 = x.astype(np.float64)
    # gate = 3 I, up = I, down = 2 I: 2 * silu(3x) * x elementwise; swapping gate and up would give 2 * silu(x) * 3x
    got = oracle.expert_ffn(x, dict(gate=_f32w(3 * eye), up=_f32w(eye), down=_f32w(2 * eye)))
    ref = 2 * (3 * x64 / (1 + np.exp(-3 * x64))) * x64
    assert np.max(np.abs(got - ref)) <= 1e-5 * np.max(np.abs(ref))
    # no gate: max(x, 0)^2, exactly zero where x < 0
    got = oracle.expert_ffn(x, dict(gate=None, up=_f32w(eye), down=_f32w(eye)))
    assert np.array_equal(got == 0, x <= 0)
    assert np.allclose(got, np.maximum(x64, 0) ** 2, rtol=1e-6)
    # a rectangular down projection picks rows of the activation: down = first 5 rows of I
    got = oracle.expert_ffn(x, dict(gate=None, up=_f32w(eye), down=_f32w(eye[:5])))
    assert got.shape == (3, 5) and np.allclose(got, np.maximum(x64[:, :5], 0) ** 2, rtol=1e-6)


def test_expert_set_is_a_weighted_sum_plus_base(oracle):
    from oracle.oracle import Q8_0
    rng = np.random.default_rng(86)
    H, I = 64, 96

    def q(n, k):
        return (Q8_0, oracle.quantize(Q8_0, (rng.standard_normal(n * k) * 0.1).astype(np.float32)), n, k)

    experts = [dict(gate=q(I, H), up=q(I, H), down=q(H, I)) for _ in range(4)]
    w = np.array([0.5, 0.25, -1.0, 2.0], np.float32)       # powers of two: scaling is exact
    x = rng.standard_normal((2, H)).astype(np.float32)
    base = rng.standard_normal((2, H)).astype(np.float32)
    full, parts = oracle.expert_set(x, experts, w)
    assert np.allclose(full, sum(p * float(c) for p, c in zip(parts, w)), rtol=1e-12, atol=1e-12)
    # linear in the route weights, additive over disjoint subsets, the base is added untouched
    assert np.allclose(oracle.expert_set(x, experts, 2 * w)[0], 2 * full, rtol=1e-12)
    a = oracle.expert_set(x, experts[:2], w[:2])[0]
    b = oracle.expert_set(x, experts[2:], w[2:])[0]
    assert np.allclose(a + b, full, rtol=1e-12, atol=1e-12)
    assert np.allclose(oracle.expert_set(x, experts, w, base)[0] - full, base, rtol=1e-12, atol=1e-12)
    # one expert with weight 1 is the expert itself; a zero weight removes an expert
    assert np.array_equal(oracle.expert_set(x, experts[:1], [1.0])[0], parts[0])
    assert np.allclose(oracle.expert_set(x, experts[:2], [1.0, 0.0])[0], parts[0])


def test_outproj_ffn_and_router_closed_forms(oracle):
    rng = np.random.default_rng(87)
    H = 48
    eye = np.eye(H, dtype=np.float32)
    r = rng.standard_normal((2, H)).astype(np.float32)
    x = rng.standard_normal((2, H)).astype(np.float32)
    ones = np.ones(H, np.float32)
    # W_out = 0, norm weight 1, eps 0, gate_up = [I; I], down = I: r + silu(r / rms) * (r / rms)
    got, mm1, mm2 = oracle.outproj_ffn(r, x, _f32w(0 * eye), ones, 0.0, _f32w(np.concatenate([eye, eye])), _f32w(eye), H)
    n = r.astype(np.float64) / np.sqrt((r.astype(np.float64) ** 2).mean(axis=1, keepdims=True))
    assert np.all(mm1 == 0)
    assert np.allclose(got, r + n / (1 + np.exp(-n)) * n, rtol=1e-5, atol=1e-6)
    # W_out = I feeds the input into the residual BEFORE the norm: the FFN sees r + x
    got, mm1, _ = oracle.outproj_ffn(r, x, _f32w(eye), ones, 0.0, _f32w(np.concatenate([eye, eye])), _f32w(eye), H)
    s = (r + x).astype(np.float64)
    n = s / np.sqrt((s ** 2).mean(axis=1, keepdims=True))
    assert np.allclose(mm1, x) and np.allclose(got, s + n / (1 + np.exp(-n)) * n, rtol=1e-5, atol=1e-6)
    # router = first three rows of 2 I: logits are twice the first three normalised values, times the norm weight
    nw = rng.uniform(0.5, 1.5, H).astype(np.float32)
    res, normed, logits, _ = oracle.outproj_norm_router(r, x, _f32w(eye), nw, 0.0, _f32w(2 * eye[:3]))
    assert np.allclose(res, s) and np.allclose(normed, n * nw, rtol=1e-5)
    assert logits.shape == (2, 3) and np.allclose(logits, 2 * normed[:, :3].astype(np.float64), rtol=1e-12)


def test_dense_weight_rows(oracle):
    from oracle.oracle import F16, BF16
    rng = np.random.default_rng(88)
    v = rng.standard_normal((4, 8)).astype(np.float32)
    h = v.astype(np.float16)
    assert np.array_equal(oracle.weight_rows(F16, h.view(np.uint8).reshape(-1), 4, 8), h.astype(np.float32))
    b = (v.view(np.uint32) >> 16).astype(np.uint16)          # truncated bf16 bit patterns
    want = (b.astype(np.uint32) << 16).view(np.float32)
    assert np.array_equal(oracle.weight_rows(BF16, b.view(np.uint8).reshape(-1), 4, 8), want)
    x = rng.standard_normal((3, 8)).astype(np.float32)
    assert np.allclose(oracle.matmul_any_f64(F16, h.view(np.uint8).reshape(-1), 4, 8, x), x.astype(np.float64) @ h.astype(np.float64).T)


def test_mul_mat_id_brute_force_and_broadcast(oracle):
    rng = np.random.default_rng(89)
    E, rows, K, T, k = 5, 3, 4, 2, 4
    w = rng.standard_normal((E, rows, K)).astype(np.float32)
    ids = rng.integers(0, E, (T, k))
    # one input slot broadcast over the k selected experts, then one slot per selected expert
    for slots in (1, k, 2):
        x = rng.standard_normal((T, slots, K)).astype(np.float32)
        got = oracle.mul_mat_id(w, x, ids)
        for t in range(T):
            for s in range(k):
                for r in range(rows):
                    want = sum(float(w[ids[t, s], r, j]) * float(x[t, s % slots, j]) for j in range(K))
                    assert abs(got[t, s, r] - want) < 1e-12
    # the id picks the expert: a one-hot expert stack returns the selected expert's marker
    mark = np.zeros((E, 1, 1), np.float32)
    mark[:, 0, 0] = np.arange(E) + 1
    assert np.array_equal(oracle.mul_mat_id(mark, np.ones((T, 1, 1), np.float32), ids)[:, :, 0], ids + 1)


def test_add_id_definition_and_reference(reference):
    """ggml_add_id (the per-expert bias of a mul_mat_id): the oracle is the definition written out; the reference's own
    CPU op must agree bit for bit."""
    from oracle.oracle import add_id
    rng = np.random.default_rng(2710)
    T, cols, rows, E = 5, 3, 37, 6
    src = rng.standard_normal((T, cols, rows)).astype(np.float32)
    bias = rng.standard_normal((E, rows)).astype(np.float32)
    ids = rng.integers(0, E, (T, cols)).astype(np.int32)
    want = add_id(src, bias, ids)
    assert np.array_equal(want, src + bias[ids])                      # the same thing through numpy's gather
    assert np.array_equal(reference.add_id(src, bias, ids).view(np.uint32), want.view(np.uint32))
