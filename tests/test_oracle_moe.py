"""MoE routing / grouping / expert FFN of the oracle (restating GptOssModel.cs:699-934)."""
import numpy as np

from oracle.oracle import MXFP4


def test_route_top_k_and_softmax_brute_force(oracle):
    rng = np.random.default_rng(11)
    T, E, k = 37, 32, 4
    logits = rng.standard_normal((T, E)).astype(np.float32)
    logits[3, 5] = logits[3, 9] = logits[3].max() + 1   # tie: first index wins
    ids, wts = oracle.moe_route(logits, k)
    for t in range(T):
        order = sorted(range(E), key=lambda i: (-logits[t, i], i))[:k]
        assert list(ids[t]) == order
        sel = logits[t, order].astype(np.float64)
        p = np.exp(sel - sel.max())
        p /= p.sum()
        np.testing.assert_allclose(wts[t], p, rtol=2e-6)
    assert list(ids[3][:2]) == [5, 9]


def test_group_is_stable_counting_sort(oracle):
    rng = np.random.default_rng(12)
    T, E, k = 50, 8, 3
    ids = np.stack([rng.permutation(E)[:k] for _ in range(T)]).astype(np.int32)
    wts = rng.random((T, k)).astype(np.float32)
    offs, tmap, wmap = oracle.moe_group(ids, wts, E)
    flat = [(int(ids[t, s]), t, float(wts[t, s])) for t in range(T) for s in range(k)]
    flat.sort(key=lambda v: v[0])          # python sort is stable: token order kept per expert
    assert [v[1] for v in flat] == list(tmap)
    np.testing.assert_array_equal(np.array([v[2] for v in flat], dtype=np.float32), wmap)
    counts = np.bincount(ids.reshape(-1), minlength=E)
    np.testing.assert_array_equal(np.diff(offs), counts)
    assert offs[0] == 0 and offs[-1] == T * k


def test_swiglu_oai_closed_form(oracle):
    gu = np.array([[0.5, 8.0, -3.0, 0.0, 1.0, 9.0, -9.0, 2.0]], dtype=np.float32)   # F=4: gate | up
    out = oracle.swiglu_oai(gu)
    g = np.minimum(gu[0, :4].astype(np.float64), 7.0)
    u = np.clip(gu[0, 4:].astype(np.float64), -7.0, 7.0)
    want = g / (1 + np.exp(-1.702 * g)) * (u + 1)
    np.testing.assert_allclose(out[0], want, rtol=1e-6)


def test_grouped_forward_equals_per_token_loop(oracle):
    rng = np.random.default_rng(13)
    E, H, F, T, k = 6, 64, 96, 9, 2
    gu_w = oracle.quantize(MXFP4, (rng.standard_normal(E * 2 * F * H) * 0.05).astype(np.float32))
    dn_w = oracle.quantize(MXFP4, (rng.standard_normal(E * H * F) * 0.05).astype(np.float32))
    gu_b = (rng.standard_normal((E, 2 * F)) * 0.1).astype(np.float32)
    dn_b = (rng.standard_normal((E, H)) * 0.1).astype(np.float32)
    hidden = rng.standard_normal((T, H)).astype(np.float32)
    ids, wts = oracle.moe_route(rng.standard_normal((T, E)).astype(np.float32), k)
    full = oracle.moe_forward(MXFP4, gu_w, gu_b, dn_w, dn_b, E, H, F, hidden, ids, wts)
    # brute force with dense dequantised experts in fp64
    gw = oracle.dequantize(MXFP4, gu_w).reshape(E, 2 * F, H).astype(np.float64)
    dw = oracle.dequantize(MXFP4, dn_w).reshape(E, H, F).astype(np.float64)
    want = np.zeros((T, H))
    for t in range(T):
        for s in range(k):
            e = ids[t, s]
            gu = gw[e] @ hidden[t].astype(np.float64) + gu_b[e]
            g = np.minimum(gu[:F], 7.0)
            u = np.clip(gu[F:], -7.0, 7.0)
            act = g / (1 + np.exp(-1.702 * g)) * (u + 1)
            want[t] += wts[t, s] * (dw[e] @ act + dn_b[e])
    np.testing.assert_allclose(full, want, rtol=2e-4, atol=2e-5)
    # single-token path (selection order) agrees with the batched path (expert order)
    for t in range(T):
        one = oracle.moe_forward(MXFP4, gu_w, gu_b, dn_w, dn_b, E, H, F, hidden[t:t + 1], ids[t:t + 1], wts[t:t + 1])
        np.testing.assert_allclose(one[0], full[t], rtol=1e-5, atol=1e-6)


def test_more_experts_than_assignments(oracle):
    # T > 1 visits all E experts even when fewer (token, expert) pairs exist; most experts stay empty
    rng = np.random.default_rng(14)
    E, H, F, T, k = 64, 32, 32, 3, 1
    gu_w = oracle.quantize(MXFP4, (rng.standard_normal(E * 2 * F * H) * 0.05).astype(np.float32))
    dn_w = oracle.quantize(MXFP4, (rng.standard_normal(E * H * F) * 0.05).astype(np.float32))
    hidden = rng.standard_normal((T, H)).astype(np.float32)
    ids, wts = oracle.moe_route(rng.standard_normal((T, E)).astype(np.float32), k)
    full = oracle.moe_forward(MXFP4, gu_w, None, dn_w, None, E, H, F, hidden, ids, wts)
    for t in range(T):
        one = oracle.moe_forward(MXFP4, gu_w, None, dn_w, None, E, H, F, hidden[t:t + 1], ids[t:t + 1], wts[t:t + 1])
        np.testing.assert_allclose(one[0], full[t], rtol=1e-5, atol=1e-6)
