"""Oracle pieces of the whole-layer decode (ggml_ops_transformer.cpp:379-470): RoPE, single-query attention and the layer
graph, against known answers computed by the reference's own ggml CPU ops (tests/golden/make_golden_layer.py) and
against what the mathematics fixes."""
import os

import numpy as np
import pytest

from oracle.oracle import Q8_0, Q4_K

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "layer.npz")
LAYER = dict(hidden=256, heads=4, kv_heads=2, head_dim=64, inter=512, max_seq=16, eps=1e-6, rope_base=10000.0, rope_mode=2)


@pytest.fixture(scope="module")
def gold():
    return np.load(GOLD)


def layer_of(gold):
    return {"attn_norm": gold["layer_attn_norm"], "q_norm": gold["layer_q_norm"], "k_norm": gold["layer_k_norm"],
            "ffn_norm": gold["layer_ffn_norm"], "qkv": (Q8_0, gold["layer_qkv"]), "o": (Q8_0, gold["layer_o"]),
            "gate_up": (Q4_K, gold["layer_gate_up"]), "down": (Q4_K, gold["layer_down"]), "intermediate": LAYER["inter"]}


def test_rope_matches_ggml_bit_for_bit(oracle, gold):
    for i, (mode, H, hd, pos, base, fs) in enumerate(gold["rope_cases"]):
        y = oracle.rope(gold[f"rope_{i}_x"], int(pos), int(mode), float(base), float(fs))
        assert np.array_equal(y.view(np.uint32), gold[f"rope_{i}_y"].view(np.uint32)), i


def test_rope_is_a_rotation(oracle):
    rng = np.random.default_rng(3)
    x = rng.standard_normal((5, 128)).astype(np.float32)
    for mode in (0, 2):
        assert np.array_equal(oracle.rope(x, 0, mode, 10000.0), x)                     # position 0: identity
        y = oracle.rope(x, 77, mode, 10000.0)
        pairs = (lambda a: a.reshape(5, 64, 2)) if mode == 0 else (lambda a: np.stack([a[:, :64], a[:, 64:]], axis=2))
        np.testing.assert_allclose(np.linalg.norm(pairs(y), axis=2), np.linalg.norm(pairs(x), axis=2), rtol=1e-5)
        # rotations compose: position a then position b == position a + b (to rounding of the angles)
        np.testing.assert_allclose(oracle.rope(oracle.rope(x, 30, mode, 10000.0), 47, mode, 10000.0), y, atol=2e-4)
        # first pair rotates by exactly `position` radians
        i1 = 1 if mode == 0 else 64
        ang = np.arctan2(y[:, i1], y[:, 0]) - np.arctan2(x[:, i1], x[:, 0])
        np.testing.assert_allclose(np.mod(ang - 77 + np.pi, 2 * np.pi) - np.pi, 0, atol=1e-5)


def test_attention_matches_ggml_flash_attn(oracle, gold):
    out = oracle.attention_decode(gold["attn_q"], gold["attn_k"], gold["attn_v"], int(gold["attn_total"]))
    np.testing.assert_allclose(out, gold["attn_out"], atol=2e-6)


def test_attention_special_cases(oracle):
    rng = np.random.default_rng(5)
    heads, kvh, hd, ms = 6, 3, 32, 20
    q = rng.standard_normal((heads, hd)).astype(np.float32)
    kc = rng.standard_normal((kvh, ms, hd)).astype(np.float32)
    vc = rng.standard_normal((kvh, ms, hd)).astype(np.float32)
    one = oracle.attention_decode(q, kc, vc, 1)                       # a single position: its value row
    for h in range(heads):
        np.testing.assert_allclose(one[h], vc[h // 2, 0], rtol=1e-6)
    kc[:, :7] = kc[:, :1]                                             # equal keys: the mean of the values
    same = oracle.attention_decode(q, kc, vc, 7)
    for h in range(heads):
        np.testing.assert_allclose(same[h], vc[h // 2, :7].mean(axis=0), atol=1e-6)
    # independent numpy softmax
    total = 20
    got = oracle.attention_decode(q, kc, vc, total)
    for h in range(heads):
        s = kc[h // 2, :total].astype(np.float64) @ q[h].astype(np.float64) / np.sqrt(hd)
        p = np.exp(s - s.max())
        np.testing.assert_allclose(got[h], (p / p.sum()) @ vc[h // 2, :total].astype(np.float64), atol=1e-6)


def test_layer_graph_matches_the_ggml_graph(oracle, gold):
    # the reference's CPU matmul quantizes activations to int8 blocks (about 1e-2 of a row): a coarse bound that still
    # catches any mis-wiring (swapped gate / up, a missing residual, wrong head grouping ...)
    L = LAYER
    layer = layer_of(gold)
    kc = np.zeros((L["kv_heads"], L["max_seq"], L["head_dim"]), dtype=np.float32)
    vc = np.zeros_like(kc)
    for pos in range(3):
        h = gold["layer_hidden_in"][pos].copy()
        oracle.layer_decode(h, layer, kc, vc, L["heads"], L["kv_heads"], L["head_dim"], pos, L["eps"], L["rope_base"], 1.0, L["rope_mode"])
        want = gold["layer_hidden_out"][pos]
        assert np.linalg.norm(h - want) <= 2e-2 * np.linalg.norm(want), pos
        assert np.linalg.norm(h - gold["layer_hidden_in"][pos]) > 0.1 * np.linalg.norm(want)     # the layer did something
    assert np.linalg.norm(kc - gold["layer_k_cache"]) <= 2e-2 * np.linalg.norm(gold["layer_k_cache"])
    assert np.linalg.norm(vc - gold["layer_v_cache"]) <= 2e-2 * np.linalg.norm(gold["layer_v_cache"])
    assert np.all(kc[:, 3:] == 0) and np.all(vc[:, 3:] == 0)
