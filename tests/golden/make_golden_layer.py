"""Regenerates tests/golden/layer.npz: known answers for the pieces of the whole-layer decode, computed by the reference's
own ggml CPU ops (compiled in place into oracle/_ref by `make -C oracle ref`, driven through oracle/ref_driver.c).

  rope_<i>_*    ggml_rope_ext (n_dims = head_dim) in adjacent-pair and NeoX mode
  attn_*        ggml_flash_attn_ext, one query row per head over fp32 KV caches (grouped-query heads)
  layer_*       the layer graph of ggml_ops_transformer.cpp:379-470 built op for op with ggml's API, three tokens in a row;
                coarse (ggml's CPU matmul quantizes activations to int8): pins the wiring, not the digits
Runs only where the reference checkout exists."""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)

from oracle.oracle import Reference, build_ref, Q8_0, Q4_K  # noqa: E402

ROPE_CASES = [(0, 4, 128, 0, 10000.0, 1.0), (0, 4, 128, 17, 1e6, 1.0), (0, 2, 64, 4095, 10000.0, 0.5), (0, 3, 96, 123, 5e5, 1.0),
              (2, 4, 128, 0, 10000.0, 1.0), (2, 4, 128, 17, 1e6, 1.0), (2, 2, 64, 4095, 10000.0, 0.5), (2, 3, 96, 123, 5e5, 1.0)]
LAYER = dict(hidden=256, heads=4, kv_heads=2, head_dim=64, inter=512, max_seq=16, eps=1e-6, rope_base=10000.0, rope_mode=2)


def main():
    assert build_ref(), "reference checkout not found"
    ref = Reference()
    rng = np.random.default_rng(20250303)
    out = {"rope_cases": np.array(ROPE_CASES, dtype=np.float64)}
    for i, (mode, H, hd, pos, base, fs) in enumerate(ROPE_CASES):
        x = rng.standard_normal((H, hd)).astype(np.float32)
        out[f"rope_{i}_x"] = x
        out[f"rope_{i}_y"] = ref.rope(x, pos, mode, base, fs)
    heads, kvh, hd, ms, total = 8, 2, 64, 40, 33
    q = rng.standard_normal((heads, hd)).astype(np.float32)
    kc = rng.standard_normal((kvh, ms, hd)).astype(np.float32)
    vc = rng.standard_normal((kvh, ms, hd)).astype(np.float32)
    out.update(attn_q=q, attn_k=kc, attn_v=vc, attn_total=np.int32(total), attn_out=ref.flash_attn(q, kc, vc, total))

    L = LAYER
    q_dim, k_dim = L["heads"] * L["head_dim"], L["kv_heads"] * L["head_dim"]
    w = lambda n, k: (rng.standard_normal(n * k) * 0.05).astype(np.float32)
    layer = {
        "attn_norm": rng.uniform(0.5, 1.5, L["hidden"]).astype(np.float32),
        "q_norm": rng.uniform(0.5, 1.5, L["head_dim"]).astype(np.float32),
        "k_norm": rng.uniform(0.5, 1.5, L["head_dim"]).astype(np.float32),
        "ffn_norm": rng.uniform(0.5, 1.5, L["hidden"]).astype(np.float32),
        "qkv": (Q8_0, ref.quantize(Q8_0, w(q_dim + 2 * k_dim, L["hidden"]), n_per_row=L["hidden"])),
        "o": (Q8_0, ref.quantize(Q8_0, w(L["hidden"], q_dim), n_per_row=q_dim)),
        "gate_up": (Q4_K, ref.quantize(Q4_K, w(2 * L["inter"], L["hidden"]), n_per_row=L["hidden"])),
        "down": (Q4_K, ref.quantize(Q4_K, w(L["hidden"], L["inter"]), n_per_row=L["inter"])),
        "intermediate": L["inter"],
    }
    for k in ("attn_norm", "q_norm", "k_norm", "ffn_norm"):
        out["layer_" + k] = layer[k]
    for k in ("qkv", "o", "gate_up", "down"):
        out["layer_" + k] = layer[k][1]
    kc = np.zeros((L["kv_heads"], L["max_seq"], L["head_dim"]), dtype=np.float32)
    vc = np.zeros_like(kc)
    hs_in, hs_out = [], []
    for pos in range(3):
        h = rng.standard_normal(L["hidden"]).astype(np.float32)
        hs_in.append(h.copy())
        ref.layer_decode(h, layer, kc, vc, L["heads"], L["kv_heads"], L["head_dim"], pos, L["eps"], L["rope_base"], 1.0, L["rope_mode"])
        hs_out.append(h.copy())
    out.update(layer_hidden_in=np.stack(hs_in), layer_hidden_out=np.stack(hs_out), layer_k_cache=kc, layer_v_cache=vc)
    path = os.path.join(HERE, "layer.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
