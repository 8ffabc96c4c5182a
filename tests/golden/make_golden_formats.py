"""Regenerates tests/golden/formats.npz: known answers for the block formats beyond Q8_0 / Q4_K / MXFP4.

Runs only where the reference checkout exists: it drives the reference's own ggml code (compiled in place
into oracle/_ref by `make -C oracle ref`) and stores inputs + outputs as data.

Contents, per format <fmt> in f16, bf16, q4_0, q4_1, q5_0, q5_1, q5_k, q6_k, iq4_nl:
  <fmt>_x     seeded fp32 values (incl. an all-zero block, a constant block, an outlier, tiny and negative-only blocks)
  <fmt>_q     the reference quantizer's bytes for them (ggml_quantize_chunk)
  <fmt>_deq   the reference dequantizer's floats for those bytes (type traits to_float)
  <fmt>_rq / <fmt>_rdeq   blocks of random bytes (scales kept finite) and the reference dequantizer's floats
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)

from oracle.oracle import Reference, MORE_TYPES, BLOCK, build_ref  # noqa: E402

# byte positions of the high bytes of the fp16 scales inside a block (made finite in the random blocks)
SCALE_HI = {"f16": [1], "bf16": [1], "q4_0": [1], "q4_1": [1, 3], "q5_0": [1], "q5_1": [1, 3], "q5_k": [1, 3],
            "q6_k": [209], "iq4_nl": [1]}


def random_blocks(name, t, nb, rng):
    bs, bb = BLOCK[t]
    raw = rng.integers(0, 256, size=(nb * (256 // bs if bs > 1 else 256), bb), dtype=np.uint8)
    for pos in SCALE_HI[name]:
        raw[:, pos] &= 0x7B if name != "bf16" else 0x7F       # no inf / NaN scales
        if name == "bf16":
            raw[:, pos] = np.where(raw[:, pos] == 0x7F, 0x3F, raw[:, pos])
    return raw.reshape(-1)


def main():
    assert build_ref(), "reference checkout not found"
    ref = Reference()
    rng = np.random.default_rng(20250117)
    out = {}
    for name, t in MORE_TYPES.items():
        bs = max(BLOCK[t][0], 32)
        n = 256 * 6
        x = (rng.standard_normal(n) * 0.02).astype(np.float32)
        x[0:bs] = 0.0
        x[bs:2 * bs] = 0.0123
        x[2 * bs + 5] = 3.0
        x[3 * bs:4 * bs] *= 1e-4
        x[4 * bs:5 * bs] = -np.abs(x[4 * bs:5 * bs])
        q = ref.quantize(t, x)
        out[f"{name}_x"] = x
        out[f"{name}_q"] = q
        out[f"{name}_deq"] = ref.dequantize(t, q)
        rq = random_blocks(name, t, 8, rng)
        out[f"{name}_rq"] = rq
        out[f"{name}_rdeq"] = ref.dequantize(t, rq)
        print(name, q.size, rq.size, flush=True)
    path = os.path.join(HERE, "formats.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
