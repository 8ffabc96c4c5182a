"""Regenerates tests/golden/golden.npz.  Runs only where the reference checkout exists: it
drives the reference's own ggml code (compiled in place into oracle/_ref by `make -C oracle
ref`) on seeded inputs and stores inputs + outputs as data.

Contents
  ref_tests_*      the hand-built vectors held by the reference's unit tests
                   (InferenceWeb.Tests/ManagedQuantizedOpsTests.cs:29-194), typed in as bytes
  blocks_<fmt>_x / _q / _deq
                   seeded fp32 values, the reference quantizer's bytes, the reference
                   dequantizer's floats (a few KB per format, incl. edge blocks)
  mm_<fmt>_*       a small matmul known-answer: reference ggml_mul_mat output on its CPU path
  q8k_*            reference Q8_K activation blocks
  sha_<name>       SHA-256 of the reference-quantized bytes of the seeded BASELINE weights
"""
import hashlib
import os
import struct
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(HERE))

from oracle.oracle import Reference, Q8_0, Q4_K, MXFP4, build_ref  # noqa: E402
import inputs  # noqa: E402

TYPES = {"q8_0": Q8_0, "q4_k": Q4_K, "mxfp4": MXFP4}


def half_bits(v):
    return struct.unpack("<H", np.float16(v).tobytes())[0]


def ref_test_vectors(out):
    # Q8_0 block: d=0.5, qs={2,-4,7,0...}  (ManagedQuantizedOpsTests.cs:29-45, :113-147)
    raw = np.zeros(34, dtype=np.uint8)
    raw[0:2] = np.frombuffer(struct.pack("<H", half_bits(0.5)), dtype=np.uint8)
    raw[2], raw[3], raw[4] = 2, (-4) & 0xFF, 7
    out["ref_tests_q8_0_raw"] = raw
    out["ref_tests_q8_0_expect_idx"] = np.array([0, 1, 2, 3], dtype=np.int32)
    out["ref_tests_q8_0_expect_val"] = np.array([1.0, -2.0, 3.5, 0.0], dtype=np.float32)
    x = np.zeros((2, 32), dtype=np.float32)
    for i in range(32):
        x[0, i] = np.float32(i) * np.float32(0.125)
        x[1, i] = np.float32(1.0) - np.float32(i) * np.float32(0.03125)
    out["ref_tests_q8_0_dot_x"] = x
    # Q4_K block (ManagedQuantizedOpsTests.cs:47-68 dequant, :149-194 dot)
    raw = np.zeros(144, dtype=np.uint8)
    raw[0:2] = np.frombuffer(struct.pack("<H", half_bits(0.5)), dtype=np.uint8)
    raw[2:4] = np.frombuffer(struct.pack("<H", half_bits(0.25)), dtype=np.uint8)
    raw[4], raw[8], raw[5], raw[9] = 2, 1, 3, 4
    raw[16] = 0x21
    out["ref_tests_q4_k_raw"] = raw.copy()
    out["ref_tests_q4_k_expect_idx"] = np.array([0, 1, 32, 33], dtype=np.int32)
    out["ref_tests_q4_k_expect_val"] = np.array([0.75, -0.25, 2.0, -1.0], dtype=np.float32)
    raw[48], raw[80], raw[112] = 0x34, 0x87, 0x65
    out["ref_tests_q4_k_dot_raw"] = raw
    x = np.zeros((3, 256), dtype=np.float32)
    for row in range(3):
        for i in range(256):
            x[row, i] = np.float32(np.float32(row + 1) * np.float32(0.01)) * np.float32((i % 17) - 8)
    out["ref_tests_q4_k_dot_x"] = x


def main():
    assert build_ref(), "reference checkout not found"
    ref = Reference()
    out = {}
    ref_test_vectors(out)
    rng = np.random.default_rng(20240611)
    for name, t in TYPES.items():
        bs = 256 if t == Q4_K else 32
        n = 256 * 12
        x = (rng.standard_normal(n) * 0.02).astype(np.float32)
        # edge blocks: all zero, constant, one huge outlier, tiny values, negative-only
        x[0:bs] = 0.0
        x[bs:2 * bs] = 0.0123
        x[2 * bs + 5] = 3.0
        x[3 * bs:4 * bs] *= 1e-4
        x[4 * bs:5 * bs] = -np.abs(x[4 * bs:5 * bs])
        q = ref.quantize(t, x)
        out[f"blocks_{name}_x"] = x
        out[f"blocks_{name}_q"] = q
        out[f"blocks_{name}_deq"] = ref.dequantize(t, q)
        N, K, M = 24, 512, 3
        w = (rng.standard_normal(N * K) * 0.02).astype(np.float32)
        wq = ref.quantize(t, w, n_per_row=K)
        xx = rng.standard_normal((M, K)).astype(np.float32)
        out[f"mm_{name}_wq"] = wq
        out[f"mm_{name}_x"] = xx
        out[f"mm_{name}_y_ggml"] = ref.mul_mat(t, wq, N, K, xx, threads=1)
    xa = rng.standard_normal(256 * 4).astype(np.float32)
    xa[256:512] = 0.0
    out["q8k_x"] = xa
    out["q8k_q"] = ref.quantize_q8_K(xa)

    # digests of the seeded BASELINE weights, quantized by the reference
    for cfg_name, cfg in (("cfg1", inputs.CFG1), ("cfg2", inputs.CFG2), ("cfg3", inputs.CFG3), ("cfg4", inputs.CFG4),
                          ("cfg5", inputs.CFG5)):
        for tname, (fmt, N, K) in cfg.items():
            tag = f"{cfg_name}.{tname}"
            w = inputs.weights(tag, N * K)
            q = ref.quantize(TYPES[fmt], w, n_per_row=K)
            out[f"sha_{tag}"] = np.frombuffer(hashlib.sha256(q.tobytes()).digest(), dtype=np.uint8)
            print(tag, hashlib.sha256(q.tobytes()).hexdigest(), flush=True)
    np.savez_compressed(os.path.join(HERE, "golden.npz"), **out)
    print("wrote golden.npz", os.path.getsize(os.path.join(HERE, "golden.npz")), "bytes")


if __name__ == "__main__":
    main()
