"""Regenerates tests/golden/tiny.gguf, tiny_align64.gguf, tiny_moe.gguf and their expected tensor bytes (.npz).

Runs only where the reference checkout exists: the file is written by the reference's own GGUF writer (gguf.cpp,
compiled in place into oracle/_ref by `make -C oracle ref`) through oracle/ref_driver.c:ref_write_gguf; the tensor bytes
come from the reference quantizers on seeded values.  The .npz holds the same tensor bytes for comparison."""
import ctypes as C
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)

from oracle.oracle import Reference, build_ref, BLOCK  # noqa: E402

TENSORS = [("token_embd.weight", 8, 64, 40), ("blk.0.attn_q.weight", 12, 256, 24), ("blk.0.ffn_down.weight", 14, 512, 16),
           ("blk.0.ffn_gate_exps.weight", 39, 96, 20), ("blk.0.attn_norm.weight", 0, 64, 1), ("output.weight", 2, 64, 12)]


# a MoE file as llama.cpp's converter lays it out: the experts of a projection stacked in one 3-D tensor [ne0, ne1, E].
# Layer 0 follows GPT-OSS (MXFP4 experts with biases, a router with bias), layer 1 Qwen3-MoE (K-quant experts, no biases).
MOE_E, MOE_USED, MOE_H, MOE_F = 4, 2, 64, 32
MOE_TENSORS = [("blk.0.ffn_gate_inp.weight", 0, MOE_H, MOE_E, 1), ("blk.0.ffn_gate_inp.bias", 0, MOE_E, 1, 1),
               ("blk.0.ffn_gate_exps.weight", 39, MOE_H, MOE_F, MOE_E), ("blk.0.ffn_gate_exps.bias", 0, MOE_F, MOE_E, 1),
               ("blk.0.ffn_up_exps.weight", 39, MOE_H, MOE_F, MOE_E), ("blk.0.ffn_up_exps.bias", 0, MOE_F, MOE_E, 1),
               ("blk.0.ffn_down_exps.weight", 39, MOE_F, MOE_H, MOE_E), ("blk.0.ffn_down_exps.bias", 0, MOE_H, MOE_E, 1),
               ("blk.1.ffn_gate_exps.weight", 12, 256, 32, MOE_E), ("blk.1.ffn_up_exps.weight", 12, 256, 32, MOE_E),
               ("blk.1.ffn_down_exps.weight", 8, 32, 256, MOE_E)]


def write_moe(ref):
    rng = np.random.default_rng(20250212)
    datas, expect = [], {}
    for name, t, ne0, ne1, ne2 in MOE_TENSORS:
        x = (rng.standard_normal(ne0 * ne1 * ne2) * (0.05 if t else 0.5)).astype(np.float32)
        q = x.view(np.uint8).copy() if t == 0 else ref.quantize(t, x, n_per_row=ne0)
        datas.append(q)
        expect[name] = q
    n = len(MOE_TENSORS)
    names = (C.c_char_p * n)(*[t[0].encode() for t in MOE_TENSORS])
    types = (C.c_int * n)(*[t[1] for t in MOE_TENSORS])
    ne0 = (C.c_int64 * n)(*[t[2] for t in MOE_TENSORS])
    ne1 = (C.c_int64 * n)(*[t[3] for t in MOE_TENSORS])
    ne2 = (C.c_int64 * n)(*[t[4] for t in MOE_TENSORS])
    ptrs = (C.c_void_p * n)(*[d.ctypes.data for d in datas])
    ref.lib.ref_write_gguf_moe.restype = C.c_int
    path = os.path.join(HERE, "tiny_moe.gguf")
    rc = ref.lib.ref_write_gguf_moe(path.encode(), b"gpt-oss", MOE_E, MOE_USED, n, names, types, ne0, ne1, ne2, ptrs)
    assert rc == 0, rc
    print("wrote", path, os.path.getsize(path), "bytes")
    np.savez_compressed(os.path.join(HERE, "tiny_moe_gguf_expect.npz"), **{k.replace(".", "__"): v for k, v in expect.items()})


def main():
    assert build_ref(), "reference checkout not found"
    ref = Reference()
    lib = ref.lib
    rng = np.random.default_rng(20250211)
    datas, expect = [], {}
    for name, t, ne0, ne1 in TENSORS:
        x = (rng.standard_normal(ne0 * ne1) * 0.05).astype(np.float32)
        q = x.view(np.uint8).copy() if t == 0 else ref.quantize(t, x, n_per_row=ne0)
        datas.append(q)
        expect[name] = q
    for alignment, fname in ((32, "tiny.gguf"), (64, "tiny_align64.gguf")):
        n = len(TENSORS)
        names = (C.c_char_p * n)(*[t[0].encode() for t in TENSORS])
        types = (C.c_int * n)(*[t[1] for t in TENSORS])
        ne0 = (C.c_int64 * n)(*[t[2] for t in TENSORS])
        ne1 = (C.c_int64 * n)(*[t[3] for t in TENSORS])
        ptrs = (C.c_void_p * n)(*[d.ctypes.data for d in datas])
        lib.ref_write_gguf.restype = C.c_int
        path = os.path.join(HERE, fname)
        rc = lib.ref_write_gguf(path.encode(), alignment, n, names, types, ne0, ne1, ptrs)
        assert rc == 0, rc
        print("wrote", path, os.path.getsize(path), "bytes")
    np.savez_compressed(os.path.join(HERE, "tiny_gguf_expect.npz"), **{k.replace(".", "__"): v for k, v in expect.items()})
    write_moe(ref)


if __name__ == "__main__":
    main()
