"""The benchmark's torch block generators against the oracle (CPU tensors)."""
import numpy as np
import torch

from oracle.oracle import Q8_0, Q4_K, MXFP4
from tensorsharp_amd import synth


def test_q8_0_and_mxfp4_generators_are_the_reference_quantizers(oracle):
    g = torch.Generator().manual_seed(3)
    w = torch.randn((64, 512), generator=g) * 0.02
    for t, fn in ((Q8_0, synth.quantize_q8_0), (MXFP4, synth.quantize_mxfp4)):
        mine = fn(w).numpy()
        want = oracle.quantize(t, w.numpy().reshape(-1))
        assert np.array_equal(mine, want), t


def test_q4_k_generator_makes_valid_blocks(oracle):
    g = torch.Generator().manual_seed(4)
    w = torch.randn((32, 1024), generator=g) * 0.02
    raw = synth.quantize_q4_k_simple(w).numpy()
    assert raw.size == 32 * 4 * 144
    deq = oracle.dequantize(Q4_K, raw)
    rms = float(np.sqrt(np.mean((deq - w.numpy().reshape(-1)) ** 2))) / 0.02
    assert rms < 0.12          # the reference's search reaches 0.071; a plain min/max fit stays close


def test_other_generators_make_valid_blocks(oracle):
    from oracle.oracle import Q5_K, Q6_K
    g = torch.Generator().manual_seed(5)
    w = torch.randn((16, 1024), generator=g) * 0.02
    from oracle.oracle import Q4_0, Q4_1
    for t, fn, size, bound in ((Q5_K, synth.quantize_q5_k_simple, 176, 0.06), (Q6_K, synth.quantize_q6_k_simple, 210, 0.04),
                               (Q4_0, synth.quantize_q4_0_simple, 8 * 18, 0.2), (Q4_1, synth.quantize_q4_1_simple, 8 * 20, 0.12)):
        raw = fn(w).numpy()
        assert raw.size == 16 * 4 * size
        deq = oracle.dequantize(t, raw)
        rms = float(np.sqrt(np.mean((deq - w.numpy().reshape(-1)) ** 2))) / 0.02
        assert rms < bound, (t, rms)
