"""Seeded synthetic inputs shared by the CPU and GPU tests (numpy Generator: same bytes on
every machine with this image)."""
import hashlib

import numpy as np

SIGMA_W = 0.02

# BASELINE config shapes: name -> (type name, N, K)
CFG1 = {"ffn_up": ("q8_0", 9728, 2560)}
CFG2 = {
    "wq": ("q4_k", 4096, 4096), "wk": ("q4_k", 1024, 4096), "wv": ("q4_k", 1024, 4096),
    "wo": ("q4_k", 4096, 4096), "gate": ("q4_k", 14336, 4096), "up": ("q4_k", 14336, 4096),
    "down": ("q4_k", 4096, 14336),
}
CFG3 = {"gate": ("q4_k", 14336, 4096)}
CFG4 = {"gate_up": ("mxfp4", 5760, 2880), "down": ("mxfp4", 2880, 2880)}
CFG5 = {"up_q8": ("q8_0", 21504, 5376), "up_q4": ("q4_k", 21504, 5376),
        "down_q8": ("q8_0", 5376, 21504), "down_q4": ("q4_k", 5376, 21504)}


def _key(tag):
    h = hashlib.sha256(tag.encode()).digest()
    return [int.from_bytes(h[i:i + 4], "little") for i in (0, 4, 8, 12)]


def weights(tag, n, seed=0):
    """W ~ N(0, 0.02), fp32, flat."""
    rng = np.random.default_rng([seed] + _key("w:" + tag))
    w = rng.standard_normal(n, dtype=np.float32)
    w *= np.float32(SIGMA_W)
    return w


def activations(tag, m, k, seed=0):
    """x ~ N(0, 1), fp32 [m, k]."""
    rng = np.random.default_rng([seed] + _key("x:" + tag))
    return rng.standard_normal((m, k), dtype=np.float32)


def row_l2_err(y, ref):
    """max_j |y[m,j]-ref[m,j]| / ||ref[m,:]||_2, worst row — the parity metric of the path."""
    y = np.asarray(y, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    nrm = np.linalg.norm(ref, axis=1)
    nrm[nrm == 0] = 1.0
    return float(np.max(np.max(np.abs(y - ref), axis=1) / nrm))


def rms_err(y, ref):
    """max|delta| / rms(ref row), worst row — the stricter per-element view."""
    y = np.asarray(y, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    rms = np.sqrt(np.mean(ref * ref, axis=1))
    rms[rms == 0] = 1.0
    return float(np.max(np.max(np.abs(y - ref), axis=1) / rms))


def random_blocks(name, rows, k, rng):
    """Valid raw blocks of a [rows x k] weight with random quants and small finite scales, for the formats whose
    reference quantizer is not restated here (the layouts: ggml-common.h block_q4_0 ... block_q5_K)."""
    def f16(lo, hi, n):
        return rng.uniform(lo, hi, n).astype(np.float16).view(np.uint8).reshape(n, 2)
    hdr = {"q4_0": 2, "iq4_nl": 2, "q4_1": 4, "q5_0": 6, "q5_1": 8}
    if name in hdr:
        nb = rows * (k // 32)
        raw = rng.integers(0, 256, size=(nb, hdr[name] + 16), dtype=np.uint8)
        raw[:, 0:2] = f16(2e-3, 8e-3, nb) if name != "iq4_nl" else f16(2e-4, 6e-4, nb)
        if name in ("q4_1", "q5_1"):
            raw[:, 2:4] = f16(-0.06, 0.0, nb)
        return raw.reshape(-1)
    if name == "mxfp4":
        nb = rows * (k // 32)
        raw = rng.integers(0, 256, size=(nb, 17), dtype=np.uint8)
        raw[:, 0] = rng.integers(112, 124, nb)          # E8M0 scales of 2^-15 .. 2^-4
        return raw.reshape(-1)
    if name == "q5_k":
        nb = rows * (k // 256)
        raw = rng.integers(0, 256, size=(nb, 176), dtype=np.uint8)
        raw[:, 0:2] = f16(5e-5, 2e-4, nb)
        raw[:, 2:4] = f16(5e-5, 2e-4, nb)
        return raw.reshape(-1)
    raise KeyError(name)
