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
