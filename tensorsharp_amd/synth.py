"""Synthetic GGUF block generators (torch, run on whatever device the input lives on).

Benchmarks need W ~ N(0, 0.02) in raw Q8_0 / Q4_K / Q6_K / MXFP4 blocks without touching the CPU
oracle.  Q8_0 and MXFP4 follow the reference quantizers exactly (closed forms,
ggml-quants.c:199-222 and :260-305).  Q4_K uses a plain min/max affine fit per 32-weight
sub-block instead of the reference's iterative scale search (ggml-quants.c:622-701): the
bytes are valid Q4_K super-blocks of the same statistics, not the reference's bytes.
"""
import torch

MXFP4_TABLE = [0, 1, 2, 3, 4, 6, 8, 12, 0, -1, -2, -3, -4, -6, -8, -12]


def _half_bytes(v):
    """fp32 tensor [n] -> uint8 [n, 2] little-endian fp16 (round to nearest even)."""
    return v.to(torch.float16).view(torch.uint8).reshape(-1, 2)


def quantize_q8_0(w):
    x = w.reshape(-1, 32).float()
    amax = x.abs().amax(dim=1)
    d = amax / 127.0
    inv = torch.where(d != 0, 1.0 / d, torch.zeros_like(d))
    s = x * inv[:, None]
    q = torch.where(s >= 0, torch.floor(s + 0.5), torch.ceil(s - 0.5)).to(torch.int8)   # roundf: half away from zero
    out = torch.empty((x.shape[0], 34), dtype=torch.uint8, device=w.device)
    out[:, :2] = _half_bytes(d)
    out[:, 2:] = q.view(torch.uint8)
    return out.reshape(-1)


def quantize_mxfp4(w):
    x = w.reshape(-1, 32).float()
    amax = x.abs().amax(dim=1)
    e = torch.where(amax > 0, torch.floor(torch.log2(amax.clamp_min(1e-38))) - 2 + 127, torch.zeros_like(amax))
    e = e.clamp(0, 255)
    d = torch.pow(torch.tensor(2.0, device=w.device), e - 128.0)
    table = torch.tensor(MXFP4_TABLE, dtype=torch.float32, device=w.device)
    err = (table[None, None, :] * d[:, None, None] - x[:, :, None]).abs()
    idx = torch.argmin(err, dim=2).to(torch.uint8)
    out = torch.empty((x.shape[0], 17), dtype=torch.uint8, device=w.device)
    out[:, 0] = e.to(torch.uint8)
    out[:, 1:] = idx[:, :16] | (idx[:, 16:] << 4)
    return out.reshape(-1)


def quantize_q4_k_simple(w):
    x = w.reshape(-1, 8, 32).float()                     # [blocks, sub-blocks, 32]
    lo = x.amin(dim=2).clamp_max(0.0)
    hi = x.amax(dim=2)
    scale = (hi - lo) / 15.0                             # per sub-block step
    mn = -lo                                             # per sub-block offset (>= 0)
    d = scale.amax(dim=1) / 63.0
    dmin = mn.amax(dim=1) / 63.0
    d16 = d.to(torch.float16).float()
    dmin16 = dmin.to(torch.float16).float()
    ls = torch.where(d16[:, None] > 0, torch.round(scale / d16[:, None].clamp_min(1e-30)), torch.zeros_like(scale)).clamp(0, 63)
    lm = torch.where(dmin16[:, None] > 0, torch.round(mn / dmin16[:, None].clamp_min(1e-30)), torch.zeros_like(mn)).clamp(0, 63)
    eff_d = d16[:, None] * ls
    eff_m = dmin16[:, None] * lm
    q = torch.where(eff_d[:, :, None] > 0, torch.round((x + eff_m[:, :, None]) / eff_d[:, :, None].clamp_min(1e-30)),
                    torch.zeros_like(x)).clamp(0, 15).to(torch.uint8)
    ls = ls.to(torch.uint8)
    lm = lm.to(torch.uint8)
    nb = x.shape[0]
    out = torch.zeros((nb, 144), dtype=torch.uint8, device=w.device)
    out[:, 0:2] = _half_bytes(d)
    out[:, 2:4] = _half_bytes(dmin)
    sc = out[:, 4:16]
    sc[:, 0:4] = ls[:, 0:4] | ((ls[:, 4:8] >> 4) << 6)
    sc[:, 4:8] = lm[:, 0:4] | ((lm[:, 4:8] >> 4) << 6)
    sc[:, 8:12] = (ls[:, 4:8] & 0x0F) | ((lm[:, 4:8] & 0x0F) << 4)
    qq = q.reshape(nb, 4, 2, 32)
    out[:, 16:] = (qq[:, :, 0, :] | (qq[:, :, 1, :] << 4)).reshape(nb, 128)
    return out.reshape(-1)


def quantize_q6_k_simple(w):
    """Valid Q6_K blocks (ggml-common.h block_q6_K) from a plain absmax fit per 16-weight group, not the reference's
    iterative search (ggml-quants.c quantize_row_q6_K_ref): same layout and statistics, not the reference's bytes."""
    x = w.reshape(-1, 16, 16).float()                    # [blocks, groups, 16]
    nb = x.shape[0]
    scale = x.abs().amax(dim=2) / 31.0                   # per group step
    d = scale.amax(dim=1) / 127.0
    d16 = d.to(torch.float16).float()
    sc = torch.where(d16[:, None] > 0, torch.round(scale / d16[:, None].clamp_min(1e-30)), torch.zeros_like(scale)).clamp(1, 127)
    eff = d16[:, None] * sc
    q = torch.where(eff[:, :, None] > 0, torch.round(x / eff[:, :, None].clamp_min(1e-30)), torch.zeros_like(x)).clamp(-32, 31)
    q = (q + 32).to(torch.uint8).reshape(nb, 2, 4, 32)   # [block, half, group of 32, l]
    out = torch.zeros((nb, 210), dtype=torch.uint8, device=w.device)
    lo, hi = q & 0x0F, q >> 4
    ql = out[:, 0:128].reshape(nb, 2, 2, 32)             # [block, half, l / 32, l % 32]
    ql[:, :, 0, :] = lo[:, :, 0, :] | (lo[:, :, 2, :] << 4)
    ql[:, :, 1, :] = lo[:, :, 1, :] | (lo[:, :, 3, :] << 4)
    out[:, 128:192] = (hi[:, :, 0, :] | (hi[:, :, 1, :] << 2) | (hi[:, :, 2, :] << 4) | (hi[:, :, 3, :] << 6)).reshape(nb, 64)
    out[:, 192:208] = sc.to(torch.int8).view(torch.uint8)
    out[:, 208:210] = _half_bytes(d)
    return out.reshape(-1)


def quantize_q5_k_simple(w):
    """Valid Q5_K blocks (ggml-common.h block_q5_K): the per-sub-block affine fit of quantize_q4_k_simple with 31 levels
    instead of 15 (the fifth bits go to qh), for synthetic weights."""
    x = w.reshape(-1, 8, 32).float()
    lo = x.amin(dim=2).clamp_max(0.0)
    hi = x.amax(dim=2)
    scale = (hi - lo) / 31.0
    mn = -lo
    d = scale.amax(dim=1) / 63.0
    dmin = mn.amax(dim=1) / 63.0
    d16 = d.to(torch.float16).float()
    dmin16 = dmin.to(torch.float16).float()
    ls = torch.where(d16[:, None] > 0, torch.round(scale / d16[:, None].clamp_min(1e-30)), torch.zeros_like(scale)).clamp(0, 63)
    lm = torch.where(dmin16[:, None] > 0, torch.round(mn / dmin16[:, None].clamp_min(1e-30)), torch.zeros_like(mn)).clamp(0, 63)
    eff_d = d16[:, None] * ls
    eff_m = dmin16[:, None] * lm
    q = torch.where(eff_d[:, :, None] > 0, torch.round((x + eff_m[:, :, None]) / eff_d[:, :, None].clamp_min(1e-30)),
                    torch.zeros_like(x)).clamp(0, 31).to(torch.uint8)
    ls = ls.to(torch.uint8)
    lm = lm.to(torch.uint8)
    nb = x.shape[0]
    out = torch.zeros((nb, 176), dtype=torch.uint8, device=w.device)
    out[:, 0:2] = _half_bytes(d)
    out[:, 2:4] = _half_bytes(dmin)
    sc = out[:, 4:16]
    sc[:, 0:4] = ls[:, 0:4] | ((ls[:, 4:8] >> 4) << 6)
    sc[:, 4:8] = lm[:, 0:4] | ((lm[:, 4:8] >> 4) << 6)
    sc[:, 8:12] = (ls[:, 4:8] & 0x0F) | ((lm[:, 4:8] & 0x0F) << 4)
    qq = q.reshape(nb, 4, 2, 32)                         # [block, 64-weight group, low / high nibble half, 32]
    qh = out[:, 16:48]
    for u in range(4):
        qh |= ((qq[:, u, 0, :] >> 4) << (2 * u)) | ((qq[:, u, 1, :] >> 4) << (2 * u + 1))
    out[:, 48:] = ((qq[:, :, 0, :] & 15) | ((qq[:, :, 1, :] & 15) << 4)).reshape(nb, 128)
    return out.reshape(-1)


def quantize_q4_0_simple(w):
    """Valid Q4_0 blocks (ggml-common.h block_q4_0): d = amax / 7, q = round(x / d) + 8, for synthetic weights."""
    x = w.reshape(-1, 32).float()
    d = x.abs().amax(dim=1) / 7.0
    d16 = d.to(torch.float16).float()
    q = torch.where(d16[:, None] > 0, torch.round(x / d16[:, None].clamp_min(1e-30)) + 8, torch.full_like(x, 8)).clamp(0, 15).to(torch.uint8)
    out = torch.empty((x.shape[0], 18), dtype=torch.uint8, device=w.device)
    out[:, 0:2] = _half_bytes(d)
    out[:, 2:] = q[:, :16] | (q[:, 16:] << 4)
    return out.reshape(-1)


def quantize_q4_1_simple(w):
    """Valid Q4_1 blocks (ggml-common.h block_q4_1): min / max fit with 15 steps, for synthetic weights."""
    x = w.reshape(-1, 32).float()
    lo = x.amin(dim=1)
    d = (x.amax(dim=1) - lo) / 15.0
    d16 = d.to(torch.float16).float()
    m16 = lo.to(torch.float16).float()
    q = torch.where(d16[:, None] > 0, torch.round((x - m16[:, None]) / d16[:, None].clamp_min(1e-30)), torch.zeros_like(x)).clamp(0, 15).to(torch.uint8)
    out = torch.empty((x.shape[0], 20), dtype=torch.uint8, device=w.device)
    out[:, 0:2] = _half_bytes(d)
    out[:, 2:4] = _half_bytes(lo)
    out[:, 4:] = q[:, :16] | (q[:, 16:] << 4)
    return out.reshape(-1)


def _random_legacy_blocks(header_bytes, with_min):
    """Blocks of 32 weights whose quant bits are random and whose fp16 scale (and minimum) suit weights ~ N(0, 0.02): for
    the formats that only the throughput measurements use (Q5_0, Q5_1, IQ4_NL); values do not follow `w`."""
    def make(w):
        nb = w.numel() // 32
        g = torch.Generator(device=w.device)
        g.manual_seed(int(w.numel()) + header_bytes)
        out = torch.randint(0, 256, (nb, header_bytes + 16), dtype=torch.uint8, device=w.device, generator=g)
        d = torch.full((nb,), 2.5e-3 if header_bytes != 2 else 4e-4, device=w.device)
        out[:, 0:2] = _half_bytes(d)
        if with_min:
            out[:, 2:4] = _half_bytes(torch.full((nb,), -0.04, device=w.device))
        return out.reshape(-1)
    return make


QUANTIZERS = {6: _random_legacy_blocks(6, False), 7: _random_legacy_blocks(8, True), 20: _random_legacy_blocks(2, False),
              2: quantize_q4_0_simple, 3: quantize_q4_1_simple, 8: quantize_q8_0, 12: quantize_q4_k_simple, 13: quantize_q5_k_simple, 14: quantize_q6_k_simple, 39: quantize_mxfp4}


def random_weight(ggml_type, n_rows, n_cols, device, seed, sigma=0.02, chunk_rows=4096):
    """Raw blocks of an [n_rows x n_cols] weight ~ N(0, sigma), generated in row chunks."""
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    parts = []
    for r0 in range(0, n_rows, chunk_rows):
        rows = min(chunk_rows, n_rows - r0)
        w = torch.randn((rows, n_cols), generator=g, device=device, dtype=torch.float32) * sigma
        parts.append(QUANTIZERS[ggml_type](w))
    return torch.cat(parts)
