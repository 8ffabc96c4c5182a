"""GPU: weights go from a GGUF file's mapping to the device (preload keyed by the mapped address, or a device copy)
and the matmul / embedding gather over them match the oracle on the same bytes."""
import os

import numpy as np
import pytest

import inputs
from tensorsharp_amd.gguf import GgufFile

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
MATS = ["token_embd.weight", "blk.0.attn_q.weight", "blk.0.ffn_down.weight", "blk.0.ffn_gate_exps.weight", "output.weight"]


def test_preload_from_the_mapping_then_host_pointer_calls(hip, oracle):
    rng = np.random.default_rng(81)
    with GgufFile(os.path.join(GOLD, "tiny.gguf")) as g:
        ws = g.preload()
        assert sorted(ws) == sorted(MATS)          # Q8_0, Q4_K, Q6_K, MXFP4 and Q4_0 matrices; the F32 norm is skipped
        for name, w in ws.items():
            for M in (1, 5):
                x = rng.standard_normal((M, w.ne0)).astype(np.float32)
                y = np.empty((M, w.ne1), dtype=np.float32)
                hip.AddmmQuant(y, x, w.ptr, w.ggml_type, w.ne0, w.ne1, w.raw_bytes)
                ref = oracle.matmul_f64(w.ggml_type, np.array(w.data), w.ne1, w.ne0, x)
                assert inputs.row_l2_err(y, ref) <= 1e-3, (name, M)
    # close() dropped the device copies: a sync of one of the former keys finds nothing to do, a matmul on the unmapped
    # address is not attempted here


def test_device_copy_and_embedding_rows(hip, oracle):
    import torch
    rng = np.random.default_rng(83)
    with GgufFile(os.path.join(GOLD, "tiny_align64.gguf")) as g:
        w = g.quantized_weight("blk.0.ffn_down.weight", device="cuda")
        assert w.is_device
        x = rng.standard_normal((7, w.ne0)).astype(np.float32)
        y = hip.LinearForward(torch.from_numpy(x).cuda(), w)
        torch.cuda.synchronize()
        raw = np.array(g.tensor_data("blk.0.ffn_down.weight"))
        assert inputs.row_l2_err(y.cpu().numpy(), oracle.matmul_f64(w.ggml_type, raw, w.ne1, w.ne0, x)) <= 1e-3
        # embedding gather from the Q4_0 output matrix and the Q8_0 token embedding, straight from the mapping
        for name in ("output.weight", "token_embd.weight"):
            info = g.Tensors[name]
            data = g.tensor_data(name)
            idx = np.array([info.Shape[1] - 1, 0, 3], dtype=np.int32)
            res = np.zeros((idx.size, info.Shape[0]), dtype=np.float32)
            hip.GetRowsQuant(res, data.ctypes.data, info.Type, info.Shape[0], info.Shape[1], data.size, idx)
            want = oracle.dequantize(info.Type, np.array(data)).reshape(info.Shape[1], info.Shape[0])[idx]
            assert np.array_equal(res.view(np.uint32), want.view(np.uint32)), name
        hip.ClearHostBufferCache()
