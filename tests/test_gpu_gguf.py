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


def _gpt_oss_layer_from_file(g, E):
    """Layer 0 of tiny_moe.gguf the way GptOssModel prepares it: expert stacks split, biases split, gate | up fused per
    expert; then the per-expert weights stacked into the operands of the grouped expert stage."""
    from tensorsharp_amd.hip_basic_ops import FuseExpertGateUpWeights, SplitExpertBiases, StackExpertWeights
    ws = g.load_quantized_weights()
    fl = {n: g.float_tensor(n) for n in g.Tensors if n.endswith(".bias") and "_exps" in n}
    SplitExpertBiases(fl, 1)
    FuseExpertGateUpWeights(ws, 1, E, fl)
    gu = StackExpertWeights([ws[f"blk.0.ffn_gate_up_exps.{e}.weight"] for e in range(E)])
    dn = StackExpertWeights([ws[f"blk.0.ffn_down_exps.{e}.weight"] for e in range(E)])
    gu_b = np.concatenate([fl[f"blk.0.ffn_gate_up_exps.{e}.bias"] for e in range(E)], axis=0)
    dn_b = np.concatenate([fl[f"blk.0.ffn_down_exps.{e}.bias"] for e in range(E)], axis=0)
    return gu, gu_b, dn, dn_b


@pytest.mark.parametrize("T", [1, 3, 50])
def test_gpt_oss_moe_stage_from_a_file_with_3d_expert_stacks(hip, oracle, T):
    """Router + expert stage of a GPT-OSS layer (GptOssModel.cs:699-898) from the 3-D `*_exps.` tensors of a file
    written by the reference's own GGUF writer, against tso_moe_route / tso_moe_forward on the same bytes."""
    import torch
    rng = np.random.default_rng(85 + T)
    with GgufFile(os.path.join(GOLD, "tiny_moe.gguf")) as g:
        E, k = g.GetUint32("gpt-oss.expert_count"), g.GetUint32("gpt-oss.expert_used_count")
        gu, gu_b, dn, dn_b = _gpt_oss_layer_from_file(g, E)
        H, F = gu.ne0, dn.ne0
        assert (gu.ne1, dn.ne1) == (E * 2 * F, E * H)
        router_w, router_b = g.float_tensor("blk.0.ffn_gate_inp.weight"), g.float_tensor("blk.0.ffn_gate_inp.bias")
        hidden = rng.standard_normal((T, H)).astype(np.float32)
        logits = (hidden.astype(np.float64) @ router_w.astype(np.float64).T + router_b).astype(np.float32)
        ids_ref, wts_ref = oracle.moe_route(logits, k)
        wts, ids = hip.MoERoute(torch.from_numpy(logits).cuda(), k)
        assert np.array_equal(ids.cpu().numpy(), ids_ref)
        c = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
        out = hip.MoEExpertsGptOssForward(c(hidden), ids, wts, c(np.array(gu.data)), c(gu_b), c(np.array(dn.data)), c(dn_b),
                                          gu.ggml_type, E, H, F)
        torch.cuda.synchronize()
        ref = oracle.moe_forward(gu.ggml_type, np.array(gu.data), gu_b, np.array(dn.data), dn_b, E, H, F, hidden, ids_ref, wts_ref)
        assert inputs.row_l2_err(out.cpu().numpy(), ref) <= 1e-3, inputs.row_l2_err(out.cpu().numpy(), ref)


@pytest.mark.parametrize("M", [1, 4])
@pytest.mark.parametrize("preload", [False, True])
def test_per_expert_calls_on_the_split_stacks(hip, oracle, M, preload):
    """Layer 1 (Q4_K gate / up, Q8_0 down, no biases): the experts of the 3-D tensors as per-expert pointers into the
    mapping, through the bridge-shaped MoEExpertsSwiGLUForward (host form; with and without preload), against the
    oracle's expert set on the same bytes."""
    rng = np.random.default_rng(87 + M)
    with GgufFile(os.path.join(GOLD, "tiny_moe.gguf")) as g:
        names = ["blk.1.ffn_gate_exps.weight", "blk.1.ffn_up_exps.weight", "blk.1.ffn_down_exps.weight"]
        ws = g.preload(names) if preload else {n: w for name in names
                                               for n, w in zip(g.expert_weight_names(name, 4), g.expert_weights(name))}
        assert len(ws) == 12
        sel = [2, 0, 3]
        pick = lambda p: [ws[f"blk.1.ffn_{p}_exps.{e}.weight"] for e in sel]
        gate, up, down = pick("gate"), pick("up"), pick("down")
        H = gate[0].ne0
        x = rng.standard_normal((M, H)).astype(np.float32)
        w = rng.uniform(0.1, 0.6, len(sel)).astype(np.float32)
        out = np.full((M, H), np.nan, np.float32)
        hip.MoEExpertsSwiGLUForward(out, x, gate, up, down, w)
        desc = lambda q: (q.ggml_type, np.array(q.data), q.ne1, q.ne0)
        ex = [dict(gate=desc(a), up=desc(b), down=desc(c)) for a, b, c in zip(gate, up, down)]
        ref, parts = oracle.expert_set(x, ex, w)
        tol = sum(2e-3 * abs(float(wi)) * np.linalg.norm(p.astype(np.float64), axis=1, keepdims=True) for p, wi in zip(parts, w))
        assert np.all(np.abs(out - ref) <= tol), float(np.max(np.abs(out - ref) / tol))
        if not preload:
            hip.ClearHostBufferCache()
