"""GGUF reader (host twin of TensorSharp.Runtime/GgufReader.cs) against files written by the reference's own GGUF
writer (tests/golden/make_golden_gguf.py): header, every metadata value kind, tensor infos, the aligned data section,
and the tensor bytes."""
import os
import struct

import numpy as np
import pytest

from tensorsharp_amd.gguf import GgufFile

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
TENSORS = {"token_embd.weight": (8, (64, 40)), "blk.0.attn_q.weight": (12, (256, 24)), "blk.0.ffn_down.weight": (14, (512, 16)),
           "blk.0.ffn_gate_exps.weight": (39, (96, 20)), "blk.0.attn_norm.weight": (0, (64,)), "output.weight": (2, (64, 12))}


@pytest.fixture(scope="module")
def expect():
    z = np.load(os.path.join(GOLD, "tiny_gguf_expect.npz"))
    return {k.replace("__", "."): z[k] for k in z.files}


@pytest.mark.parametrize("fname,alignment", [("tiny.gguf", 32), ("tiny_align64.gguf", 64)])
def test_reference_written_file(fname, alignment, expect):
    with GgufFile(os.path.join(GOLD, fname)) as g:
        assert g.Version == 3
        assert g.DataOffset % alignment == 0
        assert g.GetString("general.architecture") == "llama"
        assert g.GetString("general.name") == "tiny ✓ model"
        assert g.GetString("missing", "dflt") == "dflt"
        assert g.GetUint32("llama.block_count") == 2
        assert g.GetUint32("general.alignment", 32) == alignment
        assert g.Metadata["test.i32"] == -7 and g.Metadata["test.u8"] == 200 and g.Metadata["test.i8"] == -100
        assert g.Metadata["test.u16"] == 65000 and g.Metadata["test.i16"] == -30000
        assert g.Metadata["test.u64"] == 1 << 40 and g.Metadata["test.i64"] == -(1 << 41)
        assert g.GetFloat32("llama.attention.layer_norm_rms_epsilon") == float(np.float32(1e-5))
        assert g.Metadata["test.f64"] == 0.1
        assert g.GetBool("test.flag") is True and g.GetBool("absent", False) is False
        assert g.GetStringArray("tokenizer.ggml.tokens") == ["<s>", "</s>", "hello", "wörld"]
        np.testing.assert_array_equal(g.GetFloatArray("tokenizer.ggml.scores"), np.array([0, -1.5, 2.25, -1000], np.float32))
        np.testing.assert_array_equal(g.GetInt32Array("tokenizer.ggml.token_type"), [3, 3, 1, 1])
        np.testing.assert_array_equal(g.GetInt32Array("test.u32s"), np.array([1, 2, 4000000000], np.uint32).astype(np.int32))
        assert g.GetUint32("test.u32s") == 1
        assert set(g.Tensors) == set(TENSORS)
        for name, (t, shape) in TENSORS.items():
            info = g.Tensors[name]
            assert info.Type == t and info.Shape == shape and info.NumElements == int(np.prod(shape))
            assert info.Offset % 32 == 0
            assert g.GetTensorByteCount(info) == expect[name].size
            np.testing.assert_array_equal(g.tensor_data(name), expect[name])
        w = g.quantized_weight("blk.0.attn_q.weight")
        assert (w.ggml_type, w.ne0, w.ne1, w.raw_bytes) == (12, 256, 24, 24 * 144)
        with pytest.raises(KeyError):
            g.quantized_weight("missing")


def test_tensor_bytes_dequantize_like_the_oracle(oracle, expect):
    # the bytes in the file are the reference quantizers' bytes: the oracle reads them back to the seeded values' grid
    with GgufFile(os.path.join(GOLD, "tiny.gguf")) as g:
        for name in ("token_embd.weight", "blk.0.attn_q.weight", "blk.0.ffn_down.weight", "output.weight"):
            info = g.Tensors[name]
            y = oracle.dequantize(info.Type, np.array(g.tensor_data(name)))
            assert y.size == info.NumElements and np.all(np.isfinite(y)) and 0.01 < y.std() < 0.1


def test_sizes_follow_the_reference_table():
    # GgufReader.cs:326-369
    for t, want in {0: 4, 1: 2, 30: 2, 2: 18, 3: 20, 6: 22, 7: 24, 8: 34, 9: 36, 10: 84, 11: 110, 12: 144, 13: 176, 14: 210, 15: 292,
                    20: 18, 23: 136, 39: 17, 24: 1, 27: 8}.items():
        assert GgufFile.GetTypeSize(t) == want
    assert GgufFile.GetBlockSize(8) == 32 and GgufFile.GetBlockSize(12) == 256 and GgufFile.GetBlockSize(0) == 1
    assert GgufFile.GetBlockSize(39) == 32 and GgufFile.GetBlockSize(1000) == 256
    assert GgufFile.GetRowBytes(12, 4096) == 16 * 144 and GgufFile.GetRowBytes(39, 2880) == 1530
    with pytest.raises(NotImplementedError):
        GgufFile.GetTypeSize(1000)


def test_rejects_bad_files(tmp_path):
    p = tmp_path / "bad.gguf"
    p.write_bytes(b"GGML" + bytes(28))
    with pytest.raises(ValueError, match="Not a GGUF file"):
        GgufFile(str(p))
    p.write_bytes(struct.pack("<IIQQ", 0x46554747, 1, 0, 0))
    with pytest.raises(NotImplementedError, match="version 1"):
        GgufFile(str(p))
    whole = open(os.path.join(GOLD, "tiny.gguf"), "rb").read()
    p.write_bytes(whole[:300])
    with pytest.raises(ValueError, match="truncated"):
        GgufFile(str(p))
    p.write_bytes(whole[:-100])
    with GgufFile(str(p)) as g:
        with pytest.raises(ValueError, match="past the end"):
            g.tensor_data("output.weight")


@pytest.mark.parametrize("alignment", [0, 24])
def test_rejects_an_alignment_that_is_not_a_power_of_two(tmp_path, alignment):
    # header, then one u32 key "general.alignment" (value type 4 = UINT32)
    key = b"general.alignment"
    blob = struct.pack("<IIQQ", 0x46554747, 3, 0, 1) + struct.pack("<Q", len(key)) + key + struct.pack("<II", 4, alignment)
    p = tmp_path / "align.gguf"
    p.write_bytes(blob)
    with pytest.raises(ValueError, match="power of two"):
        GgufFile(str(p))


# ---- a MoE file: expert stacks as 3-D tensors (written by the reference's writer, tests/golden/make_golden_gguf.py) ----
MOE_E, MOE_H, MOE_F = 4, 64, 32


@pytest.fixture(scope="module")
def moe_expect():
    z = np.load(os.path.join(GOLD, "tiny_moe_gguf_expect.npz"))
    return {k.replace("__", "."): z[k] for k in z.files}


def test_expert_stacks_split_per_expert_like_the_reference(moe_expect):
    """ModelBase.cs:554-595: expert e of a 3-D `*_exps.` tensor is the view at e * (bytes / experts) of the mapping,
    stored under `<base>.<e>.weight`."""
    from tensorsharp_amd.hip_basic_ops import QuantizedWeight
    with GgufFile(os.path.join(GOLD, "tiny_moe.gguf")) as g:
        assert g.GetString("general.architecture") == "gpt-oss"
        assert g.GetUint32("gpt-oss.expert_count") == MOE_E and g.GetUint32("gpt-oss.expert_used_count") == 2
        info = g.Tensors["blk.0.ffn_gate_exps.weight"]
        assert info.Shape == (MOE_H, MOE_F, MOE_E) and info.Type == 39
        assert g.GetTensorByteCount(info) == MOE_E * MOE_F * 34 == moe_expect["blk.0.ffn_gate_exps.weight"].size
        assert g.Tensors["blk.0.ffn_gate_inp.bias"].Shape == (MOE_E,)
        with pytest.raises(ValueError, match="stack of experts"):
            g.quantized_weight("blk.0.ffn_gate_exps.weight")
        with pytest.raises(ValueError, match="not a stack"):
            g.expert_weights("blk.0.ffn_gate_inp.weight")
        for name in ("blk.0.ffn_gate_exps.weight", "blk.0.ffn_down_exps.weight", "blk.1.ffn_up_exps.weight", "blk.1.ffn_down_exps.weight"):
            info = g.Tensors[name]
            ex = g.expert_weights(name)
            whole = moe_expect[name]
            per = whole.size // MOE_E
            assert len(ex) == MOE_E
            for e, w in enumerate(ex):
                assert (w.ggml_type, w.ne0, w.ne1, w.raw_bytes) == (info.Type, info.Shape[0], info.Shape[1], per)
                assert w.HasExternalHostView
                np.testing.assert_array_equal(np.array(w.data), whole[e * per:(e + 1) * per])
            # adjacent views of one mapping: the stack is one view again, no copy
            stacked = QuantizedWeight.TryCreateConcatenatedView(*ex)
            assert stacked is not None and stacked.ptr == ex[0].ptr and stacked.ne1 == MOE_E * info.Shape[1]
            np.testing.assert_array_equal(np.array(stacked.data), whole)
        ws = g.load_quantized_weights()
        want = {f"blk.{l}.ffn_{p}_exps.{e}.weight" for l in (0, 1) for p in ("gate", "up", "down") for e in range(MOE_E)}
        assert set(ws) == want          # the F32 router and biases are not stored as blocks
        b = g.float_tensor("blk.0.ffn_down_exps.bias")
        assert b.shape == (MOE_E, MOE_H)
        np.testing.assert_array_equal(b.reshape(-1), moe_expect["blk.0.ffn_down_exps.bias"].view(np.float32))


def test_gate_up_fusion_per_expert_and_bias_split(moe_expect):
    """GptOssModel.cs:93-180: biases [E, n] are split per expert, gate and up of an expert are stacked (a copy: they live
    in different tensors), and the per-expert stacks put together are the operand of the grouped expert stage."""
    from tensorsharp_amd.hip_basic_ops import FuseExpertGateUpWeights, SplitExpertBiases, StackExpertWeights
    with GgufFile(os.path.join(GOLD, "tiny_moe.gguf")) as g:
        ws = g.load_quantized_weights()
        fl = {n: g.float_tensor(n) for n in g.Tensors if n.endswith(".bias") and "_exps" in n}
        assert SplitExpertBiases(fl, 2) == 3
        assert fl["blk.0.ffn_up_exps.2.bias"].shape == (1, MOE_F)
        assert FuseExpertGateUpWeights(ws, 2, MOE_E, fl) == 2 * MOE_E
        assert "blk.0.ffn_gate_exps.0.weight" not in ws and "blk.0.ffn_up_exps.0.bias" not in fl
        gate, up = moe_expect["blk.0.ffn_gate_exps.weight"], moe_expect["blk.0.ffn_up_exps.weight"]
        per = gate.size // MOE_E
        for e in range(MOE_E):
            w = ws[f"blk.0.ffn_gate_up_exps.{e}.weight"]
            assert (w.ne0, w.ne1, w.raw_bytes) == (MOE_H, 2 * MOE_F, 2 * per) and w.ptr % 64 == 0 and not w.HasExternalHostView
            np.testing.assert_array_equal(w.data[:per], gate[e * per:(e + 1) * per])
            np.testing.assert_array_equal(w.data[per:], up[e * per:(e + 1) * per])
            fb = fl[f"blk.0.ffn_gate_up_exps.{e}.bias"]
            assert fb.shape == (1, 2 * MOE_F)
            np.testing.assert_array_equal(fb[0, :MOE_F], moe_expect["blk.0.ffn_gate_exps.bias"].view(np.float32)[e * MOE_F:(e + 1) * MOE_F])
        gu = StackExpertWeights([ws[f"blk.0.ffn_gate_up_exps.{e}.weight"] for e in range(MOE_E)])
        assert gu.ne1 == MOE_E * 2 * MOE_F and gu.raw_bytes == 2 * gate.size
        dn = StackExpertWeights([ws[f"blk.0.ffn_down_exps.{e}.weight"] for e in range(MOE_E)])
        assert dn.HasExternalHostView                           # still a view of the mapping
        np.testing.assert_array_equal(np.array(dn.data), moe_expect["blk.0.ffn_down_exps.weight"])
