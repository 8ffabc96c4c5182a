"""Host logic: the QuantizedWeight twin (ModelBase.cs:24-202) and the load-time fusions built on it
(ModelBase.FuseGateUpWeights :768-802, FuseQKVWeights of the models).  No GPU: only TSHip_RowSize is called."""
import numpy as np
import pytest

from oracle.oracle import Q8_0, Q4_K
from tensorsharp_amd import QuantizedWeight, FuseGateUpWeights, FuseQKVWeights


class Owner:
    """stands for the GGUF mapping that keeps external views alive"""


def blocks(rng, t, rows, k):
    bs, bb = {Q8_0: (32, 34), Q4_K: (256, 144)}[t]
    return rng.integers(0, 256, rows * (k // bs) * bb, dtype=np.uint8)


def views(buf, owner, t, k, row_counts, gap=0):
    """external views of consecutive row groups inside buf, `gap` bytes apart"""
    bs, bb = {Q8_0: (32, 34), Q4_K: (256, 144)}[t]
    out, off = [], 0
    for n in row_counts:
        size = n * (k // bs) * bb
        out.append(QuantizedWeight.CreateExternalView(buf[off:off + size], t, k, n, owner))
        off += size + gap
    return out


def test_adjacent_views_of_one_owner_concatenate_without_a_copy():
    rng = np.random.default_rng(1)
    k = 256
    buf = blocks(rng, Q4_K, 7 + 5 + 3, k)
    owner = Owner()
    q, kk, v = views(buf, owner, Q4_K, k, [7, 5, 3])
    fused = QuantizedWeight.TryCreateConcatenatedView(q, kk, v)
    assert fused is not None and fused.ptr == q.ptr == buf.ctypes.data
    assert (fused.ne0, fused.ne1, fused.raw_bytes, fused.ggml_type) == (k, 15, buf.size, Q4_K)
    assert fused.HasExternalHostView and np.array_equal(fused.data, buf)
    assert QuantizedWeight.ConcatOrCreateCopy(q, kk, v).ptr == buf.ctypes.data          # the view is preferred
    # order matters: (k, q) are not adjacent in that order
    assert QuantizedWeight.TryCreateConcatenatedView(kk, q) is None
    assert QuantizedWeight.TryCreateConcatenatedView(q) is None                         # fewer than two


@pytest.mark.parametrize("why", ["gap", "other_owner", "owned", "type", "row_length"])
def test_views_that_do_not_qualify_are_copied(why):
    rng = np.random.default_rng(2)
    k = 256
    owner = Owner()
    if why == "gap":
        buf = blocks(rng, Q8_0, 20, k)
        a, b = views(buf, owner, Q8_0, k, [4, 6], gap=34)
    elif why == "other_owner":
        buf = blocks(rng, Q8_0, 10, k)
        a, _ = views(buf, owner, Q8_0, k, [4, 6])
        _, b = views(buf, Owner(), Q8_0, k, [4, 6])
    elif why == "owned":
        a = QuantizedWeight(blocks(rng, Q8_0, 4, k), Q8_0, k, 4)
        b = QuantizedWeight(blocks(rng, Q8_0, 6, k), Q8_0, k, 6)
    elif why == "type":
        buf = np.concatenate([blocks(rng, Q8_0, 4, k), blocks(rng, Q4_K, 6, k)])
        a = QuantizedWeight.CreateExternalView(buf[:4 * 8 * 34], Q8_0, k, 4, owner)
        b = QuantizedWeight.CreateExternalView(buf[4 * 8 * 34:], Q4_K, k, 6, owner)
    else:
        buf = np.concatenate([blocks(rng, Q8_0, 4, k), blocks(rng, Q8_0, 6, 2 * k)])
        a = QuantizedWeight.CreateExternalView(buf[:4 * 8 * 34], Q8_0, k, 4, owner)
        b = QuantizedWeight.CreateExternalView(buf[4 * 8 * 34:], Q8_0, 2 * k, 6, owner)
    assert QuantizedWeight.TryCreateConcatenatedView(a, b) is None
    if why in ("type", "row_length"):
        return      # the callers never concatenate these (FuseGateUpWeights checks type and ne0 first)
    fused = QuantizedWeight.ConcatOrCreateCopy(a, b)
    assert fused.ptr not in (a.ptr, b.ptr) and fused.ptr % 64 == 0 and not fused.HasExternalHostView
    assert (fused.ne1, fused.raw_bytes) == (10, a.raw_bytes + b.raw_bytes)
    assert np.array_equal(fused.data, np.concatenate([a.data, b.data]))


def test_release_and_cache_key():
    rng = np.random.default_rng(3)
    w = QuantizedWeight(blocks(rng, Q8_0, 4, 64), Q8_0, 64, 4)
    assert w.HasHostData and w.CacheKey == w.ptr
    key = w.EnsureDeviceCacheKey()
    assert key != w.ptr and w.EnsureDeviceCacheKey() == key and w.CacheKey == key
    w.ReleaseHostData()
    assert not w.HasHostData and w.ptr == key           # the matmul now receives the opaque key
    with pytest.raises(RuntimeError, match="released"):
        QuantizedWeight.ConcatOrCreateCopy(w, w)
    w.Dispose()
    with pytest.raises(RuntimeError):
        w.ptr
    with pytest.raises(ValueError):
        QuantizedWeight(blocks(rng, Q8_0, 3, 64), Q8_0, 64, 4)      # too few bytes for 4 rows
    with pytest.raises(ValueError):
        QuantizedWeight.CreateExternalView(blocks(rng, Q8_0, 4, 64), Q8_0, 64, 4, None)


def test_fuse_gate_up_and_qkv_rename_and_dispose():
    rng = np.random.default_rng(4)
    k, owner = 256, Owner()
    weights = {}
    srcs = {}
    for layer in range(3):
        buf = blocks(rng, Q4_K, 8 + 8, k)
        g, u = views(buf, owner, Q4_K, k, [8, 8])
        weights[f"blk.{layer}.ffn_gate.weight"], weights[f"blk.{layer}.ffn_up.weight"] = g, u
        srcs[layer] = (buf, g, u)
    # layer 1: a type mismatch keeps the two apart; layer 2: the up projection is missing
    weights["blk.1.ffn_up.weight"] = QuantizedWeight(blocks(rng, Q8_0, 8, k), Q8_0, k, 8)
    del weights["blk.2.ffn_up.weight"]
    assert FuseGateUpWeights(weights, 3) == 1
    assert sorted(weights) == ["blk.0.ffn_gate_up.weight", "blk.1.ffn_gate.weight", "blk.1.ffn_up.weight", "blk.2.ffn_gate.weight"]
    fused = weights["blk.0.ffn_gate_up.weight"]
    assert fused.ne1 == 16 and np.array_equal(fused.data, srcs[0][0])              # gate rows first, then up rows
    assert not srcs[0][1].HasHostData and not srcs[0][2].HasHostData                # the originals were disposed
    qkv = {}
    buf = blocks(rng, Q8_0, 12 + 4 + 4, k)
    for name, w in zip("qkv", views(buf, owner, Q8_0, k, [12, 4, 4])):
        qkv[f"blk.0.attn_{name}.weight"] = w
    assert FuseQKVWeights(qkv, 1) == 1 and list(qkv) == ["blk.0.attn_qkv.weight"]
    assert qkv["blk.0.attn_qkv.weight"].ne1 == 20 and qkv["blk.0.attn_qkv.weight"].ptr == buf.ctypes.data
