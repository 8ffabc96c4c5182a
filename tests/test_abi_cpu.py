"""C-ABI surface checks that need no GPU: the library loads, exports every symbol the header
declares, keeps the bridge's struct layout, and fails loudly (never silently) without a device."""
import ctypes as C
import os
import re

import numpy as np
import pytest

from tensorsharp_amd import hip_native as N

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_exports():
    text = open(os.path.join(ROOT, "include", "tship_ops.h")).read()
    return sorted(set(re.findall(r"TSHIP_EXPORT[^;]*?\b(TSHip_\w+)\s*\(", text)))


def test_every_declared_symbol_is_exported_and_bound():
    names = declared_exports()
    assert len(names) >= 16
    lib = N.lib()
    for n in names:
        assert hasattr(lib, n), f"{n} declared in tship_ops.h but not exported"
        assert n in N.SIGNATURES, f"{n} has no ctypes signature in hip_native.py"
    assert sorted(N.SIGNATURES) == names


def test_struct_layout_matches_bridge():
    # TensorView2DDesc is 32 bytes, ContiguousTensorDesc 24 (ggml_ops_internal.h:69-109)
    assert C.sizeof(N.TensorView2D) == 32
    assert N.TensorView2D.raw_bytes.offset == 24
    assert C.sizeof(N.ContiguousTensor) == 24


def test_row_size_contract():
    f = N.lib().TSHip_RowSize
    assert f(N.TYPE_Q8_0, 2560) == 80 * 34
    assert f(N.TYPE_Q4_K, 4096) == 16 * 144
    assert f(N.TYPE_MXFP4, 2880) == 90 * 17
    assert f(N.TYPE_F32, 7) == 28
    # 0 on unknown type, non-positive ne, ne not a block multiple (ggml_ops_core.cpp:1320-1329)
    assert f(N.TYPE_Q4_K, 4000) == 0
    assert f(N.TYPE_Q8_0, 0) == 0
    assert f(N.TYPE_Q8_0, -32) == 0
    assert f(1234, 256) == 0


def test_aligned_alloc():
    lib = N.lib()
    p = lib.TSHip_AlignedAlloc(1000)
    assert p and p % 16384 == 0
    lib.TSHip_AlignedFree(p)
    assert lib.TSHip_AlignedAlloc(0) is None
    lib.TSHip_AlignedFree(None)


def test_backend_ids():
    lib = N.lib()
    for other in (1, 2, 3, 0, 99):
        assert lib.TSHip_CanInitializeBackend(other) == 0
        assert lib.TSHip_IsBackendAvailable(other) == 0


def _no_gpu():
    import torch
    return not torch.cuda.is_available()


@pytest.mark.skipif(not _no_gpu(), reason="checks the no-device behaviour")
def test_compute_calls_fail_loudly_without_a_device():
    from tensorsharp_amd import HipBasicOps
    lib = N.lib()
    assert lib.TSHip_IsBackendAvailable(N.BACKEND_HIP) == 0
    assert "HIP device" in N.get_last_error()
    w = np.zeros(34 * 4, dtype=np.uint8)
    x = np.zeros((1, 64), dtype=np.float32)
    y = np.zeros((1, 2), dtype=np.float32)
    with pytest.raises(RuntimeError, match="addmm_quant failed"):
        HipBasicOps.AddmmQuant(y, x, w.ctypes.data, N.TYPE_Q8_0, 64, 2, w.size)
    with pytest.raises(RuntimeError):
        HipBasicOps.DequantizeToFloat32(N.TYPE_Q8_0, w, 128)
    # argument errors that are decided before the device is touched keep the bridge's codes
    assert lib.TSHip_DequantizeToF32(N.TYPE_Q8_0, None, 32, y.ctypes.data) == -1
    assert lib.TSHip_DequantizeToF32(77, w.ctypes.data, 32, y.ctypes.data) == -2
    assert lib.TSHip_DequantizeToF32(N.TYPE_Q8_0, w.ctypes.data, 0, y.ctypes.data) == 0


def test_facade_argument_errors_mirror_the_reference():
    from tensorsharp_amd import HipBasicOps
    w = np.zeros(34 * 4, dtype=np.uint8)
    with pytest.raises(ValueError, match="2D"):
        HipBasicOps.AddmmQuant(np.zeros(4, np.float32), np.zeros((1, 64), np.float32), w.ctypes.data, 8, 64, 2, w.size)
    with pytest.raises(ValueError, match="Float32"):
        HipBasicOps.AddmmQuant(np.zeros((1, 2), np.float64), np.zeros((1, 64), np.float32), w.ctypes.data, 8, 64, 2, w.size)
    with pytest.raises(NotImplementedError):      # result must be row-contiguous (TryCreateStandardView)
        HipBasicOps.AddmmQuant(np.zeros((1, 4), np.float32)[:, ::2], np.zeros((1, 64), np.float32), w.ctypes.data, 8, 64, 2, w.size)
    with pytest.raises(NotImplementedError, match="block size"):
        HipBasicOps.GetRowSizeBytes(N.TYPE_Q4_K, 100)


def test_sync_host_buffer_is_a_no_op_for_pointers_that_were_never_cached():
    # ggml_ops_core.cpp:664-684: null pointer, zero size or an uncached pointer -> success, nothing copied
    lib = N.lib()
    a = np.arange(8, dtype=np.float32)
    assert lib.TSHip_SyncHostBuffer(a.ctypes.data, a.nbytes) == 1
    assert lib.TSHip_SyncHostBuffer(None, 16) == 1
    assert lib.TSHip_SyncHostBuffer(a.ctypes.data, 0) == 1
    assert N.get_last_error() == ""
    assert np.array_equal(a, np.arange(8, dtype=np.float32))


# ---- the managed P/Invoke file declares the same argument lists as the header ----------------------------------
def _c_params(decl):
    """argument kinds of one C declaration: 'ptr', 'i32', 'i64', 'f32', 'size', or a struct name"""
    out = []
    for p in decl.split(","):
        p = " ".join(p.split())
        if not p or p == "void":
            continue
        if "*" in p:
            out.append("ptr")
            continue
        ty = " ".join(p.split(" ")[:-1]).replace("const ", "")
        out.append({"int": "i32", "int64_t": "i64", "float": "f32", "size_t": "size", "TSHipTensorView2D": "view2",
                    "TSHipTensorView3D": "view3", "TSHipContiguousTensor": "contig"}[ty])
    return out


def _cs_params(decl):
    out = []
    for p in decl.split(","):
        p = " ".join(p.split())
        if not p:
            continue
        ty = p.split(" ")[0]
        out.append({"IntPtr": "ptr", "IntPtr[]": "ptr", "long[]": "ptr", "float[]": "ptr", "int": "i32", "long": "i64",
                    "float": "f32", "UIntPtr": "size", "HipTensorView2D": "view2", "HipTensorView3D": "view3",
                    "HipContiguousTensor": "contig"}[ty])
    return out


def test_managed_pinvoke_declarations_match_the_header():
    header = open(os.path.join(ROOT, "include", "tship_ops.h")).read()
    cs = open(os.path.join(ROOT, "managed", "TensorSharp.Backends.HIP", "HipNative.cs")).read()
    c_decls = {m.group(1): _c_params(m.group(2))
               for m in re.finditer(r"TSHIP_EXPORT[^;(]*?\b(TSHip_\w+)\s*\(([^;]*?)\)\s*;", header, re.S)}
    cs_decls = {m.group(1): _cs_params(m.group(2))
                for m in re.finditer(r"static extern \S+ (TSHip_\w+)\s*\(([^;]*?)\)\s*;", cs, re.S)}
    assert len(cs_decls) >= 25
    for name, params in cs_decls.items():
        assert name in c_decls, f"{name} bound in HipNative.cs but not declared in tship_ops.h"
        assert params == c_decls[name], f"{name}: managed {params} != header {c_decls[name]}"
    # every host-pointer export is bound (the *Device family, SetStream and the profiling switch serve native callers that
    # own device memory)
    native_only = ("TSHip_SetStream", "TSHip_SetGemvTimeline")
    unbound = [n for n in c_decls if n not in cs_decls and not n.endswith("Device") and "NoAlloc" not in n and n not in native_only]
    assert unbound == [], unbound


def test_struct_layout_3d_view():
    assert C.sizeof(N.TensorView3D) == 40 and N.TensorView3D.raw_bytes.offset == 32
