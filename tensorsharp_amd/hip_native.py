"""ctypes bindings of libTsHipOps.so — the Python twin of a `HipNative.cs` P/Invoke class.

Mirrors TensorSharp.Backends.GGML/GgmlNative.cs: same struct layouts (GgmlNative.cs:27-132),
structs passed by value, int 1/0 results checked by `check_result` which raises with the
library's last error (GgmlNative.cs:1539-1547, :1622-1627).  The library is loaded from
this package directory only; there is no CPU fallback — a missing library raises.
"""
import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libTsHipOps.so")

BACKEND_HIP = 4
TYPE_F32, TYPE_Q8_0, TYPE_Q4_K, TYPE_MXFP4 = 0, 8, 12, 39
TYPE_Q8_1 = 9
TYPE_F16, TYPE_Q4_0, TYPE_Q4_1, TYPE_Q5_0, TYPE_Q5_1, TYPE_Q5_K, TYPE_Q6_K, TYPE_IQ4_NL, TYPE_BF16 = 1, 2, 3, 6, 7, 13, 14, 20, 30
DTYPE_F32, DTYPE_I32 = 0, 3


class TensorView2D(C.Structure):
    """GgmlTensorView2D (GgmlNative.cs:27-45): strides in elements, raw_bytes = span in bytes."""
    _fields_ = [("data", C.c_void_p), ("dim0", C.c_int), ("dim1", C.c_int), ("stride0", C.c_int),
                ("stride1", C.c_int), ("raw_bytes", C.c_int64)]


class TensorView3D(C.Structure):
    """GgmlTensorView3D (GgmlNative.cs:49-71): strides in elements, raw_bytes = span in bytes."""
    _fields_ = [("data", C.c_void_p), ("dim0", C.c_int), ("dim1", C.c_int), ("dim2", C.c_int), ("stride0", C.c_int),
                ("stride1", C.c_int), ("stride2", C.c_int), ("raw_bytes", C.c_int64)]


class ContiguousTensor(C.Structure):
    """GgmlContiguousTensor (GgmlNative.cs:100-113)."""
    _fields_ = [("data", C.c_void_p), ("element_count", C.c_int64), ("element_type", C.c_int)]


class NativeLibraryMissing(RuntimeError):
    """Twin of DllNotFoundException: the HIP library has not been built."""


_lib = None

# name -> (restype, argtypes); one line per export declared in include/tship_ops.h
SIGNATURES = {
    "TSHip_GetLastError": (C.c_char_p, []),
    "TSHip_CanInitializeBackend": (C.c_int, [C.c_int]),
    "TSHip_IsBackendAvailable": (C.c_int, [C.c_int]),
    "TSHip_RowSize": (C.c_size_t, [C.c_int, C.c_int64]),
    "TSHip_AlignedAlloc": (C.c_void_p, [C.c_size_t]),
    "TSHip_AlignedFree": (None, [C.c_void_p]),
    "TSHip_DequantizeToF32": (C.c_int, [C.c_int, C.c_void_p, C.c_int64, C.c_void_p]),
    "TSHip_AddmmQuantF32": (C.c_int, [TensorView2D, TensorView2D, C.c_void_p, C.c_int, C.c_int64, C.c_int64,
                                      C.c_int64]),
    "TSHip_AddmmQuantBatchF32": (C.c_int, [TensorView2D, TensorView2D, C.c_void_p, C.c_int, C.c_int64, C.c_int64,
                                           C.c_int, C.POINTER(C.c_int64), C.POINTER(C.c_int64)]),
    "TSHip_PreloadQuantizedWeight": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.c_int64, C.c_int64, C.c_int64]),
    "TSHip_InvalidateHostBuffer": (None, [C.c_void_p]),
    "TSHip_ClearHostBufferCache": (None, []),
    "TSHip_SyncHostBuffer": (C.c_int, [C.c_void_p, C.c_size_t]),
    "TSHip_SetStream": (C.c_int, [C.c_void_p]),
    "TSHip_DequantizeToF32Device": (C.c_int, [C.c_int, C.c_void_p, C.c_int64, C.c_void_p]),
    "TSHip_AddmmQuantF32Device": (C.c_int, [TensorView2D, TensorView2D, C.c_void_p, C.c_int, C.c_int64, C.c_int64,
                                            C.c_int64]),
    "TSHip_AddmmQuantF32DeviceNoAlloc": (C.c_int, [TensorView2D, TensorView2D, C.c_void_p, C.c_int, C.c_int64, C.c_int64,
                                                   C.c_int64]),
    "TSHip_AddmmQuantGroupF32Device": (C.c_int, [C.c_int, C.POINTER(TensorView2D), C.POINTER(TensorView2D),
                                                 C.POINTER(C.c_void_p), C.c_int, C.POINTER(C.c_int64),
                                                 C.POINTER(C.c_int64), C.POINTER(C.c_int64)]),
    "TSHip_FusedRmsNormMatMulQuantF32": (C.c_int, [TensorView2D, TensorView2D, C.c_void_p, C.c_int, C.c_float, C.c_void_p,
                                                   C.c_int, C.c_int64, C.c_int64, C.c_int64]),
    "TSHip_FusedMatMulQuantAddF32": (C.c_int, [TensorView2D, TensorView2D, C.c_void_p, C.c_int, C.c_int64, C.c_int64,
                                               C.c_int64]),
    "TSHip_FusedFFNSwiGLUQuantF32": (C.c_int, [TensorView2D, TensorView2D, C.c_void_p, C.c_int, C.c_float,
                                               C.c_void_p, C.c_int, C.c_int64, C.c_int64, C.c_int64,
                                               C.c_void_p, C.c_int, C.c_int64, C.c_int64, C.c_int64, C.c_int]),
    "TSHip_FusedRmsNormMatMulQuantF32Device": (C.c_int, [TensorView2D, TensorView2D, C.c_void_p, C.c_int, C.c_float,
                                                         C.c_void_p, C.c_int, C.c_int64, C.c_int64, C.c_int64]),
    "TSHip_FusedMatMulQuantAddF32Device": (C.c_int, [TensorView2D, TensorView2D, C.c_void_p, C.c_int, C.c_int64,
                                                     C.c_int64, C.c_int64]),
    "TSHip_FusedFFNSwiGLUQuantF32Device": (C.c_int, [TensorView2D, TensorView2D, C.c_void_p, C.c_int, C.c_float,
                                                     C.c_void_p, C.c_int, C.c_int64, C.c_int64, C.c_int64,
                                                     C.c_void_p, C.c_int, C.c_int64, C.c_int64, C.c_int64, C.c_int]),
    "TSHip_FusedOutProjFFNQuantF32": (C.c_int, [TensorView2D, TensorView2D, C.c_void_p, C.c_int, C.c_int64, C.c_int64, C.c_int64,
                                                C.c_void_p, C.c_int, C.c_float,
                                                C.c_void_p, C.c_int, C.c_int64, C.c_int64, C.c_int64,
                                                C.c_void_p, C.c_int, C.c_int64, C.c_int64, C.c_int64, C.c_int]),
    "TSHip_FusedOutProjNormRouterQuantF32": (C.c_int, [TensorView2D, TensorView2D, C.c_void_p, C.c_int, C.c_int64, C.c_int64,
                                                       C.c_int64, C.c_void_p, C.c_int, C.c_float, TensorView2D,
                                                       C.c_void_p, C.c_int, C.c_int64, C.c_int64, C.c_int64, TensorView2D]),
    "TSHip_MoEExpertsForwardF32": (C.c_int, [TensorView2D, TensorView2D, C.c_int, C.POINTER(C.c_void_p), C.POINTER(C.c_void_p),
                                             C.c_int, C.c_int64, C.c_int64, C.c_int64, C.c_int, C.c_int64, C.c_int64, C.c_int64,
                                             C.POINTER(C.c_float)]),
    "TSHip_MoEExpertsSwiGLUForwardF32": (C.c_int, [TensorView2D, TensorView2D, C.c_int, C.POINTER(C.c_void_p),
                                                   C.POINTER(C.c_void_p), C.POINTER(C.c_void_p),
                                                   C.c_int, C.c_int64, C.c_int64, C.c_int64, C.c_int, C.c_int64, C.c_int64, C.c_int64,
                                                   C.c_int, C.c_int64, C.c_int64, C.c_int64, C.POINTER(C.c_float)]),
    "TSHip_MoEExpertsSwiGLUResidualF32": (C.c_int, [TensorView2D, TensorView2D, C.c_int, C.POINTER(C.c_void_p),
                                                    C.POINTER(C.c_void_p), C.POINTER(C.c_void_p),
                                                    C.c_int, C.c_int64, C.c_int64, C.c_int64, C.c_int, C.c_int64, C.c_int64, C.c_int64,
                                                    C.c_int, C.c_int64, C.c_int64, C.c_int64, C.POINTER(C.c_float),
                                                    C.c_int, C.c_void_p, C.c_void_p, C.c_void_p,
                                                    C.c_int, C.c_int64, C.c_int64, C.c_int64, C.c_int, C.c_int64, C.c_int64, C.c_int64,
                                                    C.c_int, C.c_int64, C.c_int64, C.c_int64, C.c_float]),
    "TSHip_MulMatIdF32": (C.c_int, [TensorView3D, TensorView3D, TensorView3D, ContiguousTensor, C.c_int, C.c_int]),
    "TSHip_MulMatIdF32Device": (C.c_int, [TensorView3D, TensorView3D, TensorView3D, C.c_void_p, C.c_int, C.c_int]),
    "TSHip_SetGemvTimeline": (C.c_int, [C.c_void_p, C.c_int64]),
    "TSHip_AddIdF32": (C.c_int, [TensorView3D, TensorView3D, TensorView2D, ContiguousTensor, C.c_int, C.c_int]),
    "TSHip_AddIdF32Device": (C.c_int, [TensorView3D, TensorView3D, TensorView2D, C.c_void_p, C.c_int, C.c_int]),
    "TSHip_GetRowsQuantF32": (C.c_int, [TensorView2D, C.c_void_p, C.c_int, C.c_int64, C.c_int64, C.c_int64,
                                        ContiguousTensor]),
    "TSHip_GetRowsQuantF32Device": (C.c_int, [TensorView2D, C.c_void_p, C.c_int, C.c_int64, C.c_int64, C.c_int64,
                                              C.c_void_p, C.c_int64]),
    "TSHip_MoERouteF32Device": (C.c_int, [TensorView2D, C.c_int, C.c_void_p, C.c_void_p]),
    "TSHip_MoEExpertsGptOssForwardF32Device": (C.c_int, [TensorView2D, TensorView2D, C.c_void_p, C.c_void_p, C.c_int, C.c_void_p,
                                                   C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int64,
                                                   C.c_int64, C.c_float, C.c_float]),
    "TSHip_TransformerLayerDecodeDevice": (C.c_int, [
        C.c_void_p, C.c_int, C.c_void_p,
        C.c_void_p, C.c_int, C.c_int64, C.c_int64, C.c_int64,
        C.c_void_p, C.c_void_p, C.c_int,
        C.c_void_p, C.c_int, C.c_int64, C.c_int64, C.c_int64,
        C.c_void_p,
        C.c_void_p, C.c_int, C.c_int64, C.c_int64, C.c_int64,
        C.c_void_p, C.c_int, C.c_int64, C.c_int64, C.c_int64,
        C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_float, C.c_float, C.c_float, C.c_int, C.c_int]),
    "TSHip_TransformerModelDecodeDevice": (C.c_int, [
        C.c_void_p, C.c_int, C.c_int,
        C.POINTER(C.c_void_p), C.POINTER(C.c_void_p), C.POINTER(C.c_void_p), C.POINTER(C.c_void_p), C.POINTER(C.c_void_p),
        C.POINTER(C.c_void_p), C.POINTER(C.c_void_p), C.POINTER(C.c_void_p), C.POINTER(C.c_void_p), C.POINTER(C.c_void_p),
        C.c_int, C.c_int64, C.c_int64, C.c_int64, C.c_int, C.c_int64, C.c_int64, C.c_int64,
        C.c_int, C.c_int64, C.c_int64, C.c_int64, C.c_int, C.c_int64, C.c_int64, C.c_int64,
        C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_float, C.c_float, C.c_float, C.c_int, C.c_int]),
}
# the host-pointer forms take the same argument lists
for _name in ("TSHip_FusedOutProjFFNQuantF32", "TSHip_FusedOutProjNormRouterQuantF32", "TSHip_MoEExpertsForwardF32",
              "TSHip_MoEExpertsSwiGLUForwardF32", "TSHip_MoEExpertsSwiGLUResidualF32"):
    SIGNATURES[_name + "Device"] = SIGNATURES[_name]
SIGNATURES["TSHip_TransformerLayerDecode"] = SIGNATURES["TSHip_TransformerLayerDecodeDevice"]
SIGNATURES["TSHip_TransformerModelDecode"] = SIGNATURES["TSHip_TransformerModelDecodeDevice"]


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise NativeLibraryMissing(
                f"{LIB_PATH} not found: build it with `python -m tensorsharp_amd.build` (needs hipcc).")
        # PyTorch wheels ship their own copy of the HIP runtime.  Two HIP runtimes in one process cannot
        # both open the GPU, so when torch is installed its runtime is loaded first and this library
        # (which only asks for libamdhip64.so.7) binds to the same copy.  Without torch the system
        # runtime under /opt/rocm is used.
        try:
            import torch  # noqa: F401
        except ImportError:
            pass
        L = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            f = getattr(L, name)
            f.restype = res
            f.argtypes = args
        _lib = L
    return _lib


def get_last_error():
    msg = lib().TSHip_GetLastError()
    return msg.decode("utf-8", "replace") if msg else ""


def check_result(ok, what):
    """GgmlNative.CheckResult: 0 -> InvalidOperationException with the native message."""
    if ok == 0:
        raise RuntimeError(f"{what} failed: {get_last_error() or 'unknown native error'}")
