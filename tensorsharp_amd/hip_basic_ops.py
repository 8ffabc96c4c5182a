"""Host-side operator facade of the HIP backend — the Python twin of a `HipBasicOps` class.

Names, argument meaning and error behaviour follow the quantized entry points of
TensorSharp.Backends.GGML/GgmlBasicOps.cs (:313-329 AddmmQuant, :689-704 AddmmQuantBatch,
:706-709 PreloadQuantizedWeight) and GgmlGgufTensorDequant.cs (:9-33 row size, :36-86 dequant).
ArgumentException -> ValueError, NotSupportedException -> NotImplementedError,
InvalidOperationException (native failure) -> RuntimeError.

Host tensors are numpy float32 arrays (the reference's tensors are host memory); device
tensors are torch CUDA tensors, which only supply memory and the stream.
"""
import ctypes as C

import numpy as np

from . import hip_native as N


class QuantizedWeight:
    """Raw GGUF blocks of one 2-D weight: twin of ModelBase.QuantizedWeight (TensorSharp.Models/ModelBase.cs:24-202).

    data        numpy uint8 array (host) or torch uint8 CUDA tensor (device) holding ne1 rows of row_size(type, ne0) bytes
    cache_key   the pointer the matmul entry points take as m2_data: the host address, or - after
                EnsureDeviceCacheKey() - an opaque key that stays valid once the host bytes are released
    An instance either owns its bytes (built from an array, or a concatenated copy) or is an external view of a larger
    buffer kept alive by `owner_token` (the GGUF mapping); adjacent external views of one owner concatenate without
    a copy."""

    def __init__(self, data, ggml_type, ne0, ne1, owner_token=None):
        self.ggml_type = int(ggml_type)
        self.ne0 = int(ne0)   # K, in features
        self.ne1 = int(ne1)   # N, out features
        self.data = data
        self.raw_bytes = int(data.numel() if hasattr(data, "numel") else data.size)
        self._owner_token = owner_token
        self._owns_buffer = owner_token is None
        self._key = None      # opaque device cache key (EnsureDeviceCacheKey)
        expect = HipBasicOps.GetRowSizeBytes(self.ggml_type, self.ne0) * self.ne1
        if self.raw_bytes < expect:
            raise ValueError(f"weight bytes {self.raw_bytes} < {expect} for {ne1}x{ne0} type {ggml_type}")

    # -- storage -----------------------------------------------------------------------------
    @property
    def is_device(self):
        return hasattr(self.data, "data_ptr")

    @property
    def HasHostData(self):
        return self.data is not None and not self.is_device

    @property
    def HasExternalHostView(self):
        return self.HasHostData and not self._owns_buffer and self._owner_token is not None

    @property
    def ptr(self):
        """what the matmul entry points receive: the cache key when the bytes were released, else the data address"""
        if self.data is None:
            if self._key is None:
                raise RuntimeError("Quantized weight has neither host data nor a device cache key.")
            return self._key
        return self.data.data_ptr() if self.is_device else self.data.ctypes.data

    @property
    def CacheKey(self):
        return self._key if self._key is not None else (0 if self.data is None else self.ptr)

    @staticmethod
    def AllocateBuffer(size):
        """64-byte aligned host bytes (ModelBase.cs:189-195)"""
        raw = np.empty(int(size) + 64, dtype=np.uint8)
        off = (-raw.ctypes.data) % 64
        return raw[off:off + int(size)]

    @staticmethod
    def CreateExternalView(data, ggml_type, ne0, ne1, owner_token):
        """A view of bytes owned by `owner_token` (ModelBase.cs:82-90)."""
        if data is None or (hasattr(data, "size") and data.size == 0):
            raise ValueError("External quantized weight view requires a non-empty data view.")
        if owner_token is None:
            raise ValueError("ownerToken must not be None.")
        return QuantizedWeight(data, ggml_type, ne0, ne1, owner_token=owner_token)

    @staticmethod
    def TryCreateConcatenatedView(*weights):
        """One weight of ne1 = sum(ne1) over byte-adjacent external views of the same owner, type and row length; None when
        the views do not qualify (ModelBase.cs:92-126)."""
        if len(weights) < 2 or weights[0] is None:
            return None
        first = weights[0]
        if not first.HasHostData or first._owns_buffer or first._owner_token is None:
            return None
        total_bytes = total_ne1 = 0
        expected = first.ptr
        for w in weights:
            if (w is None or not w.HasHostData or w._owns_buffer or w._owner_token is not first._owner_token or
                    w.ggml_type != first.ggml_type or w.ne0 != first.ne0 or w.ptr != expected):
                return None
            total_bytes += w.raw_bytes
            total_ne1 += w.ne1
            expected += w.raw_bytes
        span = (C.c_uint8 * total_bytes).from_address(first.ptr)
        data = np.frombuffer(span, dtype=np.uint8)
        fused = QuantizedWeight(data, first.ggml_type, first.ne0, total_ne1, owner_token=first._owner_token)
        fused._keepalive = [w.data for w in weights]     # the span borrows these views' memory
        return fused

    @staticmethod
    def ConcatOrCreateCopy(*weights):
        """Rows of the weights stacked in order: a view when they are adjacent in one mapping, else a copy into a fresh
        aligned buffer (ModelBase.cs:128-159)."""
        if len(weights) == 0 or weights[0] is None:
            raise ValueError("At least one quantized weight is required.")
        fused = QuantizedWeight.TryCreateConcatenatedView(*weights)
        if fused is not None:
            return fused
        first = weights[0]
        total = 0
        for w in weights:
            if w is None:
                raise ValueError("Quantized weight list cannot contain null entries.")
            if not w.HasHostData:
                raise RuntimeError("Cannot concatenate quantized weights after their host storage has been released.")
            total += w.raw_bytes
        buf = QuantizedWeight.AllocateBuffer(total)
        off = 0
        for w in weights:
            buf[off:off + w.raw_bytes] = w.data.reshape(-1)
            off += w.raw_bytes
        return QuantizedWeight(buf, first.ggml_type, first.ne0, sum(w.ne1 for w in weights))

    def EnsureDeviceCacheKey(self):
        """An opaque key for PreloadQuantizedWeight that outlives the host bytes (ModelBase.cs:161-170: a GCHandle there,
        the address of a small pinned-by-reference buffer here)."""
        if self._key is None:
            self._key_anchor = np.zeros(1, dtype=np.uint8)
            self._key = self._key_anchor.ctypes.data
        return self._key

    def ReleaseHostData(self):
        """Drop the host bytes (ModelBase.cs:172-187); the weight stays usable through its device cache key."""
        self.data = None
        self._owns_buffer = False
        self._owner_token = None
        self._keepalive = None

    def Dispose(self):
        self.ReleaseHostData()
        self._key = None


def FuseGateUpWeights(quant_weights, num_layers):
    """Twin of ModelBase.FuseGateUpWeights (ModelBase.cs:768-802) for the quantized branch: blk.L.ffn_gate.weight and
    blk.L.ffn_up.weight of equal type and row length become blk.L.ffn_gate_up.weight (gate rows, then up rows); the two
    originals are removed and disposed.  Returns the number of layers fused."""
    fused = 0
    for layer in range(int(num_layers)):
        gate_name, up_name = f"blk.{layer}.ffn_gate.weight", f"blk.{layer}.ffn_up.weight"
        gw, uw = quant_weights.get(gate_name), quant_weights.get(up_name)
        if gw is None or uw is None or gw.ggml_type != uw.ggml_type or gw.ne0 != uw.ne0:
            continue
        quant_weights[f"blk.{layer}.ffn_gate_up.weight"] = QuantizedWeight.ConcatOrCreateCopy(gw, uw)
        del quant_weights[gate_name], quant_weights[up_name]
        gw.Dispose()
        uw.Dispose()
        fused += 1
    return fused


def FuseExpertGateUpWeights(quant_weights, num_layers, num_experts, biases=None):
    """Twin of GptOssModel.FuseExpertGateUpWeights (GptOssModel.cs:126-180): per layer and expert,
    blk.L.ffn_gate_exps.E.weight and blk.L.ffn_up_exps.E.weight of equal type and row length become
    blk.L.ffn_gate_up_exps.E.weight (gate rows, then up rows; a copy, since gate and up live in different tensors of the
    file).  `biases` (name -> float32 array [1, n], the split biases of GptOssModel.cs:95-121) are fused the same way.
    Returns the number of experts fused."""
    fused = 0
    for layer in range(int(num_layers)):
        for e in range(int(num_experts)):
            gate_name, up_name = f"blk.{layer}.ffn_gate_exps.{e}.weight", f"blk.{layer}.ffn_up_exps.{e}.weight"
            gw, uw = quant_weights.get(gate_name), quant_weights.get(up_name)
            if gw is not None and uw is not None and gw.ggml_type == uw.ggml_type and gw.ne0 == uw.ne0:
                quant_weights[f"blk.{layer}.ffn_gate_up_exps.{e}.weight"] = QuantizedWeight.ConcatOrCreateCopy(gw, uw)
                del quant_weights[gate_name], quant_weights[up_name]
                gw.Dispose()
                uw.Dispose()
                fused += 1
            if biases is not None:
                gb_name, ub_name = f"blk.{layer}.ffn_gate_exps.{e}.bias", f"blk.{layer}.ffn_up_exps.{e}.bias"
                if gb_name in biases and ub_name in biases:
                    biases[f"blk.{layer}.ffn_gate_up_exps.{e}.bias"] = np.concatenate(
                        [biases.pop(gb_name).reshape(1, -1), biases.pop(ub_name).reshape(1, -1)], axis=1)
    return fused


def SplitExpertBiases(float_weights, num_layers):
    """Twin of GptOssModel.SplitExpertBiases (GptOssModel.cs:93-124): blk.L.ffn_{gate,up,down}_exps.bias [E, n] become
    blk.L.ffn_*_exps.E.bias [1, n].  Returns the number of tensors split."""
    split = 0
    for layer in range(int(num_layers)):
        for kind in ("ffn_gate_exps", "ffn_up_exps", "ffn_down_exps"):
            name = f"blk.{layer}.{kind}.bias"
            if name not in float_weights:
                continue
            b = float_weights.pop(name)
            for e in range(b.shape[0]):
                float_weights[f"blk.{layer}.{kind}.{e}.bias"] = np.ascontiguousarray(b[e]).reshape(1, -1)
            split += 1
    return split


def StackExpertWeights(weights):
    """One weight holding the rows of all experts in order ([E * ne1] rows), the operand of
    HipBasicOps.MoEExpertsGptOssForward: a view when the experts are byte-adjacent views of one mapping (a `*_exps.` tensor
    split by GgufFile.expert_weights), else a copy into one aligned buffer (experts fused from two tensors)."""
    if len(weights) == 1:
        return weights[0]
    return QuantizedWeight.ConcatOrCreateCopy(*weights)


def FuseQKVWeights(quant_weights, num_layers):
    """Twin of the models' FuseQKVWeights (Qwen3Model.cs:57-85): attn_q / attn_k / attn_v of equal type and row length
    become blk.L.attn_qkv.weight."""
    fused = 0
    for layer in range(int(num_layers)):
        names = [f"blk.{layer}.attn_{p}.weight" for p in "qkv"]
        ws = [quant_weights.get(n) for n in names]
        if any(w is None for w in ws) or any(w.ggml_type != ws[0].ggml_type or w.ne0 != ws[0].ne0 for w in ws):
            continue
        quant_weights[f"blk.{layer}.attn_qkv.weight"] = QuantizedWeight.ConcatOrCreateCopy(*ws)
        for n, w in zip(names, ws):
            del quant_weights[n]
            w.Dispose()
        fused += 1
    return fused


def _host_view(a, standard):
    if not isinstance(a, np.ndarray) or a.ndim != 2:
        raise ValueError("AddmmQuant requires 2D tensors for result and m1.")
    if a.dtype != np.float32:
        raise ValueError("AddmmQuant requires Float32 tensors for result and m1.")
    s0, s1 = a.strides[0] // 4, a.strides[1] // 4
    if a.strides[0] % 4 or a.strides[1] % 4 or s0 < 0 or s1 < 0 or (standard and s1 != 1):
        raise NotImplementedError("HIP AddmmQuant requires tensors with supported row-contiguous layouts.")
    span = ((a.shape[0] - 1) * s0 + (a.shape[1] - 1) * s1 + 1) * 4
    return N.TensorView2D(a.ctypes.data, a.shape[0], a.shape[1], s0, s1, span)


def _device_view(t):
    import torch
    if not isinstance(t, torch.Tensor) or t.dim() != 2:
        raise ValueError("AddmmQuant requires 2D tensors for result and m1.")
    if t.dtype != torch.float32:
        raise ValueError("AddmmQuant requires Float32 tensors for result and m1.")
    if not t.is_cuda:
        raise ValueError("device AddmmQuant requires tensors in GPU memory.")
    s0, s1 = t.stride()
    if s1 != 1 and t.shape[1] > 1:
        raise NotImplementedError("HIP AddmmQuant requires tensors with supported row-contiguous layouts.")
    span = ((t.shape[0] - 1) * s0 + (t.shape[1] - 1) + 1) * 4
    return N.TensorView2D(t.data_ptr(), t.shape[0], t.shape[1], s0, 1, span)


class HipBasicOps:
    """Static quantized-matmul entry points of the HIP backend."""

    @staticmethod
    def IsAvailable():
        return N.lib().TSHip_IsBackendAvailable(N.BACKEND_HIP) == 1

    @staticmethod
    def GetRowSizeBytes(ggml_type, ne0):
        rb = N.lib().TSHip_RowSize(int(ggml_type), int(ne0))
        if rb <= 0:
            raise NotImplementedError(
                f"GGML tensor type {ggml_type} is not supported, or ne[0]={ne0} is not aligned to the type block size.")
        return int(rb)

    # -- dequantization -------------------------------------------------------------------
    @staticmethod
    def DequantizeToFloat32(ggml_type, src, num_elements):
        """Host bytes -> host fp32 (computed on the GPU).  Codes as GgmlNative.cs:1493-1503."""
        if not isinstance(src, np.ndarray) or src.dtype != np.uint8:
            raise ValueError("Source must be a uint8 array.")
        if num_elements < 0:
            raise ValueError("numElements out of range.")
        dst = np.empty(int(num_elements), dtype=np.float32)
        rc = N.lib().TSHip_DequantizeToF32(int(ggml_type), src.ctypes.data, int(num_elements), dst.ctypes.data)
        if rc == -2:
            raise NotImplementedError(f"HIP backend cannot dequantize GGUF tensor type {ggml_type}.")
        if rc != 0:
            raise RuntimeError(f"Native HIP dequantization failed (code {rc}): {N.get_last_error()}")
        return dst

    @staticmethod
    def DequantizeToFloat32Device(ggml_type, src, num_elements, dst=None):
        import torch
        if dst is None:
            dst = torch.empty(int(num_elements), dtype=torch.float32, device=src.device)
        HipBasicOps.UseCurrentStream()
        rc = N.lib().TSHip_DequantizeToF32Device(int(ggml_type), src.data_ptr(), int(num_elements), dst.data_ptr())
        if rc == -2:
            raise NotImplementedError(f"HIP backend cannot dequantize GGUF tensor type {ggml_type}.")
        if rc != 0:
            raise RuntimeError(f"Native HIP dequantization failed (code {rc}): {N.get_last_error()}")
        return dst

    # -- fused wrappers (GgmlBasicOps.FusedRmsNormMatMulQuant / FusedMatMulQuantAdd / FusedFFNSwiGLUQuant) ------
    @staticmethod
    def _views(out, inp):
        """host (numpy) or device (torch) views of the in/out pair and the export suffix that takes them"""
        if isinstance(out, np.ndarray):
            return _host_view(out, standard=True), _host_view(inp, standard=False), ""
        return _device_view(out), _device_view(inp), "Device"

    @staticmethod
    def _addr(a):
        return a.ctypes.data if isinstance(a, np.ndarray) else a.data_ptr()

    @staticmethod
    def FusedRmsNormMatMulQuant(result, input, norm_weight, eps, weight):
        """result = (RMSNorm(input) * norm_weight) * W^T; all host (numpy) or all device (torch) tensors."""
        rv, iv, sfx = HipBasicOps._views(result, input)
        fn = getattr(N.lib(), "TSHip_FusedRmsNormMatMulQuantF32" + sfx)
        ok = fn(rv, iv, C.c_void_p(HipBasicOps._addr(norm_weight)), int(norm_weight.shape[0]), float(eps),
                C.c_void_p(weight.ptr), weight.ggml_type, weight.ne0, weight.ne1, weight.raw_bytes)
        N.check_result(ok, "fused_rms_norm_matmul_quant")

    @staticmethod
    def FusedMatMulQuantAdd(residual, input, weight):
        """residual += input * W^T, in place."""
        rv, iv, sfx = HipBasicOps._views(residual, input)
        fn = getattr(N.lib(), "TSHip_FusedMatMulQuantAddF32" + sfx)
        ok = fn(rv, iv, C.c_void_p(weight.ptr), weight.ggml_type, weight.ne0, weight.ne1, weight.raw_bytes)
        N.check_result(ok, "fused_matmul_quant_add")

    @staticmethod
    def FusedFFNSwiGLUQuant(residual, input, norm_weight, eps, gate_up, down, half_dim):
        """residual += W_down * (silu(g) * u), [g | u] = W_gate_up * (RMSNorm(input) * norm_weight)."""
        rv, iv, sfx = HipBasicOps._views(residual, input)
        fn = getattr(N.lib(), "TSHip_FusedFFNSwiGLUQuantF32" + sfx)
        ok = fn(rv, iv, C.c_void_p(HipBasicOps._addr(norm_weight)), int(norm_weight.shape[0]), float(eps),
                C.c_void_p(gate_up.ptr), gate_up.ggml_type, gate_up.ne0, gate_up.ne1, gate_up.raw_bytes,
                C.c_void_p(down.ptr), down.ggml_type, down.ne0, down.ne1, down.raw_bytes, int(half_dim))
        N.check_result(ok, "fused_ffn_swiglu_quant")

    @staticmethod
    def _weight_args(w):
        return (C.c_void_p(w.ptr), w.ggml_type, w.ne0, w.ne1, w.raw_bytes)

    @staticmethod
    def FusedOutProjFFN(residual, input, out_proj, ffn_norm_weight, eps, gate_up, down, half_dim):
        """residual += input * W_out^T, then residual += W_down * (silu(g) * u) with [g | u] = W_gate_up * (RMSNorm(residual) *
        ffn_norm_weight) (GgmlBasicOps.cs:449-480).  All host (numpy) or all device (torch) tensors."""
        rv, iv, sfx = HipBasicOps._views(residual, input)
        fn = getattr(N.lib(), "TSHip_FusedOutProjFFNQuantF32" + sfx)
        ok = fn(rv, iv, *HipBasicOps._weight_args(out_proj), C.c_void_p(HipBasicOps._addr(ffn_norm_weight)),
                int(ffn_norm_weight.shape[0]), float(eps), *HipBasicOps._weight_args(gate_up), *HipBasicOps._weight_args(down),
                int(half_dim))
        N.check_result(ok, "fused_outproj_ffn")

    @staticmethod
    def FusedOutProjNormRouter(residual, input, out_proj, norm_weight, eps, normed_output, router, router_output):
        """residual += input * W_out^T; normed_output = RMSNorm(residual) * norm_weight; router_output = normed_output *
        W_router^T (GgmlBasicOps.cs:416-447).  The router weight may be F32 / F16 / BF16 or a block format."""
        rv, iv, sfx = HipBasicOps._views(residual, input)
        view = (lambda a: _host_view(a, standard=True)) if sfx == "" else _device_view
        fn = getattr(N.lib(), "TSHip_FusedOutProjNormRouterQuantF32" + sfx)
        ok = fn(rv, iv, *HipBasicOps._weight_args(out_proj), C.c_void_p(HipBasicOps._addr(norm_weight)),
                int(norm_weight.shape[0]), float(eps), view(normed_output), *HipBasicOps._weight_args(router),
                view(router_output))
        N.check_result(ok, "fused_outproj_norm_router")

    @staticmethod
    def _expert_ptrs(weights):
        return (C.c_void_p * len(weights))(*[w.ptr for w in weights])

    @staticmethod
    def _shape_args(w):
        return (w.ggml_type, w.ne0, w.ne1, w.raw_bytes)

    @staticmethod
    def MoEExpertsForward(result, input, up, down, route_weights):
        """result = sum_e route_weights[e] * W_down[e] * relu(W_up[e] * input)^2 for up to 16 selected experts
        (GgmlBasicOps.cs:586-613; Nemotron).  up / down: lists of QuantizedWeight sharing type and shape."""
        rv, iv, sfx = HipBasicOps._views(result, input)
        n = len(up)
        rw = (C.c_float * n)(*[float(v) for v in route_weights])
        fn = getattr(N.lib(), "TSHip_MoEExpertsForwardF32" + sfx)
        ok = fn(rv, iv, n, HipBasicOps._expert_ptrs(up), HipBasicOps._expert_ptrs(down), *HipBasicOps._shape_args(up[0]),
                *HipBasicOps._shape_args(down[0]), rw)
        N.check_result(ok, "moe_experts_forward")

    @staticmethod
    def MoEExpertsSwiGLUForward(result, input, gate, up, down, route_weights):
        """result = sum_e route_weights[e] * W_down[e] * (silu(W_gate[e] x) * (W_up[e] x)) (GgmlBasicOps.cs:615-645)."""
        rv, iv, sfx = HipBasicOps._views(result, input)
        n = len(up)
        rw = (C.c_float * n)(*[float(v) for v in route_weights])
        fn = getattr(N.lib(), "TSHip_MoEExpertsSwiGLUForwardF32" + sfx)
        ok = fn(rv, iv, n, HipBasicOps._expert_ptrs(gate), HipBasicOps._expert_ptrs(up), HipBasicOps._expert_ptrs(down),
                *HipBasicOps._shape_args(gate[0]), *HipBasicOps._shape_args(up[0]), *HipBasicOps._shape_args(down[0]), rw)
        N.check_result(ok, "moe_experts_swiglu_forward")

    @staticmethod
    def MoEExpertsSwiGLUResidual(residual, input, gate, up, down, route_weights, shared=None, shared_scalar=1.0):
        """residual += sum_e route_weights[e] * expert_e(input) [+ shared_scalar * shared_expert(input)]
        (GgmlBasicOps.cs:647-700); shared = (gate, up, down) QuantizedWeights or None; up to 32 routed experts."""
        rv, iv, sfx = HipBasicOps._views(residual, input)
        n = len(up)
        rw = (C.c_float * n)(*[float(v) for v in route_weights])
        if shared is None:
            sh = (0, None, None, None, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0)
        else:
            sh = (1, C.c_void_p(shared[0].ptr), C.c_void_p(shared[1].ptr), C.c_void_p(shared[2].ptr),
                  *HipBasicOps._shape_args(shared[0]), *HipBasicOps._shape_args(shared[1]), *HipBasicOps._shape_args(shared[2]))
        fn = getattr(N.lib(), "TSHip_MoEExpertsSwiGLUResidualF32" + sfx)
        ok = fn(rv, iv, n, HipBasicOps._expert_ptrs(gate), HipBasicOps._expert_ptrs(up), HipBasicOps._expert_ptrs(down),
                *HipBasicOps._shape_args(gate[0]), *HipBasicOps._shape_args(up[0]), *HipBasicOps._shape_args(down[0]), rw,
                *sh, float(shared_scalar))
        N.check_result(ok, "moe_experts_swiglu_residual")

    @staticmethod
    def _view3(a):
        """3-D fp32 view of a numpy array or a torch CUDA tensor (strides in elements)"""
        host = isinstance(a, np.ndarray)
        if (a.ndim if host else a.dim()) != 3 or str(a.dtype).split(".")[-1] != "float32":
            raise ValueError("MulMatId requires 3D Float32 tensors.")
        st = [v // 4 for v in a.strides] if host else list(a.stride())
        span = (sum((d - 1) * s for d, s in zip(a.shape, st)) + 1) * 4
        return N.TensorView3D(HipBasicOps._addr(a), a.shape[0], a.shape[1], a.shape[2], st[0], st[1], st[2], span)

    @staticmethod
    def MulMatId(result, expert_weights, input, ids):
        """result[t, s, :] = expert_weights[ids[t, s]] @ input[t, s % slots] with F32 experts [E, rows, K]
        (GgmlNative.MulMatId, GgmlNative.cs:1076-1079).  All host (numpy; ids int32 or float32) or all device (torch; ids
        int32) tensors."""
        host = isinstance(result, np.ndarray)
        rows, cols = int(ids.shape[0]), int(ids.shape[1])
        if host:
            idc = np.ascontiguousarray(ids)
            if idc.dtype not in (np.int32, np.float32):
                raise ValueError("MulMatId ids must be Int32 or Float32.")
            desc = N.ContiguousTensor(idc.ctypes.data, int(idc.size), 3 if idc.dtype == np.int32 else 0)
            ok = N.lib().TSHip_MulMatIdF32(HipBasicOps._view3(result), HipBasicOps._view3(expert_weights),
                                           HipBasicOps._view3(input), desc, rows, cols)
        else:
            HipBasicOps.UseCurrentStream()
            ok = N.lib().TSHip_MulMatIdF32Device(HipBasicOps._view3(result), HipBasicOps._view3(expert_weights),
                                                 HipBasicOps._view3(input), C.c_void_p(ids.contiguous().data_ptr()), rows, cols)
        N.check_result(ok, "mulmatid")

    @staticmethod
    def AddId(result, src, bias, ids):
        """result[t, s, :] = src[t, s, :] + bias[ids[t, s], :] (GgmlBasicOps.AddID, GgmlBasicOps.cs:1092-1108; the bias of
        a MulMatId).  All host (numpy; ids int32 or float32) or all device (torch; ids int32) tensors; result may be src."""
        host = isinstance(result, np.ndarray)
        if (ids.ndim if host else ids.dim()) != 2 or (bias.ndim if host else bias.dim()) != 2:
            raise NotImplementedError("addid expects 2D bias and id tensors.")
        rows, cols = int(ids.shape[0]), int(ids.shape[1])
        if host:
            idc = np.ascontiguousarray(ids)
            if idc.dtype not in (np.int32, np.float32):
                raise ValueError("AddId ids must be Int32 or Float32.")
            desc = N.ContiguousTensor(idc.ctypes.data, int(idc.size), 3 if idc.dtype == np.int32 else 0)
            ok = N.lib().TSHip_AddIdF32(HipBasicOps._view3(result), HipBasicOps._view3(src), _host_view(bias, standard=True), desc, rows, cols)
        else:
            HipBasicOps.UseCurrentStream()
            ok = N.lib().TSHip_AddIdF32Device(HipBasicOps._view3(result), HipBasicOps._view3(src), _device_view(bias),
                                              C.c_void_p(ids.contiguous().data_ptr()), rows, cols)
        N.check_result(ok, "addid")

    # -- embedding gather ------------------------------------------------------------------
    @staticmethod
    def GetRowsQuant(result, weight_data, ggml_type, ne0, ne1, raw_bytes, indices):
        """result[i] = dequantized row indices[i] (GgmlBasicOps.cs:565-579). Host tensors; weight_data: address."""
        if not isinstance(result, np.ndarray) or result.ndim != 2 or result.dtype != np.float32:
            raise ValueError("GetRowsQuant requires a 2D Float32 result tensor.")
        idx = np.asarray(indices)
        if idx.dtype != np.int32 or not idx.flags["C_CONTIGUOUS"]:
            raise NotImplementedError("HIP GetRowsQuant requires a standard-layout result and contiguous Int32 indices.")
        rv = _host_view(result, standard=True)
        desc = N.ContiguousTensor(idx.ctypes.data, int(idx.size), 3)
        ok = N.lib().TSHip_GetRowsQuantF32(rv, C.c_void_p(weight_data), int(ggml_type), int(ne0), int(ne1),
                                           int(raw_bytes), desc)
        N.check_result(ok, "get_rows_quant")

    @staticmethod
    def GetRowsQuantDevice(result, weight, indices):
        """Device form: result [n x K] fp32 CUDA tensor, weight a device QuantizedWeight, indices int32 CUDA tensor."""
        rv = _device_view(result)
        ok = N.lib().TSHip_GetRowsQuantF32Device(rv, C.c_void_p(weight.ptr), weight.ggml_type, weight.ne0, weight.ne1,
                                                 weight.raw_bytes, C.c_void_p(indices.data_ptr()), int(indices.numel()))
        N.check_result(ok, "get_rows_quant")

    # -- matmul ---------------------------------------------------------------------------
    @staticmethod
    def AddmmQuant(result, m1, weight_data, ggml_type, ne0, ne1, raw_bytes):
        """result = m1 * W^T with host tensors (GgmlBasicOps.cs:313-329). weight_data: address (int)."""
        rv = _host_view(result, standard=True)
        mv = _host_view(m1, standard=False)
        ok = N.lib().TSHip_AddmmQuantF32(rv, mv, C.c_void_p(weight_data), int(ggml_type), int(ne0), int(ne1),
                                         int(raw_bytes))
        N.check_result(ok, "addmm_quant")

    @staticmethod
    def AddmmQuantDevice(result, m1, weight_data, ggml_type, ne0, ne1, raw_bytes):
        """Same contract with every pointer in device memory; asynchronous on the current stream."""
        rv = _device_view(result)
        mv = _device_view(m1)
        ok = N.lib().TSHip_AddmmQuantF32Device(rv, mv, C.c_void_p(weight_data), int(ggml_type), int(ne0), int(ne1),
                                               int(raw_bytes))
        N.check_result(ok, "addmm_quant")

    @staticmethod
    def AddmmQuantDeviceNoAlloc(result, m1, weight_data, ggml_type, ne0, ne1, raw_bytes):
        """AddmmQuantDevice for callers that cannot allocate device memory: scratch lives in a static device array."""
        rv = _device_view(result)
        mv = _device_view(m1)
        ok = N.lib().TSHip_AddmmQuantF32DeviceNoAlloc(rv, mv, C.c_void_p(weight_data), int(ggml_type), int(ne0), int(ne1),
                                                      int(raw_bytes))
        N.check_result(ok, "addmm_quant")

    @staticmethod
    def PrepareGroup(results, m1s, weights):
        """Marshal a list of (result, m1, QuantizedWeight) problems once; returns the argument pack
        that AddmmQuantGroupDevice launches (decode loops reuse the pack every token)."""
        n = len(weights)
        if not (n == len(results) == len(m1s)) or n == 0:
            raise ValueError("results, m1s and weights must be equally long and non-empty.")
        t = weights[0].ggml_type
        if any(w.ggml_type != t for w in weights):
            raise ValueError("all weights of a group must share one block type.")
        rv = (N.TensorView2D * n)(*[_device_view(r) for r in results])
        mv = (N.TensorView2D * n)(*[_device_view(m) for m in m1s])
        wp = (C.c_void_p * n)(*[w.ptr for w in weights])
        ne0 = (C.c_int64 * n)(*[w.ne0 for w in weights])
        ne1 = (C.c_int64 * n)(*[w.ne1 for w in weights])
        rb = (C.c_int64 * n)(*[w.raw_bytes for w in weights])
        return (n, rv, mv, wp, t, ne0, ne1, rb)

    @staticmethod
    def AddmmQuantGroupDevice(pack):
        """count independent AddmmQuantDevice problems; one launch when all are decode GEMVs."""
        ok = N.lib().TSHip_AddmmQuantGroupF32Device(*pack)
        N.check_result(ok, "addmm_quant_group")

    @staticmethod
    def AddmmQuantBatch(result, m1, weight_data, ggml_type, ne0, raw_bytes, weight_offsets, weight_ne1):
        """Row b of m1 times the sub-weight at weight_offsets[b] (GgmlBasicOps.cs:689-704)."""
        rv = _host_view(result, standard=True)
        mv = _host_view(m1, standard=False)
        n = len(weight_offsets)
        if n != len(weight_ne1):
            raise ValueError("weight_offsets and weight_ne1 must have the same length.")
        offs = (C.c_int64 * n)(*[int(v) for v in weight_offsets])
        ne1s = (C.c_int64 * n)(*[int(v) for v in weight_ne1])
        ok = N.lib().TSHip_AddmmQuantBatchF32(rv, mv, C.c_void_p(weight_data), int(ggml_type), int(ne0),
                                              int(raw_bytes), n, offs, ne1s)
        N.check_result(ok, "addmm_quant_batch")

    @staticmethod
    def PreloadQuantizedWeight(cache_key, host_data, ggml_type, ne0, ne1, raw_bytes):
        ok = N.lib().TSHip_PreloadQuantizedWeight(C.c_void_p(cache_key), C.c_void_p(host_data), int(ggml_type),
                                                  int(ne0), int(ne1), int(raw_bytes))
        N.check_result(ok, "preload_quantized_weight")

    @staticmethod
    def InvalidateHostBuffer(ptr):
        N.lib().TSHip_InvalidateHostBuffer(C.c_void_p(ptr))

    @staticmethod
    def ClearHostBufferCache():
        N.lib().TSHip_ClearHostBufferCache()

    @staticmethod
    def SyncHostBuffer(array):
        """Copy the device copy kept for this host array (a KV cache the layer decode updates) back into it."""
        ok = N.lib().TSHip_SyncHostBuffer(C.c_void_p(array.ctypes.data), int(array.nbytes))
        N.check_result(ok, "sync_host_buffer")

    # -- MoE (GptOssModel.MoERoute / MoEForward twins, device tensors) --------------------------
    @staticmethod
    def MoERoute(logits, k):
        """logits [T x E] (CUDA fp32) -> (weights [T x k] fp32, ids [T x k] int32)."""
        import torch
        T = logits.shape[0]
        ids = torch.empty((T, k), dtype=torch.int32, device=logits.device)
        wts = torch.empty((T, k), dtype=torch.float32, device=logits.device)
        HipBasicOps.UseCurrentStream()
        ok = N.lib().TSHip_MoERouteF32Device(_device_view(logits), int(k), ids.data_ptr(), wts.data_ptr())
        N.check_result(ok, "moe_route")
        return wts, ids

    @staticmethod
    def MoEExpertsGptOssForward(hidden, ids, weights, gate_up_w, gate_up_b, down_w, down_b, ggml_type, n_experts, H, F,
                          alpha=1.702, limit=7.0):
        """Expert stage of GptOssModel.MoEForward for routed tokens; all tensors on the device."""
        import torch
        out = torch.empty((hidden.shape[0], H), dtype=torch.float32, device=hidden.device)
        HipBasicOps.UseCurrentStream()
        ok = N.lib().TSHip_MoEExpertsGptOssForwardF32Device(
            _device_view(out), _device_view(hidden), ids.data_ptr(), weights.data_ptr(), int(ids.shape[1]),
            gate_up_w.data_ptr(), None if gate_up_b is None else gate_up_b.data_ptr(), down_w.data_ptr(),
            None if down_b is None else down_b.data_ptr(), int(ggml_type), int(n_experts), int(H), int(F), float(alpha),
            float(limit))
        N.check_result(ok, "moe_experts_forward")
        return out

    # -- whole-layer decode (GgmlBasicOps.TransformerLayerDecode / TransformerModelDecode twins) ----
    @staticmethod
    def TransformerLayerDecode(hidden, attn_norm, qkv, q_norm, k_norm, o, ffn_norm, gate_up, down, k_cache, v_cache,
                               num_heads, num_kv_heads, head_dim, position, eps, rope_base, rope_freq_scale=1.0, rope_mode=2):
        """One token through one layer, in place on `hidden` [hidden_size] fp32.  Either everything is on the device (torch
        CUDA tensors, device QuantizedWeights; asynchronous on the current stream) or everything is in host memory (numpy
        arrays, host QuantizedWeights; weights, norms and KV caches are kept on the device under their host address, and
        SyncHostBuffer(k_cache) brings a cache back).  k_cache / v_cache fp32 [num_kv_heads, max_seq_len, head_dim];
        q_norm / k_norm may be None."""
        host = isinstance(hidden, np.ndarray)
        if host:
            fn = N.lib().TSHip_TransformerLayerDecode
        else:
            HipBasicOps.UseCurrentStream()
            fn = N.lib().TSHip_TransformerLayerDecodeDevice
        p = lambda t: None if t is None else HipBasicOps._addr(t)
        ok = fn(
            p(hidden), int(hidden.size if host else hidden.numel()), p(attn_norm),
            qkv.ptr, qkv.ggml_type, qkv.ne0, qkv.ne1, qkv.raw_bytes, p(q_norm), p(k_norm), int(head_dim),
            o.ptr, o.ggml_type, o.ne0, o.ne1, o.raw_bytes, p(ffn_norm),
            gate_up.ptr, gate_up.ggml_type, gate_up.ne0, gate_up.ne1, gate_up.raw_bytes,
            down.ptr, down.ggml_type, down.ne0, down.ne1, down.raw_bytes,
            p(k_cache), p(v_cache), int(num_heads), int(num_kv_heads), int(k_cache.shape[1]), int(position),
            float(eps), float(rope_base), float(rope_freq_scale), int(gate_up.ne1 // 2), int(rope_mode))
        N.check_result(ok, "transformer_layer_decode")

    @staticmethod
    def TransformerModelDecode(hidden, layers, num_heads, num_kv_heads, head_dim, position, eps, rope_base, rope_freq_scale=1.0,
                               rope_mode=2):
        """The same for a list of layers; each layer is a dict with the argument names of TransformerLayerDecode
        (attn_norm, qkv, q_norm, k_norm, o, ffn_norm, gate_up, down, k_cache, v_cache); shapes and types are shared.
        Host arrays or device tensors throughout, as for TransformerLayerDecode."""
        import ctypes as C
        host = isinstance(hidden, np.ndarray)
        if host:
            fn = N.lib().TSHip_TransformerModelDecode
        else:
            HipBasicOps.UseCurrentStream()
            fn = N.lib().TSHip_TransformerModelDecodeDevice
        n = len(layers)

        def arr(key, weight=False):
            vals = []
            for L in layers:
                t = L.get(key)
                vals.append(None if t is None else (t.ptr if weight else HipBasicOps._addr(t)))
            if all(v is None for v in vals):
                return None
            return (C.c_void_p * n)(*vals)
        l0 = layers[0]
        qkv, o, gu, dn = l0["qkv"], l0["o"], l0["gate_up"], l0["down"]
        ok = fn(
            HipBasicOps._addr(hidden), int(hidden.size if host else hidden.numel()), n, arr("attn_norm"), arr("qkv", True), arr("q_norm"), arr("k_norm"), arr("o", True),
            arr("ffn_norm"), arr("gate_up", True), arr("down", True), arr("k_cache"), arr("v_cache"),
            qkv.ggml_type, qkv.ne0, qkv.ne1, qkv.raw_bytes, o.ggml_type, o.ne0, o.ne1, o.raw_bytes,
            gu.ggml_type, gu.ne0, gu.ne1, gu.raw_bytes, dn.ggml_type, dn.ne0, dn.ne1, dn.raw_bytes,
            int(head_dim), int(num_heads), int(num_kv_heads), int(l0["k_cache"].shape[1]), int(position), float(eps),
            float(rope_base), float(rope_freq_scale), int(gu.ne1 // 2), int(rope_mode))
        N.check_result(ok, "transformer_model_decode")

    # -- LinearForward twin (ModelBase.cs:875-905): allocate result, route by residency -----
    @staticmethod
    def LinearForward(m1, qw: QuantizedWeight):
        if qw.is_device:
            import torch
            result = torch.empty((m1.shape[0], qw.ne1), dtype=torch.float32, device=m1.device)
            HipBasicOps.UseCurrentStream()
            HipBasicOps.AddmmQuantDevice(result, m1, qw.ptr, qw.ggml_type, qw.ne0, qw.ne1, qw.raw_bytes)
            return result
        result = np.empty((m1.shape[0], qw.ne1), dtype=np.float32)
        HipBasicOps.AddmmQuant(result, m1, qw.ptr, qw.ggml_type, qw.ne0, qw.ne1, qw.raw_bytes)
        return result

    @staticmethod
    def UseCurrentStream():
        """Launch the *Device entry points on torch's current stream."""
        import torch
        N.lib().TSHip_SetStream(C.c_void_p(torch.cuda.current_stream().cuda_stream))
