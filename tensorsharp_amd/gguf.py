"""GGUF file reader and weight upload: the host-side twin of TensorSharp.Runtime/GgufReader.cs.

The file is memory-mapped read-only; tensor bytes are handed to the HIP library straight from the mapping (no
intermediate copy on the host), either through the bridge's preload export keyed by the mapped address
(TSGgml_PreloadQuantizedWeight semantics, ModelBase.cs:660-706) or into a device tensor owned by the caller.

Layout restated from GgufReader.cs:78-118 (header, metadata, tensor infos, aligned data section), :371-480 (strings,
values, arrays), :288-369 (row bytes, block sizes, type sizes).
"""
import mmap
import struct

import numpy as np

GGUF_MAGIC = 0x46554747          # "GGUF" little-endian (GgufReader.cs:82-84)

# GgufValueType (GgufReader.cs:19-24)
(VT_UINT8, VT_INT8, VT_UINT16, VT_INT16, VT_UINT32, VT_INT32, VT_FLOAT32, VT_BOOL, VT_STRING, VT_ARRAY, VT_UINT64, VT_INT64,
 VT_FLOAT64) = range(13)
_SCALAR = {VT_UINT8: "<B", VT_INT8: "<b", VT_UINT16: "<H", VT_INT16: "<h", VT_UINT32: "<I", VT_INT32: "<i", VT_FLOAT32: "<f",
           VT_UINT64: "<Q", VT_INT64: "<q", VT_FLOAT64: "<d"}
_ARRAY_DTYPE = {VT_UINT8: np.uint8, VT_INT8: np.int8, VT_UINT16: np.uint16, VT_INT16: np.int16, VT_UINT32: np.uint32,
                VT_INT32: np.int32, VT_FLOAT32: np.float32, VT_UINT64: np.uint64, VT_INT64: np.int64, VT_FLOAT64: np.float64,
                VT_BOOL: np.bool_}

# GgmlTensorType -> (block size, type size) (GgufReader.cs:303-369)
TYPE_TABLE = {
    0: (1, 4), 1: (1, 2), 30: (1, 2), 2: (32, 18), 3: (32, 20), 6: (32, 22), 7: (32, 24), 8: (32, 34), 9: (32, 36),
    10: (256, 84), 11: (256, 110), 12: (256, 144), 13: (256, 176), 14: (256, 210), 15: (256, 292),
    16: (256, 66), 17: (256, 74), 18: (256, 98), 19: (256, 50), 20: (32, 18), 21: (256, 110), 22: (256, 82), 23: (256, 136),
    29: (256, 56), 34: (256, 54), 35: (256, 66), 39: (32, 17), 24: (1, 1), 25: (1, 2), 26: (1, 4), 27: (1, 8), 28: (1, 8),
}
# block formats the matmul kernels read (tship_internal.h is_quant_type): Q4_0, Q4_1, Q5_0, Q5_1, Q8_0, Q4_K, Q5_K, Q6_K,
# IQ4_NL, MXFP4
MATMUL_TYPES = (2, 3, 6, 7, 8, 12, 13, 14, 20, 39)
TYPE_NAMES = {0: "F32", 1: "F16", 2: "Q4_0", 3: "Q4_1", 6: "Q5_0", 7: "Q5_1", 8: "Q8_0", 9: "Q8_1", 10: "Q2_K", 11: "Q3_K",
              12: "Q4_K", 13: "Q5_K", 14: "Q6_K", 15: "Q8_K", 20: "IQ4_NL", 30: "BF16", 39: "MXFP4"}


class GgufTensorInfo:
    """GgufTensorInfo (GgufReader.cs:39-55): name, shape (ne0 first), type id, offset inside the data section."""

    def __init__(self, name, shape, ggml_type, offset):
        self.Name = name
        self.Shape = tuple(int(d) for d in shape)
        self.Type = int(ggml_type)
        self.Offset = int(offset)

    @property
    def NumElements(self):
        n = 1
        for d in self.Shape:
            n *= d
        return n

    def __repr__(self):
        return f"GgufTensorInfo({self.Name!r}, {self.Shape}, {TYPE_NAMES.get(self.Type, self.Type)}, +{self.Offset})"


class _Cursor:
    def __init__(self, buf):
        self.buf = buf
        self.pos = 0

    def take(self, fmt):
        size = struct.calcsize(fmt)
        if self.pos + size > len(self.buf):
            raise ValueError("GGUF file is truncated.")
        v = struct.unpack_from(fmt, self.buf, self.pos)[0]
        self.pos += size
        return v

    def string(self):
        n = self.take("<Q")
        if self.pos + n > len(self.buf):
            raise ValueError("GGUF file is truncated.")
        s = bytes(self.buf[self.pos:self.pos + n]).decode("utf-8", errors="replace")
        self.pos += n
        return s


class GgufFile:
    """Parsed GGUF file over a read-only memory map.  Metadata: key -> python value (arrays of numbers as numpy arrays,
    arrays of strings as lists); Tensors: name -> GgufTensorInfo; DataOffset: start of the aligned data section."""

    def __init__(self, path):
        self.path = path
        self._file = open(path, "rb")
        try:
            self._map = mmap.mmap(self._file.fileno(), 0, access=mmap.ACCESS_READ)
        except ValueError:
            self._file.close()
            raise ValueError("Not a GGUF file (empty).")
        self._bytes = np.frombuffer(self._map, dtype=np.uint8)
        self.Metadata = {}
        self.Tensors = {}
        self._preloaded = []          # cache keys (mapped addresses) handed to PreloadQuantizedWeight
        try:
            self._parse()
        except Exception:
            self.close()
            raise

    # -- parsing (GgufReader.cs:78-118) ----------------------------------------------------------
    def _parse(self):
        c = _Cursor(self._map)
        magic = c.take("<I")
        if magic != GGUF_MAGIC:
            raise ValueError(f"Not a GGUF file (magic: 0x{magic:08X})")
        self.Version = c.take("<I")
        if self.Version < 2:
            raise NotImplementedError(f"GGUF version {self.Version} not supported")
        tensor_count = c.take("<Q")
        kv_count = c.take("<Q")
        for _ in range(kv_count):
            key = c.string()
            self.Metadata[key] = self._value(c, c.take("<I"))
        for _ in range(tensor_count):
            name = c.string()
            dims = c.take("<I")
            shape = [c.take("<Q") for _ in range(dims)]
            ggml_type = c.take("<I")
            offset = c.take("<Q")
            self.Tensors[name] = GgufTensorInfo(name, shape, ggml_type, offset)
        alignment = int(self.Metadata.get("general.alignment", 32))
        if alignment <= 0 or alignment & (alignment - 1):
            # the reference divides by it (GgufReader.cs:115-118); the GGUF format requires a power of two
            raise ValueError(f"GGUF general.alignment must be a positive power of two, not {alignment}.")
        self.DataOffset = c.pos + (alignment - c.pos % alignment) % alignment

    def _value(self, c, vt):
        if vt in _SCALAR:
            return c.take(_SCALAR[vt])
        if vt == VT_BOOL:
            return c.take("<B") != 0
        if vt == VT_STRING:
            return c.string()
        if vt == VT_ARRAY:
            et = c.take("<I")
            n = c.take("<Q")
            if et == VT_STRING:
                return [c.string() for _ in range(n)]
            if et in _ARRAY_DTYPE:
                dt = np.dtype(_ARRAY_DTYPE[et])
                size = dt.itemsize * n
                if c.pos + size > len(c.buf):
                    raise ValueError("GGUF file is truncated.")
                a = np.frombuffer(c.buf, dtype=dt, count=n, offset=c.pos).copy()
                c.pos += size
                return a
            raise NotImplementedError(f"Unknown GGUF array element type: {et}")
        raise NotImplementedError(f"Unknown GGUF value type: {vt}")

    # -- typed metadata getters (GgufReader.cs:120-203) -----------------------------------------
    def GetString(self, key, default=None):
        v = self.Metadata.get(key)
        return v if isinstance(v, str) else default

    def GetUint32(self, key, default=0):
        v = self.Metadata.get(key)
        if v is None:
            return default
        if isinstance(v, np.ndarray):
            return int(v[0]) & 0xFFFFFFFF if v.size else default
        return int(v)

    def GetFloat32(self, key, default=0.0):
        v = self.Metadata.get(key)
        if v is None:
            return default
        if isinstance(v, np.ndarray):
            return float(v[0]) if v.size else default
        return float(v)

    def GetBool(self, key, default=False):
        v = self.Metadata.get(key)
        return default if v is None else bool(v)

    def GetStringArray(self, key):
        v = self.Metadata.get(key)
        return v if isinstance(v, list) else None

    def GetFloatArray(self, key):
        v = self.Metadata.get(key)
        return v if isinstance(v, np.ndarray) and v.dtype == np.float32 else None

    def GetInt32Array(self, key):
        v = self.Metadata.get(key)
        if isinstance(v, np.ndarray) and v.dtype in (np.int32, np.uint32):
            return v.astype(np.int32)
        return None

    # -- sizes (GgufReader.cs:288-369) ------------------------------------------------------------
    @staticmethod
    def GetBlockSize(ggml_type):
        return TYPE_TABLE[int(ggml_type)][0] if int(ggml_type) in TYPE_TABLE else 256

    @staticmethod
    def GetTypeSize(ggml_type):
        if int(ggml_type) not in TYPE_TABLE:
            raise NotImplementedError(f"Unknown GGML tensor type: {ggml_type}")
        return TYPE_TABLE[int(ggml_type)][1]

    @classmethod
    def GetRowBytes(cls, ggml_type, ne0):
        return (int(ne0) // cls.GetBlockSize(ggml_type)) * cls.GetTypeSize(ggml_type)

    def GetTensorByteCount(self, info):
        rows = 1
        for d in info.Shape[1:]:
            rows *= d
        return self.GetRowBytes(info.Type, info.Shape[0]) * rows

    # -- data --------------------------------------------------------------------------------------
    def tensor_data(self, name):
        """The tensor's bytes as a read-only uint8 view of the mapping (TryGetTensorDataPointer, GgufReader.cs:267-279)."""
        info = self.Tensors[name]
        begin = self.DataOffset + info.Offset
        end = begin + self.GetTensorByteCount(info)
        if end > self._bytes.size:
            raise ValueError(f"tensor {name!r} extends past the end of the file.")
        return self._bytes[begin:end]

    def _device_bytes(self, offset, count, device):
        """`count` bytes of the mapping from `offset` as a new torch uint8 tensor on `device`: one host-to-device copy
        straight from the page cache"""
        import torch
        import warnings
        t = torch.empty(count, dtype=torch.uint8, device=device)
        with warnings.catch_warnings():
            warnings.simplefilter("ignore", UserWarning)      # read-only mapping: it is only ever read
            src = torch.frombuffer(self._map, dtype=torch.uint8, count=count, offset=offset)
        t.copy_(src)
        return t

    @staticmethod
    def is_expert_stack(info):
        """A 3-D tensor holding the experts of one projection, [ne0, ne1, experts] (ModelBase.cs:507-510, :554)."""
        return len(info.Shape) == 3 and "_exps." in info.Name

    @classmethod
    def should_store_quantized(cls, info):
        """BackendExecutionPlan.ShouldStoreWeightQuantized (ModelBase.cs:499-511) for a backend that reads raw blocks:
        everything but F32 that is a matrix or a stack of expert matrices."""
        return info.Type != 0 and (len(info.Shape) == 2 or cls.is_expert_stack(info))

    def quantized_weight(self, name, device=None):
        """A 2-D tensor as a QuantizedWeight: over the mapping (host form), or copied to `device` (torch device)."""
        from .hip_basic_ops import QuantizedWeight
        info = self.Tensors[name]
        if len(info.Shape) != 2:
            raise ValueError(f"tensor {name!r} is not a matrix: shape {info.Shape}" +
                             (" (a stack of experts: use expert_weights)" if self.is_expert_stack(info) else ""))
        data = self.tensor_data(name)
        if device is not None:
            t = self._device_bytes(self.DataOffset + info.Offset, data.size, device)
            return QuantizedWeight(t, info.Type, info.Shape[0], info.Shape[1])
        # a view of the mapping, kept alive by this file object: adjacent tensors concatenate without a copy
        return QuantizedWeight.CreateExternalView(data, info.Type, info.Shape[0], info.Shape[1], self)

    @staticmethod
    def expert_weight_names(name, num_experts):
        """Names of the per-expert weights a stack is split into: `blk.L.ffn_up_exps.weight` -> `blk.L.ffn_up_exps.<e>.weight`
        (ModelBase.cs:559-569)."""
        base = name[:-len(".weight")] if name.endswith(".weight") else name
        return [f"{base}.{e}.weight" for e in range(int(num_experts))]

    def expert_weights(self, name, device=None):
        """The experts of a 3-D `*_exps.` tensor [ne0, ne1, E] as E QuantizedWeights of ne1 rows: expert e is the bytes at
        e * (bytes / E) of the tensor (ModelBase.cs:554-595).  Host form: external views of the mapping, adjacent to
        each other, so the whole stack concatenates back into one view without a copy; device form: one upload of
        the whole tensor, the experts are slices of it."""
        from .hip_basic_ops import QuantizedWeight
        info = self.Tensors[name]
        if not self.is_expert_stack(info):
            raise ValueError(f"tensor {name!r} is not a stack of expert matrices: shape {info.Shape}")
        ne0, ne1, count = info.Shape
        data = self.tensor_data(name)
        per_expert = data.size // count
        if device is not None:
            whole = self._device_bytes(self.DataOffset + info.Offset, data.size, device)
            return [QuantizedWeight(whole[e * per_expert:(e + 1) * per_expert], info.Type, ne0, ne1) for e in range(count)]
        return [QuantizedWeight.CreateExternalView(data[e * per_expert:(e + 1) * per_expert], info.Type, ne0, ne1, self)
                for e in range(count)]

    def float_tensor(self, name):
        """An F32 / F16 / BF16 tensor as a float32 numpy array shaped [.., ne1, ne0] (the managed side's `_weights`)."""
        info = self.Tensors[name]
        raw = self.tensor_data(name)
        shape = tuple(reversed(info.Shape))
        if info.Type == 0:
            return np.array(raw.view(np.float32)).reshape(shape)
        if info.Type == 1:
            return raw.view(np.float16).astype(np.float32).reshape(shape)
        if info.Type == 30:
            return (raw.view(np.uint16).astype(np.uint32) << 16).view(np.float32).reshape(shape)
        raise ValueError(f"tensor {name!r} has a block format; use quantized_weight / expert_weights")

    def load_quantized_weights(self, device=None):
        """name -> QuantizedWeight for every tensor the reference keeps as raw blocks: matrices under their own name,
        expert stacks split into `<base>.<e>.weight` (the `_quantWeights` dictionary of ModelBase.LoadWeights,
        ModelBase.cs:540-625)."""
        out = {}
        for name, info in self.Tensors.items():
            if not self.should_store_quantized(info):
                continue
            if self.is_expert_stack(info):
                out.update(zip(self.expert_weight_names(name, info.Shape[2]), self.expert_weights(name, device)))
            else:
                out[name] = self.quantized_weight(name, device)
        return out

    def preload(self, names=None):
        """Upload weights once through the bridge's preload export, keyed by their mapped address: later host-pointer
        calls with the same weight pointer run from the device copy (ModelBase.cs:660-706).  Expert stacks go up expert
        by expert under `<base>.<e>.weight`, which is what the per-expert calls pass.  Returns the weights."""
        from .hip_basic_ops import HipBasicOps
        out = {}
        for name in (names if names is not None else list(self.Tensors)):
            info = self.Tensors[name]
            # every block format the matmul kernels read (F32 / F16 / BF16 tensors stay with the host path)
            if info.Type not in MATMUL_TYPES or not self.should_store_quantized(info):
                continue
            if self.is_expert_stack(info):
                ws = dict(zip(self.expert_weight_names(name, info.Shape[2]), self.expert_weights(name)))
            else:
                ws = {name: self.quantized_weight(name)}
            for n, w in ws.items():
                HipBasicOps.PreloadQuantizedWeight(w.ptr, w.ptr, w.ggml_type, w.ne0, w.ne1, w.raw_bytes)
                self._preloaded.append(w.ptr)
                out[n] = w
        return out

    def close(self):
        # the device copies are keyed by addresses inside the mapping: once it is gone another file may be mapped at
        # the same address, and a preload of equal size under the same key would be taken for a repeat
        if self._preloaded:
            from .hip_basic_ops import HipBasicOps
            for key in self._preloaded:
                HipBasicOps.InvalidateHostBuffer(key)
            self._preloaded = []
        self._bytes = None
        try:
            self._map.close()
        except (BufferError, ValueError, AttributeError):
            pass          # numpy views of the mapping are still alive: the map goes with the last of them
        self._file.close()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()
