"""tensorsharp_amd — MI355X (gfx950) backend for TensorSharp's GGUF quantized matmul.

hip_native      ctypes bindings of libTsHipOps' C ABI (the P/Invoke layer's twin)
hip_basic_ops   host-side operator facade with the reference's names and error behaviour
synth           synthetic GGUF block generators for benchmarks
gguf            GGUF file reader (memory-mapped) and weight upload from the mapping
build           hipcc build of the shared library
"""
from . import hip_native  # noqa: F401
from .hip_basic_ops import HipBasicOps, QuantizedWeight, FuseGateUpWeights, FuseQKVWeights  # noqa: F401
from .gguf import GgufFile  # noqa: F401
