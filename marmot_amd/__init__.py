"""marmot_amd — MI355X (gfx950) implementation of marmot's block-quantized GGUF matmul path.

The product is the C-ABI shared library ``marmot_amd/lib/libmarmot_hip.so`` (declared in
``include/marmot_hip.h``). This package is the thin host-side mirror used by tests and the
benchmark: it loads the library with ctypes and exposes the reference's operator names
(``linear``, ``dequantize``, ``quantize_activations``, ``topk``, ``moe_experts``) over numpy
arrays and device buffers. There is no CPU fallback: if the library is missing, loading raises.
"""
from .capi import (DT_F16, DT_F32, KIND_Q2_K, KIND_Q3_K, KIND_Q4_0, KIND_Q4_1, KIND_Q4_K, KIND_Q5_0, KIND_Q5_1, KIND_Q5_K, KIND_Q6_K, KIND_Q8_0,
                   KIND_Q8_1, KIND_Q8_K, MarmotHipError, lib_path, load_library)
from .backend import DeviceBuffer, HipBackend, block_bytes, block_values, row_bytes

__all__ = [
    "DT_F16", "DT_F32", "KIND_Q2_K", "KIND_Q3_K", "KIND_Q4_0", "KIND_Q4_1", "KIND_Q5_0", "KIND_Q5_1", "KIND_Q4_K", "KIND_Q5_K", "KIND_Q6_K", "KIND_Q8_0", "KIND_Q8_1", "KIND_Q8_K", "MarmotHipError",
    "lib_path", "load_library", "DeviceBuffer", "HipBackend", "block_bytes", "block_values", "row_bytes",
]
