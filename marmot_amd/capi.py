"""ctypes declarations of include/marmot_hip.h (one entry per exported symbol)."""
from __future__ import annotations

import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))

KIND_Q4_0, KIND_Q8_0, KIND_Q4_K, KIND_Q5_K, KIND_Q6_K, KIND_Q8_K = 1, 5, 9, 10, 11, 12
KIND_Q4_1, KIND_Q5_0, KIND_Q5_1 = 2, 3, 4
KIND_Q2_K, KIND_Q3_K = 7, 8
KIND_Q8_1 = 6
DT_F32, DT_F16 = 0, 1
DT_BF16 = 2  # paged attention and conversions
DT_U32 = 8  # row indices of gather_rows
DT_F8_E4M3 = 14  # paged attention only: the KV cache
DT_I32, DT_I64 = 3, 11  # position tensors of the rotary epilogue
FLAG_FORCE_PACK = 1

ERROR_NAMES = {
    0: "SUCCESS", -1: "INVALID_ARGUMENT", -2: "OUT_OF_MEMORY", -3: "DEVICE_NOT_AVAILABLE", -4: "BACKEND_INIT_FAILED",
    -5: "INVALID_OPERATION", -6: "UNSUPPORTED_DTYPE", -7: "DIMENSION_MISMATCH", -8: "NOT_IMPLEMENTED",
}


class MarmotHipError(RuntimeError):
    def __init__(self, code: int, detail: str):
        super().__init__(f"marmot_hip error {code} ({ERROR_NAMES.get(code, '?')}): {detail}")
        self.code = code
        self.detail = detail


class Caps(C.Structure):
    _fields_ = [
        ("name", C.c_char * 64), ("arch", C.c_char * 32), ("num_compute_units", C.c_uint32),
        ("wavefront_size", C.c_uint32), ("clock_mhz", C.c_uint32), ("mem_clock_mhz", C.c_uint32),
        ("mem_bus_bits", C.c_uint32), ("l2_cache_kb", C.c_uint32), ("lds_kb_per_cu", C.c_uint32),
        ("total_mem_bytes", C.c_uint64), ("mem_bw_gbps", C.c_float), ("peak_tflops_fp16", C.c_float),
        ("peak_tops_int8", C.c_float),
    ]


class Rope(C.Structure):
    """marmot_hip_rope_t"""
    _fields_ = [("d_positions", C.c_void_p), ("positions_dtype", C.c_int), ("d_freqs", C.c_void_p),
                ("attn_scale", C.c_float), ("head_dim", C.c_uint32), ("rope_type", C.c_int),
                ("apply_to_q", C.c_int), ("apply_to_k", C.c_int)]


class PagedAttention(C.Structure):
    """marmot_hip_paged_attention_t: device pointers and element strides of the paged attention tensors"""
    _fields_ = [("token_count", C.c_uint32), ("layer_idx", C.c_uint32), ("num_q_heads", C.c_uint32),
                ("num_kv_heads", C.c_uint32), ("head_dim", C.c_uint32), ("block_size", C.c_uint32),
                ("scale", C.c_float), ("act_dtype", C.c_int), ("kv_dtype", C.c_int),
                ("d_token_meta", C.c_void_p), ("meta_stride", C.c_size_t * 2),
                ("d_q", C.c_void_p), ("d_k_new", C.c_void_p), ("d_v_new", C.c_void_p),
                ("q_stride", C.c_size_t * 3), ("k_stride", C.c_size_t * 3), ("v_stride", C.c_size_t * 3),
                ("d_kv_k", C.c_void_p), ("d_kv_v", C.c_void_p), ("kv_stride", C.c_size_t * 5),
                ("kv_blocks", C.c_size_t), ("kv_layers", C.c_size_t),
                ("d_block_table", C.c_void_p), ("table_stride", C.c_size_t * 2),
                ("max_seqs", C.c_size_t), ("max_blocks_per_seq", C.c_size_t),
                ("d_out", C.c_void_p), ("out_stride", C.c_size_t * 3),
                ("d_kv_k_scale", C.c_void_p), ("d_kv_v_scale", C.c_void_p), ("scale_stride", C.c_size_t * 3)]


class GgufTensor(C.Structure):
    """marmot_hip_gguf_tensor_t"""
    _fields_ = [("name", C.c_char_p), ("ggml_type", C.c_uint32), ("kind", C.c_int), ("dtype", C.c_int),
                ("ndim", C.c_uint32), ("shape", C.c_uint64 * 4), ("data", C.c_void_p), ("nbytes", C.c_size_t)]


class GgufKv(C.Structure):
    """marmot_hip_gguf_kv_t"""
    _fields_ = [("key", C.c_char_p), ("type", C.c_uint32), ("elem_type", C.c_uint32), ("count", C.c_uint64),
                ("data", C.c_void_p), ("nbytes", C.c_size_t)]


class MoeProbe(C.Structure):
    """marmot_hip_moe_probe_t"""
    _fields_ = [("d_sorted_tokens", C.c_void_p), ("d_route_pos", C.c_void_p), ("d_gate_out", C.c_void_p),
                ("d_up_out", C.c_void_p), ("d_fused_packed", C.c_void_p), ("d_fused_override", C.c_void_p)]


class PackedLayout(C.Structure):
    """marmot_hip_packed_layout_t"""
    _fields_ = [("act_kind", C.c_int), ("total_bytes", C.c_size_t), ("values_offset", C.c_size_t),
                ("values_per_row", C.c_size_t), ("scales_offset", C.c_size_t), ("blocks_per_row", C.c_size_t),
                ("sums_offset", C.c_size_t), ("sums_per_block", C.c_size_t)]


_vp, _sz, _i, _u32, _f = C.c_void_p, C.c_size_t, C.c_int, C.c_uint32, C.c_float

# name -> (restype, argtypes); every symbol include/marmot_hip.h declares
SIGNATURES = {
    "marmot_hip_device_create": (_i, [_i, C.POINTER(_vp)]),
    "marmot_hip_device_destroy": (None, [_vp]),
    "marmot_hip_alloc": (_i, [_vp, _sz, C.POINTER(_vp)]),
    "marmot_hip_free": (None, [_vp, _vp]),
    "marmot_hip_memcpy_to_device": (_i, [_vp, _vp, _vp, _sz]),
    "marmot_hip_memcpy_from_device": (_i, [_vp, _vp, _vp, _sz]),
    "marmot_hip_memcpy_device": (_i, [_vp, _vp, _vp, _sz]),
    "marmot_hip_memset": (_i, [_vp, _vp, _i, _sz]),
    "marmot_hip_synchronize": (_i, [_vp]),
    "marmot_hip_read_probe": (_i, [_vp, _vp, _sz, _vp]),
    "marmot_hip_timeline_attach": (_i, [_vp, _vp, _sz]),
    "marmot_hip_rows_plan_probe": (_i, [_i, C.c_uint32, _sz, _sz, _sz, _i, _i, C.POINTER(C.c_uint32), _sz]),
    "marmot_hip_timestamp": (_i, [_vp, _vp]),
    "marmot_hip_allocator_usage": (_i, [_vp, C.POINTER(_sz), C.POINTER(_sz), C.POINTER(_sz)]),
    "marmot_hip_stream": (_vp, [_vp]),
    "marmot_hip_last_error": (C.c_char_p, []),
    "marmot_hip_get_caps": (_i, [_vp, C.POINTER(Caps)]),
    "marmot_hip_branch_begin": (_i, [_vp]),
    "marmot_hip_branch_next": (_i, [_vp]),
    "marmot_hip_branch_join": (_i, [_vp]),
    "marmot_hip_graph_begin_capture": (_i, [_vp]),
    "marmot_hip_graph_end_capture": (_i, [_vp, C.POINTER(_vp)]),
    "marmot_hip_graph_launch": (_i, [_vp, _vp]),
    "marmot_hip_graph_destroy": (None, [_vp, _vp]),
    "marmot_hip_graph_max_nodes": (_sz, []),
    "marmot_hip_graph_last_capture_nodes": (_sz, [_vp]),
    "marmot_hip_event_create": (_i, [_vp, C.POINTER(_vp)]),
    "marmot_hip_event_destroy": (None, [_vp, _vp]),
    "marmot_hip_event_record": (_i, [_vp, _vp]),
    "marmot_hip_event_elapsed_ms": (_i, [_vp, _vp, _vp, C.POINTER(_f)]),
    "marmot_hip_block_values": (_sz, [_i]),
    "marmot_hip_block_bytes": (_sz, [_i]),
    "marmot_hip_row_bytes": (_sz, [_i, _sz]),
    "marmot_hip_dequantize": (_i, [_vp, _i, _vp, _sz, _sz, _vp]),
    "marmot_hip_quantize_activations": (_i, [_vp, _i, _vp, _i, _sz, _sz, _vp]),
    "marmot_hip_quantize_weights": (_i, [_vp, _i, _vp, _sz, _sz, _vp]),
    "marmot_hip_matmul_quantized": (_i, [_vp, _i, _vp, _vp, _i, _sz, _sz, _sz, _vp, _i, _vp, _i, _u32]),
    "marmot_hip_matmul_quantized_noalloc": (_i, [_vp, _i, _vp, _vp, _i, _sz, _sz, _sz, _vp, _i, _vp, _i, _u32]),
    "marmot_hip_matmul_quantized_dual": (_i, [_vp, _i, _vp, _vp, _vp, _i, _sz, _sz, _sz, _vp, _vp, _i, _u32]),
    "marmot_hip_matmul_qkv_quantized": (_i, [_vp, _i, _vp, _vp, _vp, _vp, _i, _sz, _sz, _sz, _vp, _vp, _vp, _i, _vp,
                                             _vp, _vp, _i]),
    "marmot_hip_matmul_qkv_rope_quantized": (_i, [_vp, _i, _vp, _vp, _vp, _vp, _i, _sz, _sz, _sz, _vp, _vp, _vp, _i,
                                                  _vp, _vp, _vp, _i, C.POINTER(Rope)]),
    "marmot_hip_rope_frequencies": (_i, [_i, _f, _f, _f, _f, _f, _f, _u32, _u32, _sz, _vp, C.POINTER(_f),
                                         C.POINTER(_u32)]),
    "marmot_hip_embedding_gather_quantized": (_i, [_vp, _i, _vp, _sz, _sz, _vp, _i, _sz, _vp, _i, _f, C.c_int32, _i]),
    "marmot_hip_packed_activation_bytes": (_sz, [_i, _sz, _sz]),
    "marmot_hip_pack_activations": (_i, [_vp, _i, _vp, _i, _sz, _sz, _vp]),
    "marmot_hip_matmul_prepacked": (_i, [_vp, _i, _vp, _vp, _sz, _sz, _sz, _vp, _i, _vp, _i]),
    "marmot_hip_rms_norm": (_i, [_vp, _vp, _vp, _vp, _f, _f, _sz, _sz, _vp]),
    "marmot_hip_rms_norm_pack": (_i, [_vp, _vp, _vp, _vp, _f, _f, _sz, _sz, _i, _vp, _vp]),
    "marmot_hip_glu": (_i, [_vp, _i, _vp, _vp, _sz, _sz, _sz, _sz, _sz, _vp]),
    "marmot_hip_swiglu_pack": (_i, [_vp, _vp, _vp, _sz, _sz, _i, _vp]),
    "marmot_hip_add": (_i, [_vp, _vp, _vp, _sz, _vp]),
    "marmot_hip_rope": (_i, [_vp, _vp, _i, _sz, _sz, _sz, _sz, C.POINTER(Rope), _vp]),
    "marmot_hip_unary": (_i, [_vp, _i, _vp, _i, _sz, _vp]),
    "marmot_hip_softmax": (_i, [_vp, _vp, _sz, _sz, _sz, _vp]),
    "marmot_hip_softmax_typed": (_i, [_vp, _i, _vp, _sz, _sz, _sz, _vp]),
    "marmot_hip_convert": (_i, [_vp, _vp, _i, _vp, _i, _sz]),
    "marmot_hip_gather_rows": (_i, [_vp, _vp, _sz, _sz, _sz, _vp, _i, _sz, _sz, _vp, _sz]),
    "marmot_hip_slice": (_i, [_vp, _vp, _sz, _i, C.POINTER(_sz), C.POINTER(_sz), C.POINTER(_sz), _vp]),
    "marmot_hip_paged_attention": (_i, [_vp, C.POINTER(PagedAttention), _i]),
    "marmot_hip_topk": (_i, [_vp, _vp, _sz, _sz, _sz, _vp, _vp]),
    "marmot_hip_softmax_rows": (_i, [_vp, _vp, _sz, _sz, _vp]),
    "marmot_hip_moe_experts": (_i, [_vp, _vp, _sz, _sz, _sz, _sz, _sz, _i, _i, _vp, _vp, _vp, _vp, _vp, _f, _i, _i,
                                    _vp]),
    "marmot_hip_moe_experts_probe": (_i, [_vp, _vp, _sz, _sz, _sz, _sz, _sz, _i, _i, _vp, _vp, _vp, _vp, _vp, _f, _i,
                                          _i, _vp, C.POINTER(MoeProbe)]),
    "marmot_hip_packed_activation_layout": (_i, [_i, _sz, _sz, C.POINTER(PackedLayout)]),
    "marmot_hip_last_route": (C.c_char_p, []),
    "marmot_hip_version": (C.c_char_p, []),
    "marmot_hip_gguf_open": (_i, [C.c_char_p, C.POINTER(_vp)]),
    "marmot_hip_gguf_close": (None, [_vp]),
    "marmot_hip_gguf_tensor_count": (_sz, [_vp]),
    "marmot_hip_gguf_alignment": (_sz, [_vp]),
    "marmot_hip_gguf_tensor": (_i, [_vp, _sz, C.POINTER(GgufTensor)]),
    "marmot_hip_gguf_find": (_i, [_vp, C.c_char_p, C.POINTER(GgufTensor)]),
    "marmot_hip_gguf_upload": (_i, [_vp, _vp, _sz, C.POINTER(_vp)]),
    "marmot_hip_gguf_kv_count": (_sz, [_vp]),
    "marmot_hip_gguf_kv": (_i, [_vp, _sz, C.POINTER(GgufKv)]),
    "marmot_hip_gguf_find_kv": (_i, [_vp, C.c_char_p, C.POINTER(GgufKv)]),
    "marmot_hip_gguf_kv_int": (_i, [C.POINTER(GgufKv), C.c_uint64, C.POINTER(C.c_int64)]),
    "marmot_hip_gguf_kv_float": (_i, [C.POINTER(GgufKv), C.c_uint64, C.POINTER(C.c_double)]),
    "marmot_hip_gguf_kv_string": (_i, [C.POINTER(GgufKv), C.c_uint64, C.POINTER(C.c_char_p), C.POINTER(_sz)]),
}

_lib = None


def lib_path() -> str:
    return os.environ.get("MARMOT_HIP_LIBRARY", os.path.join(HERE, "lib", "libmarmot_hip.so"))


def load_library():
    """Loads libmarmot_hip.so and declares every entry point. Raises if the library is not built."""
    global _lib
    if _lib is not None:
        return _lib
    path = lib_path()
    if not os.path.exists(path):
        raise FileNotFoundError(
            f"{path} is not built: run `python -c 'import __graft_entry__ as g; g.build()'` or "
            f"`make -C marmot_amd/csrc`. There is no CPU fallback for the HIP path.")
    lib = C.CDLL(path)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the header and the library disagree
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(code: int):
    if code != 0:
        detail = load_library().marmot_hip_last_error()
        raise MarmotHipError(code, detail.decode() if detail else "")
