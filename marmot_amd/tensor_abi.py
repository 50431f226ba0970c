"""Caller side of the marmot_tensor_t-level HIP backend, for tests and harnesses outside the marmot tree.

It plays the part marmot's core plays for a backend: builds ``marmot_tensor_t`` objects over host buffers with the
reference's exact struct layout, fills ``marmot_op_signature_t`` the way ``marmot_matmul_build`` does
(src/core/dispatch/matmul_build.c:86-146), asks ``marmot_hip_query_kernel`` for an op index, encodes bytecode
immediates as ``marmot_bc_compile`` does (src/core/bytecode/bytecode_compile.c:459-504, 628-669, 912-962) and runs
the program against the tables of ``marmot_hip_bc_get_tables`` with the loop of ``marmot_bc_execute``
(src/core/bytecode/bytecode.c:196-290). Tensor data moves only through the device vtable
(``memcpy_to_device(p, p)`` = "host copy is newer", ``memcpy_from_device(p, p)`` = "make the host copy current",
src/core/tensor/transfer.c:22, 49-55).

The struct definitions mirror include/marmot_hip_backend.h member for member.
"""
from __future__ import annotations

import ctypes as C
import struct
from typing import List, Optional, Sequence

import numpy as np

from . import capi

MAX_DIMS = 8

# marmot_error_t
SUCCESS, INVALID_ARGUMENT, OUT_OF_MEMORY, DEVICE_NOT_AVAILABLE, BACKEND_INIT_FAILED = 0, -1, -2, -3, -4
INVALID_OPERATION, UNSUPPORTED_DTYPE, DIMENSION_MISMATCH, NOT_IMPLEMENTED = -5, -6, -7, -8
# marmot_dtype_t
DTYPE_F32, DTYPE_F16, DTYPE_I32, DTYPE_I8, DTYPE_U8, DTYPE_I64 = 0, 1, 3, 5, 6, 11
DTYPE_BF16, DTYPE_U32, DTYPE_F8_E4M3 = 2, 8, 14
# marmot_quant_kind_t / marmot_quant_layout_t / marmot_memory_location_t
KIND_GENERIC, KIND_Q4_0, KIND_Q8_0, KIND_Q4_K, KIND_Q5_K, KIND_Q6_K, KIND_Q8_K = 0, 1, 5, 9, 10, 11, 12
KIND_Q4_1, KIND_Q5_0, KIND_Q5_1 = 2, 3, 4
KIND_Q2_K, KIND_Q3_K = 7, 8
KIND_Q8_1 = 6
LAYOUT_GENERIC, LAYOUT_GGUF = 0, 1
MEMORY_HOST, MEMORY_DEVICE = 0, 1
BACKEND_HIP = 3
# marmot_op_id_t / marmot_qscheme_id_t
OP_DEQUANTIZE, OP_MOE_EXPERTS, OP_MATMUL, OP_QUANTIZE, OP_LINEAR, OP_TOPK = 210, 263, 498, 524, 708, 901
OP_QKV_PROJECTION, OP_QKV_SHARED_INPUT, OP_QKV_ROPE = 191, 771, 778
OP_EMBEDDING = 853
OP_ROPE = 843
OP_PAGED_ATTENTION = 503
OP_SWIGLU, OP_GEGLU, OP_RMS_NORM_GEMMA, OP_ADD, OP_RMS_NORM = 331, 410, 447, 876, 929
OP_GATHER_ROWS, OP_RESHAPE, OP_SILU, OP_VIEW, OP_GELU, OP_GELU_TANH, OP_SLICE, OP_CONVERT, OP_SOFTMAX = (
    244, 258, 352, 502, 621, 642, 809, 932, 994)
# this backend's bytecode ops for them (include/marmot_hip_backend.h)
BC_OP_RMS_NORM_F32, BC_OP_RMS_NORM_GEMMA_F32, BC_OP_SWIGLU_F32, BC_OP_GEGLU_F32, BC_OP_ADD_F32 = 48, 49, 50, 51, 52
BC_OP_ROPE = 53
BC_OP_PAGED_ATTENTION = 54
BC_OP_GELU, BC_OP_GELU_TANH, BC_OP_SILU, BC_OP_SOFTMAX_F32 = 55, 56, 57, 58
BC_OP_RESHAPE, BC_OP_VIEW, BC_OP_SLICE, BC_OP_GATHER_ROWS, BC_OP_CONVERT = 59, 60, 61, 62, 63
PREFERENCE_DEFAULT, PREFERENCE_ENABLE, PREFERENCE_DISABLE = 0, 1, 2
QKV_LAYOUT_FUSED, QKV_LAYOUT_SEPARATE = 1, 2
QSCHEME_OF_KIND = {KIND_Q4_0: 1, KIND_Q4_1: 2, KIND_Q5_0: 3, KIND_Q5_1: 4, KIND_Q8_0: 5, KIND_Q2_K: 6, KIND_Q3_K: 7, KIND_Q4_K: 8,
                   KIND_Q5_K: 9, KIND_Q6_K: 10, KIND_Q8_K: 11, KIND_Q8_1: 12}
PROFILE_SCALAR = 4
MATMUL_LAYOUT_NT = 2
WEIGHT_LAYOUT_SEPARATE = 1
EPILOGUE_BIAS = 1
EPILOGUE_ROPE = 8
BC_END, BC_REG_INVALID, BC_INVALID_OFFSET = 0, 0xFFFF, 0xFFFFFFFF

DTYPE_F64, DTYPE_I16, DTYPE_U16, DTYPE_U64 = 10, 4, 7, 9
_NP_OF_DTYPE = {DTYPE_F32: np.float32, DTYPE_F16: np.float16, DTYPE_I32: np.int32, DTYPE_I8: np.int8,
                DTYPE_U8: np.uint8, DTYPE_I64: np.int64, DTYPE_U32: np.uint32, DTYPE_F64: np.float64,
                DTYPE_I16: np.int16, DTYPE_U16: np.uint16, DTYPE_U64: np.uint64}
_DTYPE_OF_NP = {np.dtype(v): k for k, v in _NP_OF_DTYPE.items()}


class Shape(C.Structure):
    _fields_ = [("ndim", C.c_size_t), ("shape", C.c_size_t * MAX_DIMS), ("strides", C.c_size_t * MAX_DIMS)]


class Tensor(C.Structure):
    _fields_ = [
        ("shape", Shape), ("dtype", C.c_int), ("data", C.c_void_p), ("capacity_bytes", C.c_size_t),
        ("owns_data", C.c_bool), ("quant_params", C.c_void_p), ("quant_kind", C.c_int), ("quant_layout", C.c_int),
        ("backend", C.c_int), ("ctx", C.c_void_p), ("memory_location", C.c_int), ("needs_sync", C.c_bool),
        ("packed_data", C.c_void_p), ("packed_src_data", C.c_void_p), ("packed_bytes", C.c_size_t),
        ("packed_row_bytes", C.c_size_t), ("packed_rows", C.c_size_t),
    ]


class Epilogue(C.Structure):
    _fields_ = [("bias", C.POINTER(Tensor)), ("enable_output_cast", C.c_bool), ("output_dtype", C.c_int)]


class RopeParams(C.Structure):
    _fields_ = [("positions", C.POINTER(Tensor)), ("scaling_type", C.c_int), ("rope_type", C.c_int),
                ("theta", C.c_float), ("freq_scale", C.c_float), ("ext_factor", C.c_float),
                ("attn_factor", C.c_float), ("beta_fast", C.c_float), ("beta_slow", C.c_float),
                ("orig_ctx_len", C.c_uint32), ("head_dim", C.c_uint32), ("apply_to_q", C.c_bool),
                ("apply_to_k", C.c_bool)]


class QkvFused(C.Structure):
    _fields_ = [("weight", C.POINTER(Tensor)), ("bias", C.POINTER(Tensor))]


class QkvSeparate(C.Structure):
    _fields_ = [(n, C.POINTER(Tensor)) for n in ("wq", "wk", "wv", "bq", "bk", "bv")]


class _QkvWeights(C.Union):
    _fields_ = [("fused", QkvFused), ("separate", QkvSeparate)]


class QkvDesc(C.Structure):
    _anonymous_ = ("weights",)
    _fields_ = [("input", C.POINTER(Tensor)), ("layout", C.c_int), ("weights", _QkvWeights),
                ("epilogue", C.POINTER(Epilogue)), ("out_q", C.POINTER(Tensor)), ("out_k", C.POINTER(Tensor)),
                ("out_v", C.POINTER(Tensor)), ("rope_params", C.POINTER(RopeParams))]


class EmbeddingGatherDesc(C.Structure):
    _fields_ = [("weights", C.POINTER(Tensor)), ("token_ids", C.POINTER(Tensor)), ("out", C.POINTER(Tensor)),
                ("dtype_out", C.c_int), ("scale", C.c_float), ("padding_id", C.c_int32), ("bounds_check", C.c_bool),
                ("prefer_gpu_private", C.c_int), ("allow_quant_decode_on_the_fly", C.c_int)]


class TopkDesc(C.Structure):
    _fields_ = [("x", C.POINTER(Tensor)), ("values_out", C.POINTER(Tensor)), ("indices_out", C.POINTER(Tensor)),
                ("axis", C.c_int32), ("k", C.c_uint32)]


class SoftmaxDesc(C.Structure):
    _fields_ = [("x", C.POINTER(Tensor)), ("out", C.POINTER(Tensor)), ("axis", C.c_int32)]


class ActivationParams(C.Structure):
    _fields_ = [("parameter_tensor", C.POINTER(Tensor)), ("bias", C.POINTER(Tensor)), ("alpha", C.c_float),
                ("beta", C.c_float), ("gamma", C.c_float)]


class RmsNormDesc(C.Structure):
    """marmot_rmsnorm_desc_t"""
    _fields_ = [("x", C.POINTER(Tensor)), ("residual", C.POINTER(Tensor)), ("weight", C.POINTER(Tensor)),
                ("out", C.POINTER(Tensor)), ("eps", C.c_float)]


class PagedAttentionKvScaleExt(C.Structure):
    """marmot_paged_attention_kv_scale_ext_t"""
    _fields_ = [("struct_size", C.c_uint32), ("struct_version", C.c_uint32), ("kv_k_scale", C.POINTER(Tensor)),
                ("kv_v_scale", C.POINTER(Tensor))]


class PagedAttentionDesc(C.Structure):
    """marmot_paged_attention_desc_t"""
    _fields_ = [("struct_size", C.c_uint32), ("struct_version", C.c_uint32), ("flags", C.c_uint64),
                ("token_count", C.c_uint32), ("layer_idx", C.c_uint32), ("num_q_heads", C.c_uint32),
                ("num_kv_heads", C.c_uint32), ("head_dim", C.c_uint32), ("block_size", C.c_uint32),
                ("scale", C.c_float)] + [(n, C.POINTER(Tensor)) for n in
                                         ("token_meta", "q", "k_new", "v_new", "kv_k", "kv_v", "block_table", "out")] + [
                    ("pnext", C.c_void_p), ("reserved", C.c_uint64 * 4)]

    @classmethod
    def default(cls) -> "PagedAttentionDesc":
        """marmot_paged_attention_desc_default (include/marmot/ops/paged_attention.h:59-83)"""
        d = cls()
        d.struct_size, d.struct_version, d.scale = C.sizeof(cls), 1, 1.0
        return d


class MoeDesc(C.Structure):
    _fields_ = [(n, C.POINTER(Tensor)) for n in
                ("hidden_states", "gate_exps", "up_exps", "down_exps", "topk_ids", "topk_weights", "out")] + [
        ("ffn_type", C.c_int), ("weights_scale", C.c_float), ("router_weight_policy", C.c_int)]


class MatmulDims(C.Structure):
    _fields_ = [("N", C.c_size_t), ("K", C.c_size_t), ("M", C.c_size_t)]


class SoftmaxDims(C.Structure):
    _fields_ = [("axis_size", C.c_uint32), ("inner_stride", C.c_uint32), ("outer_size", C.c_uint32),
                ("row_count", C.c_uint32)]


class SigDims(C.Union):
    _fields_ = [("matmul", MatmulDims), ("softmax", SoftmaxDims)]


class QuantBlock(C.Structure):
    _fields_ = [("block_size", C.c_uint32), ("group_size", C.c_uint32), ("scale_dtype", C.c_int),
                ("zero_point_dtype", C.c_int)]


class OpSignature(C.Structure):
    _fields_ = [
        ("op_id", C.c_int), ("profile_id", C.c_int), ("matmul_layout", C.c_int), ("input_dtype", C.c_int),
        ("weight_dtype", C.c_int), ("output_dtype", C.c_int), ("accum_dtype", C.c_int), ("qscheme_id", C.c_int),
        ("quant_block", QuantBlock), ("weight_layout", C.c_int), ("stride_mode", C.c_int),
        ("epilogue_flags", C.c_uint32), ("activation", C.c_int), ("variant_flags", C.c_uint32), ("dims", SigDims),
    ]


class KernelSelection(C.Structure):
    _fields_ = [
        ("supported", C.c_bool), ("kernel_id", C.c_int), ("op_index", C.c_uint16), ("estimated_us", C.c_double),
        ("est_comm_us", C.c_double), ("est_workspace_mb", C.c_double), ("confidence", C.c_float),
        ("fallback_reason", C.c_char_p), ("shardable_axes", C.c_uint32), ("device_affinity", C.c_uint32),
    ]


class _CapsApple(C.Structure):
    _fields_ = [("has_amx", C.c_bool), ("neural_engine_tops", C.c_uint32), ("has_arm_bf16", C.c_bool),
                ("has_arm_dotprod", C.c_bool), ("has_arm_sve", C.c_bool), ("cpu_microarch", C.c_int)]


class _CapsCuda(C.Structure):
    _fields_ = [("sm_count", C.c_uint32), ("shared_mem_kb", C.c_uint32), ("compute_capability", C.c_uint32)]


class _CapsBackend(C.Union):
    _fields_ = [("apple", _CapsApple), ("cuda", _CapsCuda)]


class _CapsTopology(C.Structure):
    _fields_ = [("total_cores", C.c_uint32), ("p_cores", C.c_uint32), ("e_cores", C.c_uint32),
                ("is_hybrid", C.c_bool)]


class DeviceCaps(C.Structure):
    _fields_ = [
        ("peak_flops_tflops_fp32", C.c_float), ("peak_flops_tflops_fp16", C.c_float), ("mem_bw_gbps", C.c_float),
        ("launch_overhead_us", C.c_float), ("edge_penalty_alpha", C.c_float),
        ("l1_cache_kb", C.c_uint32), ("l2_cache_kb", C.c_uint32), ("l3_cache_mb", C.c_uint32),
        ("num_compute_units", C.c_uint32), ("simd_width", C.c_uint32),
        ("has_fma", C.c_bool), ("has_fp16_compute", C.c_bool), ("has_bf16_compute", C.c_bool),
        ("has_tensor_cores", C.c_bool), ("has_simdgroup_mm", C.c_bool),
        ("h2d_bw_gbps", C.c_float), ("d2h_bw_gbps", C.c_float), ("d2d_bw_gbps", C.c_float),
        ("d2d_lat_us", C.c_float), ("copy_engines", C.c_uint32), ("max_streams", C.c_uint32),
        ("calib_dequant_us_q4k", C.c_float), ("calib_dequant_us_q5k", C.c_float),
        ("calib_dequant_us_q6k", C.c_float), ("calib_dequant_us_q8_0", C.c_float),
        ("calib_epilogue_scale", C.c_float),
        ("backend", _CapsBackend), ("topology", _CapsTopology),
    ]


class ContextPolicy(C.Structure):
    _fields_ = [("embedding_quant_output_dtype", C.c_int), ("quant_activation_mode", C.c_int),
                ("variant_flags_mask", C.c_uint32), ("embedding_prefer_gpu_private", C.c_bool),
                ("embedding_allow_quant_decode_on_the_fly", C.c_bool), ("matmul_requires_temp_tensors", C.c_bool),
                ("matmul_prefer_packed_weights", C.c_bool)]


class BackendPreferences(C.Structure):
    _fields_ = [("policy", ContextPolicy), ("routing_policy", C.c_int)]


class AllocatorUsage(C.Structure):
    _fields_ = [("current_bytes", C.c_size_t), ("peak_bytes", C.c_size_t), ("pooled_bytes", C.c_size_t),
                ("active_allocations", C.c_size_t), ("peak_allocations", C.c_size_t),
                ("total_allocations", C.c_uint64), ("pool_hits", C.c_uint64), ("pool_misses", C.c_uint64)]


class DeviceOps(C.Structure):
    _fields_ = [
        ("init", C.CFUNCTYPE(C.c_int, C.POINTER(C.c_void_p))),
        ("destroy", C.CFUNCTYPE(None, C.c_void_p)),
        ("configure", C.CFUNCTYPE(C.c_int, C.c_void_p, C.c_void_p)),
        ("alloc", C.CFUNCTYPE(C.c_int, C.c_void_p, C.c_size_t, C.POINTER(C.c_void_p))),
        ("free", C.CFUNCTYPE(None, C.c_void_p, C.c_void_p)),
        ("memcpy_to_device", C.CFUNCTYPE(C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t)),
        ("memcpy_from_device", C.CFUNCTYPE(C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t)),
        ("synchronize", C.CFUNCTYPE(C.c_int, C.c_void_p)),
        ("allocator_usage", C.CFUNCTYPE(C.c_int, C.c_void_p, C.POINTER(AllocatorUsage))),
        ("graph_batch_begin", C.CFUNCTYPE(C.c_int, C.c_void_p)),
        ("graph_batch_end", C.CFUNCTYPE(C.c_int, C.c_void_p, C.c_bool)),
        ("on_host_ptr_freed", C.CFUNCTYPE(None, C.c_void_p, C.c_void_p)),
        ("on_host_range_freed", C.CFUNCTYPE(None, C.c_void_p, C.c_void_p, C.c_size_t)),
    ]


class BcExecCtx(C.Structure):
    _fields_ = [("ctx", C.c_void_p), ("device_ctx", C.c_void_p)]


BcExecFn = C.CFUNCTYPE(C.c_int, C.c_void_p, C.POINTER(C.POINTER(Tensor)), C.POINTER(C.c_uint8),
                       C.POINTER(C.c_uint8))


class BcTables(C.Structure):
    _fields_ = [("imm_size", C.POINTER(C.c_uint16)), ("exec_table", C.POINTER(BcExecFn)),
                ("schema_id", C.POINTER(C.c_int)), ("op_count", C.c_uint16)]


class ResidencyStats(C.Structure):
    _fields_ = [("mirrors", C.c_size_t), ("mirrored_bytes", C.c_size_t), ("uploads", C.c_uint64),
                ("upload_bytes", C.c_uint64), ("downloads", C.c_uint64), ("download_bytes", C.c_uint64),
                ("activation_packs", C.c_uint64), ("activation_pack_hits", C.c_uint64)]


#: exported symbols of the tensor-level layer (checked against include/marmot_hip_backend.h by the tests)
BACKEND_SYMBOLS = [
    "marmot_get_hip_ops", "marmot_hip_query_kernel", "marmot_hip_detect_default_caps",
    "marmot_hip_default_preferences", "marmot_hip_bc_get_tables",
    "hip_matmul_quantized_q4_0", "hip_matmul_quantized_q8_0", "hip_matmul_quantized_q4_k",
    "hip_matmul_quantized_q5_k", "hip_matmul_quantized_q6_k", "hip_matmul_quantized_q4_1",
    "hip_matmul_quantized_q5_0", "hip_matmul_quantized_q5_1", "hip_matmul_qkv_q4_1", "hip_matmul_qkv_q5_0",
    "hip_matmul_qkv_q5_1", "hip_matmul_quantized_q2_k", "hip_matmul_quantized_q3_k", "hip_matmul_qkv_q2_k",
    "hip_matmul_qkv_q3_k", "hip_matmul_quantized_q8_1", "hip_matmul_qkv_q8_1", "hip_matmul_qkv_q4_0", "hip_matmul_qkv_q8_0", "hip_matmul_qkv_q4_k",
    "hip_matmul_qkv_q5_k", "hip_matmul_qkv_q6_k", "hip_embedding_gather", "hip_moe_experts_impl", "hip_topk_impl", "hip_quantize_block",
    "hip_dequantize_block", "marmot_hip_backend_last_error", "marmot_hip_backend_residency_stats",
    "hip_rmsnorm_impl", "hip_rmsnorm_gemma_impl", "hip_swiglu_f32", "hip_geglu_f32", "hip_add_f32",
    "hip_rope", "hip_paged_attention_impl",
    "hip_gelu", "hip_gelu_tanh", "hip_silu", "hip_softmax_impl", "hip_reshape", "hip_view", "hip_slice",
    "hip_gather_rows", "hip_convert",
]


def bind(lib: C.CDLL) -> C.CDLL:
    """Attach argument/return types of the tensor-level exports to an already loaded libmarmot_hip."""
    lib.marmot_get_hip_ops.restype = C.POINTER(DeviceOps)
    lib.marmot_get_hip_ops.argtypes = []
    lib.marmot_hip_query_kernel.restype = KernelSelection
    lib.marmot_hip_query_kernel.argtypes = [C.POINTER(OpSignature), C.POINTER(DeviceCaps)]
    lib.marmot_hip_detect_default_caps.restype = DeviceCaps
    lib.marmot_hip_detect_default_caps.argtypes = []
    lib.marmot_hip_default_preferences.restype = C.c_bool
    lib.marmot_hip_default_preferences.argtypes = [C.POINTER(DeviceCaps), C.POINTER(BackendPreferences)]
    lib.marmot_hip_bc_get_tables.restype = C.c_bool
    lib.marmot_hip_bc_get_tables.argtypes = [C.POINTER(BcTables)]
    for name in ("q4_0", "q4_1", "q5_0", "q5_1", "q8_0", "q8_1", "q2_k", "q3_k", "q4_k", "q5_k", "q6_k"):
        fn = getattr(lib, f"hip_matmul_quantized_{name}")
        fn.restype = C.c_int
        fn.argtypes = [C.c_void_p, C.POINTER(Tensor), C.POINTER(Tensor), C.POINTER(Epilogue), C.POINTER(Tensor)]
        fn = getattr(lib, f"hip_matmul_qkv_{name}")
        fn.restype = C.c_int
        fn.argtypes = [C.c_void_p, C.POINTER(QkvDesc)]
    lib.hip_embedding_gather.restype = C.c_int
    lib.hip_embedding_gather.argtypes = [C.c_void_p, C.POINTER(EmbeddingGatherDesc)]
    lib.hip_moe_experts_impl.restype = C.c_int
    lib.hip_moe_experts_impl.argtypes = [C.c_void_p, C.POINTER(MoeDesc)]
    lib.hip_topk_impl.restype = C.c_int
    lib.hip_topk_impl.argtypes = [C.c_void_p, C.POINTER(TopkDesc)]
    for name in ("hip_quantize_block", "hip_dequantize_block"):
        fn = getattr(lib, name)
        fn.restype = C.c_int
        fn.argtypes = [C.c_void_p, C.POINTER(Tensor), C.POINTER(Tensor)]
    for name in ("hip_rmsnorm_impl", "hip_rmsnorm_gemma_impl"):
        fn = getattr(lib, name)
        fn.restype = C.c_int
        fn.argtypes = [C.c_void_p, C.POINTER(RmsNormDesc)]
    for name in ("hip_swiglu_f32", "hip_geglu_f32", "hip_add_f32"):
        fn = getattr(lib, name)
        fn.restype = C.c_int
        fn.argtypes = [C.c_void_p, C.POINTER(Tensor), C.POINTER(Tensor), C.POINTER(Tensor)]
    lib.hip_paged_attention_impl.restype = C.c_int
    lib.hip_paged_attention_impl.argtypes = [C.c_void_p, C.POINTER(PagedAttentionDesc)]
    lib.hip_rope.restype = C.c_int
    lib.hip_rope.argtypes = [C.c_void_p, C.POINTER(Tensor), C.POINTER(RopeParams), C.POINTER(Tensor)]
    for name in ("hip_gelu", "hip_gelu_tanh", "hip_silu"):
        fn = getattr(lib, name)
        fn.restype = C.c_int
        fn.argtypes = [C.c_void_p, C.POINTER(Tensor), C.POINTER(ActivationParams), C.POINTER(Tensor)]
    lib.hip_softmax_impl.restype = C.c_int
    lib.hip_softmax_impl.argtypes = [C.c_void_p, C.POINTER(SoftmaxDesc)]
    lib.hip_reshape.restype = C.c_int
    lib.hip_reshape.argtypes = [C.c_void_p, C.POINTER(Tensor), C.POINTER(Tensor), C.POINTER(C.c_size_t), C.c_size_t]
    lib.hip_view.restype = C.c_int
    lib.hip_view.argtypes = [C.c_void_p, C.POINTER(Tensor), C.POINTER(Tensor), C.c_size_t]
    lib.hip_slice.restype = C.c_int
    lib.hip_slice.argtypes = [C.c_void_p, C.POINTER(Tensor), C.POINTER(Tensor), C.POINTER(C.c_size_t),
                              C.POINTER(C.c_size_t)]
    lib.hip_gather_rows.restype = C.c_int
    lib.hip_gather_rows.argtypes = [C.c_void_p, C.POINTER(Tensor), C.POINTER(Tensor), C.POINTER(Tensor)]
    lib.hip_convert.restype = C.c_int
    lib.hip_convert.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_int, C.c_void_p, C.c_size_t]
    lib.marmot_hip_backend_last_error.restype = C.c_int
    lib.marmot_hip_backend_last_error.argtypes = [C.POINTER(C.c_char_p)]
    lib.marmot_hip_backend_residency_stats.restype = None
    lib.marmot_hip_backend_residency_stats.argtypes = [C.c_void_p, C.POINTER(ResidencyStats)]
    return lib


class BackendError(RuntimeError):
    def __init__(self, code: int, detail: str):
        super().__init__(f"marmot HIP backend error {code}: {detail}")
        self.code = code
        self.detail = detail


class HostTensor:
    """A marmot_tensor_t over a numpy host buffer (the buffer is kept alive by this object)."""

    def __init__(self, array: np.ndarray, shape: Sequence[int], dtype: int, quant_kind: int = KIND_GENERIC):
        self.array = np.ascontiguousarray(array)
        self.t = Tensor()
        self.t.shape.ndim = len(shape)
        stride = 1
        for i in reversed(range(len(shape))):
            self.t.shape.shape[i] = shape[i]
            self.t.shape.strides[i] = stride
            stride *= shape[i]
        self.t.dtype = dtype
        self.t.data = self.array.ctypes.data
        self.t.capacity_bytes = self.array.nbytes
        self.t.owns_data = True
        self.t.quant_kind = quant_kind
        self.t.quant_layout = LAYOUT_GGUF if quant_kind != KIND_GENERIC else LAYOUT_GENERIC
        self.t.backend = BACKEND_HIP
        self.t.memory_location = MEMORY_HOST
        self.t.needs_sync = False

    @property
    def ptr(self):
        return C.pointer(self.t)

    @classmethod
    def dense(cls, array: np.ndarray) -> "HostTensor":
        a = np.ascontiguousarray(array)
        return cls(a, a.shape, _DTYPE_OF_NP[a.dtype])

    @classmethod
    def empty(cls, shape: Sequence[int], dtype: int) -> "HostTensor":
        return cls(np.zeros(shape, dtype=_NP_OF_DTYPE[dtype]), shape, dtype)

    @classmethod
    def strided(cls, view: np.ndarray, dtype: Optional[int] = None) -> "HostTensor":
        """A tensor over a numpy array or view as it lies in memory (any strides; the view keeps its base alive).
        `dtype` overrides the type the element size suggests (bfloat16 bits travel in uint16 arrays)."""
        obj = cls.__new__(cls)
        obj.array = view
        obj.t = Tensor()
        obj.t.shape.ndim = view.ndim
        last = 0
        for i in range(view.ndim):
            assert view.strides[i] % view.itemsize == 0 and view.strides[i] >= 0
            obj.t.shape.shape[i] = view.shape[i]
            obj.t.shape.strides[i] = view.strides[i] // view.itemsize
            last += (view.shape[i] - 1) * view.strides[i] if view.shape[i] else 0
        obj.extent_bytes = last + view.itemsize if view.size else 0
        obj.t.dtype = _DTYPE_OF_NP[view.dtype] if dtype is None else dtype
        obj.t.data = view.ctypes.data
        obj.t.capacity_bytes = obj.extent_bytes
        obj.t.owns_data = False
        obj.t.quant_kind, obj.t.quant_layout = KIND_GENERIC, LAYOUT_GENERIC
        obj.t.backend, obj.t.memory_location, obj.t.needs_sync = BACKEND_HIP, MEMORY_HOST, False
        return obj

    @classmethod
    def header(cls, shape: Sequence[int], dtype: int) -> "HostTensor":
        """A tensor without storage: what a graph hands a reshape or view node as its output. Its strides are zero
        (reshape fills them in when none is set), its data pointer null."""
        obj = cls.__new__(cls)
        obj.array = None
        obj.t = Tensor()
        obj.t.shape.ndim = len(shape)
        for i, n in enumerate(shape):
            obj.t.shape.shape[i] = n
        obj.t.dtype = dtype
        obj.t.data = None
        obj.t.capacity_bytes = 0
        obj.t.owns_data = False
        obj.t.quant_kind, obj.t.quant_layout = KIND_GENERIC, LAYOUT_GENERIC
        obj.t.backend, obj.t.memory_location, obj.t.needs_sync = BACKEND_HIP, MEMORY_HOST, False
        return obj

    @classmethod
    def quantized(cls, blocks: np.ndarray, shape: Sequence[int], kind: int) -> "HostTensor":
        """blocks: uint8 GGUF block bytes; shape: logical element shape as marmot stores it ([rows, cols] for a
        weight, [cols, rows, experts] for an expert stack)."""
        return cls(np.ascontiguousarray(blocks, dtype=np.uint8).reshape(-1), shape, DTYPE_U8, kind)


class HipContext:
    """What marmot_init(MARMOT_BACKEND_HIP) + the tensor transfer helpers amount to for one device."""

    def __init__(self, lib: Optional[C.CDLL] = None):
        self.lib = bind(lib if lib is not None else capi.load_library())
        self.ops = self.lib.marmot_get_hip_ops().contents
        dc = C.c_void_p()
        self._check(self.ops.init(C.byref(dc)))
        self.device_ctx = dc
        self._check(self.ops.configure(self.device_ctx, None))
        self.exec_ctx = BcExecCtx(C.c_void_p(1), self.device_ctx)  # ctx is opaque to the backend, must be non-null
        self.tables = BcTables()
        if not self.lib.marmot_hip_bc_get_tables(C.byref(self.tables)):
            raise BackendError(INVALID_ARGUMENT, "no bytecode tables")

    def close(self):
        if self.device_ctx:
            self.ops.destroy(self.device_ctx)
            self.device_ctx = C.c_void_p()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def last_error(self):
        detail = C.c_char_p()
        code = self.lib.marmot_hip_backend_last_error(C.byref(detail))
        return code, (detail.value or b"").decode()

    def _check(self, code: int):
        if code != SUCCESS:
            raise BackendError(code, self.last_error()[1])

    # --- transfers, as src/core/tensor/transfer.c does them
    def host_changed(self, t: HostTensor):
        self._check(self.ops.memcpy_to_device(self.device_ctx, t.t.data, t.t.data, t.array.nbytes))
        t.t.memory_location = MEMORY_HOST
        t.t.needs_sync = False

    def to_host(self, t: HostTensor) -> np.ndarray:
        if t.t.needs_sync:
            nbytes = getattr(t, "extent_bytes", t.array.nbytes)  # a strided view: its whole extent in memory
            self._check(self.ops.memcpy_from_device(self.device_ctx, t.t.data, t.t.data, nbytes))
            t.t.needs_sync = False
        return t.array

    def host_freed(self, t: HostTensor):
        self.ops.on_host_ptr_freed(self.device_ctx, t.t.data)

    def host_range_freed(self, t: HostTensor):
        """on_host_range_freed over the tensor's whole extent: no mirror that touches it survives."""
        nbytes = getattr(t, "extent_bytes", t.array.nbytes)
        self.ops.on_host_range_freed(self.device_ctx, t.t.data, nbytes)

    def synchronize(self):
        self._check(self.ops.synchronize(self.device_ctx))

    def residency(self) -> ResidencyStats:
        s = ResidencyStats()
        self.lib.marmot_hip_backend_residency_stats(self.device_ctx, C.byref(s))
        return s

    # --- kernel query (src/core/dispatch/matmul_build.c:120-135 for the signature)
    def matmul_signature(self, x: HostTensor, w: HostTensor, out: HostTensor, bias: bool = False) -> OpSignature:
        sig = OpSignature()
        sig.op_id = OP_MATMUL
        sig.profile_id = PROFILE_SCALAR
        sig.matmul_layout = MATMUL_LAYOUT_NT
        sig.input_dtype = x.t.dtype
        sig.weight_dtype = w.t.dtype
        sig.output_dtype = out.t.dtype
        sig.accum_dtype = DTYPE_F32
        sig.qscheme_id = QSCHEME_OF_KIND.get(w.t.quant_kind, 0)
        sig.weight_layout = WEIGHT_LAYOUT_SEPARATE
        sig.epilogue_flags = EPILOGUE_BIAS if bias else 0
        sig.dims.matmul.N = x.t.shape.shape[0]
        sig.dims.matmul.K = x.t.shape.shape[1]
        sig.dims.matmul.M = w.t.shape.shape[0]
        return sig

    def qkv_signature(self, x: HostTensor, wq: HostTensor, out_q: HostTensor, bias: bool = False,
                      rope: bool = False, op_id: int = OP_QKV_SHARED_INPUT) -> OpSignature:
        """marmot_matmul_qkv_build (src/core/dispatch/matmul_build.c:148-217)."""
        sig = self.matmul_signature(x, wq, out_q, bias)
        sig.op_id = op_id
        sig.weight_dtype = x.t.dtype  # quantized weights: the signature carries the activation dtype (:170)
        if rope:
            sig.epilogue_flags |= EPILOGUE_ROPE
        return sig

    def embedding_signature(self, table: HostTensor, ids: HostTensor, out: HostTensor) -> OpSignature:
        """The index dtype is this operation's input dtype (src/backends/cpu/kernels/embedding.def:19-30)."""
        sig = OpSignature()
        sig.op_id = OP_EMBEDDING
        sig.input_dtype = ids.t.dtype
        sig.weight_dtype = table.t.dtype
        sig.output_dtype = out.t.dtype
        sig.accum_dtype = DTYPE_F32
        sig.qscheme_id = QSCHEME_OF_KIND.get(table.t.quant_kind, 0)
        sig.weight_layout = WEIGHT_LAYOUT_SEPARATE
        return sig

    def float_op_signature(self, op_id: int, dtype: int = DTYPE_F32) -> OpSignature:
        """Normalization and elementwise operations: one dtype for input, weight, output (cpu/kernels/normalization.def,
        elementwise.def)."""
        sig = OpSignature()
        sig.op_id = op_id
        sig.input_dtype = sig.weight_dtype = sig.output_dtype = dtype
        sig.accum_dtype = DTYPE_F32
        return sig

    def query(self, sig: OpSignature, caps: Optional[DeviceCaps] = None) -> KernelSelection:
        caps = caps if caps is not None else self.lib.marmot_hip_detect_default_caps()
        return self.lib.marmot_hip_query_kernel(C.byref(sig), C.byref(caps))

    # --- bytecode execution (src/core/bytecode/bytecode.c:196-290)
    def execute(self, program: "Program") -> int:
        code = bytes(program.code) + struct.pack("<H", BC_END)
        regs = (C.POINTER(Tensor) * max(1, len(program.regs)))(*[r.ptr for r in program.regs])
        pool = (C.c_uint8 * max(1, len(program.const_pool))).from_buffer_copy(
            bytes(program.const_pool) or b"\0")
        pc, end = 0, len(code)
        while True:
            if pc + 2 > end:
                return INVALID_ARGUMENT  # truncated stream
            (op,) = struct.unpack_from("<H", code, pc)
            pc += 2
            if op == BC_END:
                return SUCCESS
            if op >= self.tables.op_count:
                return INVALID_ARGUMENT
            n = self.tables.imm_size[op]
            if pc + n > end:
                return INVALID_ARGUMENT
            imm = (C.c_uint8 * max(1, n)).from_buffer_copy(code[pc:pc + n] or b"\0")
            pc += n
            fn = self.tables.exec_table[op]
            if not fn:
                return NOT_IMPLEMENTED
            status = fn(C.cast(C.pointer(self.exec_ctx), C.c_void_p), regs, imm, pool)
            if status != SUCCESS:
                return status


class Program:
    """Bytecode builder for the schemas the HIP backend executes."""

    def __init__(self):
        self.code = bytearray()
        self.const_pool = bytearray()
        self.regs: List[HostTensor] = []
        self._keep = []

    def reg(self, t: Optional[HostTensor]) -> int:
        if t is None:
            return BC_REG_INVALID
        for i, r in enumerate(self.regs):
            if r is t:
                return i
        self.regs.append(t)
        return len(self.regs) - 1

    def _const(self, blob: bytes, align: int) -> int:
        while len(self.const_pool) % align:
            self.const_pool.append(0)
        off = len(self.const_pool)
        self.const_pool += blob
        return off

    def matmul(self, op_index: int, x: HostTensor, w: HostTensor, out: HostTensor,
               bias: Optional[HostTensor] = None, with_epilogue: Optional[bool] = None):
        with_epilogue = (bias is not None) if with_epilogue is None else with_epilogue
        off = BC_INVALID_OFFSET
        if with_epilogue:
            ep = Epilogue()
            ep.bias = bias.ptr if bias is not None else None
            ep.enable_output_cast = False
            ep.output_dtype = out.t.dtype
            self._keep.append(ep)
            off = self._const(bytes(ep), 8)
        self.code += struct.pack("<HHHHIH", op_index, self.reg(x), self.reg(w), self.reg(bias), off, self.reg(out))

    def qkv(self, op_index: int, x: HostTensor, wq, wk, wv, out_q, out_k, out_v, bq=None, bk=None, bv=None,
            rope: Optional[RopeParams] = None):
        """bytecode_compile.c:670-715."""
        rope_off = BC_INVALID_OFFSET
        if rope is not None:
            self._keep.append(rope)
            rope_off = self._const(bytes(rope), 8)
        self.code += struct.pack("<H7HII3H", op_index, *[self.reg(t) for t in (x, wq, wk, wv, bq, bk, bv)],
                                 BC_INVALID_OFFSET, rope_off, self.reg(out_q), self.reg(out_k), self.reg(out_v))

    def embedding(self, op_index: int, table: HostTensor, ids: HostTensor, out: HostTensor, scale: float = 1.0,
                  padding_id: int = -1, bounds_check: bool = True):
        """bytecode_compile.c:989-1018."""
        self.code += struct.pack("<H3HIfI3B", op_index, self.reg(table), self.reg(ids), self.reg(out), out.t.dtype,
                                 scale, padding_id & 0xFFFFFFFF, int(bounds_check), 0, 1)

    def moe_experts(self, op_index: int, hidden, gate, up, down, ids, weights, out, ffn_type=0, weights_scale=1.0,
                    policy=1):
        self.code += struct.pack("<H7HIfI", op_index, *[self.reg(t) for t in (hidden, gate, up, down, ids, weights,
                                                                              out)],
                                 ffn_type, weights_scale, policy)

    def topk(self, op_index: int, x, values, indices, k: int, axis: int = 1):
        self.code += struct.pack("<HHHHII", op_index, self.reg(x), self.reg(values), self.reg(indices),
                                 axis & 0xFFFFFFFF, k)

    def rms_norm(self, op_index: int, x, weight, residual, out, eps: float):
        self.code += struct.pack("<HHHHHf", op_index, self.reg(x), self.reg(weight), self.reg(residual),
                                 self.reg(out), eps)

    def binary(self, op_index: int, a, b, out):
        self.code += struct.pack("<HHHH", op_index, self.reg(a), self.reg(b), self.reg(out))

    def rope(self, op_index: int, x, out, params: Optional[RopeParams], positions: Optional[HostTensor] = None,
             n_past: int = 0, n_rot: int = 0):
        """bytecode_compile.c:598-623: the parameters travel in the constant pool; a positions register replaces
        the tensor they name."""
        off = BC_INVALID_OFFSET
        if params is not None:
            self._keep.append(params)
            off = self._const(bytes(params), 8)
        self.code += struct.pack("<HHHHIII", op_index, self.reg(x), self.reg(out), self.reg(positions), off, n_past,
                                 n_rot)

    def paged_attention(self, op_index: int, token_meta, q, k_new, v_new, kv_k, kv_v, block_table, out, token_count: int,
                        layer_idx: int, num_q_heads: int, num_kv_heads: int, head_dim: int, block_size: int,
                        scale: float, kv_k_scale=None, kv_v_scale=None):
        """bytecode_compile.c:553-597: ten tensor registers (the two scale tensors of the FP8 cache may be absent), six
        u32 and the scale."""
        self.code += struct.pack("<H10H6If", op_index, self.reg(token_meta), self.reg(q), self.reg(k_new),
                                 self.reg(v_new), self.reg(kv_k), self.reg(kv_v), self.reg(block_table),
                                 self.reg(kv_k_scale), self.reg(kv_v_scale), self.reg(out), token_count, layer_idx,
                                 num_q_heads, num_kv_heads, head_dim, block_size, scale)

    def quantize(self, op_index: int, x, out):
        self.code += struct.pack("<HHIHII", op_index, self.reg(x), BC_INVALID_OFFSET, self.reg(out),
                                 out.t.quant_kind, out.t.quant_layout)

    def dequantize(self, op_index: int, x, out):
        self.code += struct.pack("<HHHII", op_index, self.reg(x), self.reg(out), x.t.quant_kind, x.t.quant_layout)

    def unary(self, op_index: int, x, out, params: Optional[ActivationParams] = None):
        """bytecode_compile.c:331-356."""
        off = BC_INVALID_OFFSET
        if params is not None:
            self._keep.append(params)
            off = self._const(bytes(params), 8)
        self.code += struct.pack("<HHHI", op_index, self.reg(x), self.reg(out), off)

    def softmax(self, op_index: int, x, out, axis: int = -1):
        """bytecode_compile.c:440-458."""
        self.code += struct.pack("<HHHI", op_index, self.reg(x), self.reg(out), axis & 0xFFFFFFFF)

    def reshape(self, op_index: int, x, out, new_shape: Sequence[int]):
        """bytecode_compile.c:718-745: the shape travels in the constant pool as size_t values."""
        off = self._const(struct.pack(f"<{len(new_shape)}Q", *new_shape), 8)
        self.code += struct.pack("<HHHIQ", op_index, self.reg(x), self.reg(out), off, len(new_shape))

    def view(self, op_index: int, x, out, byte_offset: int):
        """bytecode_compile.c:746-763."""
        self.code += struct.pack("<HHHQ", op_index, self.reg(x), self.reg(out), byte_offset)

    def slice(self, op_index: int, x, out, starts: Sequence[int], sizes: Sequence[int]):
        """bytecode_compile.c:863-892."""
        s0 = self._const(struct.pack(f"<{len(starts)}Q", *starts), 8)
        s1 = self._const(struct.pack(f"<{len(sizes)}Q", *sizes), 8)
        self.code += struct.pack("<HHHII", op_index, self.reg(x), self.reg(out), s0, s1)

    def gather_rows(self, op_index: int, x, indices, out):
        """bytecode_compile.c:893-911."""
        self.code += struct.pack("<HHHH", op_index, self.reg(x), self.reg(indices), self.reg(out))

    def convert(self, op_index: int, dst: HostTensor, src: HostTensor, n: int):
        """bytecode_compile.c:1020-1043: the two host addresses travel by value in the constant pool."""
        self._keep += [dst, src]
        d = self._const(struct.pack("<Q", dst.t.data), 8)
        s_ = self._const(struct.pack("<Q", src.t.data), 8)
        self.code += struct.pack("<HIIQII", op_index, d, s_, n, dst.t.dtype, src.t.dtype)
