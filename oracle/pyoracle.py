"""ctypes bindings for the CPU oracle and for the reference-built leaf library.

TEST INFRASTRUCTURE ONLY: imported by tests/, by ``__graft_entry__.smoke()`` and by the
``cpu_baseline`` leg of ``bench.py`` — never by the product package.

``Oracle``  wraps ``oracle/libmarmot_oracle.so`` (own restatement, see marmot_oracle.h).
``RefLib``  wraps ``oracle/_ref/libmarmot_ref.so`` — the reference's own quantizer / dequantizer /
            packer / block-dot translation units compiled as they lie (oracle/Makefile, target ``ref``).
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ORACLE_SO = os.path.join(HERE, "libmarmot_oracle.so")
REF_SO = os.path.join(HERE, "_ref", "libmarmot_ref.so")

KIND_Q4_0, KIND_Q8_0, KIND_Q4_K, KIND_Q5_K, KIND_Q6_K, KIND_Q8_K = 1, 5, 9, 10, 11, 12
KIND_Q4_1, KIND_Q5_0, KIND_Q5_1 = 2, 3, 4
KIND_Q2_K, KIND_Q3_K = 7, 8
KIND_Q8_1 = 6
KINDS = {"q4_0": KIND_Q4_0, "q8_0": KIND_Q8_0, "q4_k": KIND_Q4_K, "q5_k": KIND_Q5_K, "q6_k": KIND_Q6_K,
         "q8_k": KIND_Q8_K, "q4_1": KIND_Q4_1, "q5_0": KIND_Q5_0, "q5_1": KIND_Q5_1,
         "q2_k": KIND_Q2_K, "q3_k": KIND_Q3_K, "q8_1": KIND_Q8_1}
BLOCK_VALUES = {KIND_Q4_0: 32, KIND_Q8_0: 32, KIND_Q4_K: 256, KIND_Q5_K: 256, KIND_Q6_K: 256, KIND_Q8_K: 256,
                KIND_Q4_1: 32, KIND_Q5_0: 32, KIND_Q5_1: 32, KIND_Q2_K: 256, KIND_Q3_K: 256,
                KIND_Q8_1: 32}
BLOCK_BYTES = {KIND_Q4_0: 18, KIND_Q8_0: 34, KIND_Q4_K: 144, KIND_Q5_K: 176, KIND_Q6_K: 210, KIND_Q8_K: 292,
               KIND_Q4_1: 20, KIND_Q5_0: 22, KIND_Q5_1: 24, KIND_Q2_K: 84, KIND_Q3_K: 110,
               KIND_Q8_1: 36}
DT_F32, DT_F16 = 0, 1
DT_BF16 = 2
DT_F8_E4M3 = 14
DT_I32, DT_I64 = 3, 11  # marmot_dtype_t values of the position tensors the rotary epilogue accepts
ROPE_SCALING_NONE, ROPE_SCALING_LINEAR, ROPE_SCALING_YARN, ROPE_SCALING_LONGROPE = 0, 1, 2, 3
ROPE_TYPE_NORM, ROPE_TYPE_NEOX = 0, 1



class PagedAttentionArgs(C.Structure):
    """mo_paged_attention_args: the tensors of marmot_paged_attention_desc_t as pointers and element strides."""
    _fields_ = [("token_count", C.c_uint32), ("layer_idx", C.c_uint32), ("num_q_heads", C.c_uint32),
                ("num_kv_heads", C.c_uint32), ("head_dim", C.c_uint32), ("block_size", C.c_uint32),
                ("scale", C.c_float), ("act_dtype", C.c_int), ("kv_dtype", C.c_int),
                ("token_meta", C.c_void_p), ("meta_stride", C.c_size_t * 2),
                ("q", C.c_void_p), ("k_new", C.c_void_p), ("v_new", C.c_void_p),
                ("q_stride", C.c_size_t * 3), ("k_stride", C.c_size_t * 3), ("v_stride", C.c_size_t * 3),
                ("kv_k", C.c_void_p), ("kv_v", C.c_void_p), ("kv_stride", C.c_size_t * 5),
                ("kv_blocks", C.c_size_t), ("kv_layers", C.c_size_t),
                ("block_table", C.c_void_p), ("table_stride", C.c_size_t * 2),
                ("max_seqs", C.c_size_t), ("max_blocks_per_seq", C.c_size_t),
                ("out", C.c_void_p), ("out_stride", C.c_size_t * 3),
                ("kv_k_scale", C.c_void_p), ("kv_v_scale", C.c_void_p), ("scale_stride", C.c_size_t * 3)]


def float_dtype_code(a: np.ndarray, bf16: bool = False) -> int:
    """marmot_dtype_t of a float tensor held in numpy: bfloat16 travels as uint16 bits."""
    if bf16:
        assert a.dtype == np.uint16
        return DT_BF16
    return {np.dtype(np.float32): DT_F32, np.dtype(np.float16): DT_F16}[a.dtype]


def element_strides(a: np.ndarray):
    assert all(s % a.itemsize == 0 for s in a.strides)
    return [s // a.itemsize for s in a.strides]


def paged_attention_args(token_meta, q, k_new, v_new, kv_k, kv_v, block_table, layer_idx, scale, act_bf16=False,
                         kv_bf16=False, token_count=None, ptr=None, kv_k_scale=None, kv_v_scale=None):
    """(PagedAttentionArgs over the given numpy arrays, freshly allocated out array). `ptr` maps an array to the
    address to put into the struct (default: the array's own memory)."""
    ptr = ptr or (lambda a: a.ctypes.data)
    assert token_meta.dtype == np.uint32 and block_table.dtype == np.uint32
    out = np.zeros(q.shape, dtype=q.dtype)
    a = PagedAttentionArgs()
    a.token_count = q.shape[0] if token_count is None else token_count
    a.layer_idx, a.scale = layer_idx, scale
    a.num_q_heads, a.num_kv_heads, a.head_dim, a.block_size = q.shape[1], k_new.shape[1], q.shape[2], kv_k.shape[3]
    a.act_dtype = float_dtype_code(q, act_bf16)
    if kv_k.dtype == np.uint8:  # the FLOAT8_E4M3 cache with its per-block scales [blocks, layers, kv heads]
        a.kv_dtype = DT_F8_E4M3
        if kv_k_scale is not None:
            assert kv_k_scale.dtype == np.float32 and kv_k_scale.strides == kv_v_scale.strides
            a.kv_k_scale, a.kv_v_scale = ptr(kv_k_scale), ptr(kv_v_scale)
            a.scale_stride = (C.c_size_t * 3)(*element_strides(kv_k_scale))
    else:
        a.kv_dtype = float_dtype_code(kv_k, kv_bf16)
    a.token_meta, a.meta_stride = ptr(token_meta), (C.c_size_t * 2)(*element_strides(token_meta))
    a.q, a.k_new, a.v_new = ptr(q), ptr(k_new), ptr(v_new)
    a.q_stride = (C.c_size_t * 3)(*element_strides(q))
    a.k_stride = (C.c_size_t * 3)(*element_strides(k_new))
    a.v_stride = (C.c_size_t * 3)(*element_strides(v_new))
    assert kv_k.shape == kv_v.shape and kv_k.strides == kv_v.strides
    a.kv_k, a.kv_v, a.kv_stride = ptr(kv_k), ptr(kv_v), (C.c_size_t * 5)(*element_strides(kv_k))
    a.kv_blocks, a.kv_layers = kv_k.shape[0], kv_k.shape[1]
    a.block_table, a.table_stride = ptr(block_table), (C.c_size_t * 2)(*element_strides(block_table))
    a.max_seqs, a.max_blocks_per_seq = block_table.shape
    a.out, a.out_stride = ptr(out), (C.c_size_t * 3)(*element_strides(out))
    return a, out

class RopeParams(C.Structure):
    """mo_rope_params: marmot_rope_params_t without the positions tensor."""
    _fields_ = [("scaling_type", C.c_int), ("rope_type", C.c_int), ("theta", C.c_float), ("freq_scale", C.c_float),
                ("ext_factor", C.c_float), ("attn_factor", C.c_float), ("beta_fast", C.c_float),
                ("beta_slow", C.c_float), ("orig_ctx_len", C.c_uint32), ("head_dim", C.c_uint32),
                ("apply_to_q", C.c_int), ("apply_to_k", C.c_int)]

    @classmethod
    def default(cls, **kw) -> "RopeParams":
        """marmot_rope_params_default (include/marmot/ops/matmul.h:45-61)."""
        p = cls(ROPE_SCALING_NONE, ROPE_TYPE_NORM, 10000.0, 1.0, 0.0, 1.0, 32.0, 1.0, 0, 0, 1, 1)
        for k, v in kw.items():
            setattr(p, k, v)
        return p


def row_bytes(kind: int, k: int) -> int:
    bv = BLOCK_VALUES[kind]
    return ((k + bv - 1) // bv) * BLOCK_BYTES[kind]


def build_oracle(force: bool = False) -> str:
    if force or not os.path.exists(ORACLE_SO):
        subprocess.check_call(["make", "-C", HERE, "-B" if force else "-s", "all"])
    return ORACLE_SO


def _ptr(a: np.ndarray):
    return a.ctypes.data_as(C.c_void_p)


class Oracle:
    def __init__(self, path: str | None = None):
        path = path or build_oracle()
        L = C.CDLL(path)
        self.L = L
        L.mo_f16_to_f32.restype = C.c_float
        L.mo_f16_to_f32.argtypes = [C.c_uint16]
        L.mo_f32_to_f16.restype = C.c_uint16
        L.mo_f32_to_f16.argtypes = [C.c_float]
        L.mo_quantize_rows.restype = C.c_int
        L.mo_quantize_rows.argtypes = [C.c_int, C.c_void_p, C.c_size_t, C.c_size_t, C.c_void_p]
        L.mo_dequantize_rows.restype = C.c_int
        L.mo_dequantize_rows.argtypes = [C.c_int, C.c_void_p, C.c_size_t, C.c_size_t, C.c_void_p]
        for n in ("mo_pack_q8_0", "mo_pack_q8_k"):
            f = getattr(L, n)
            f.restype = None
            f.argtypes = [C.c_void_p, C.c_int, C.c_size_t, C.c_void_p]
        for n in ("mo_vec_dot_q8_0_q8_0", "mo_vec_dot_q4_0_q8_0", "mo_vec_dot_q4_k_q8_k", "mo_vec_dot_q5_k_q8_k",
                  "mo_vec_dot_q6_k_q8_k", "mo_vec_dot_q4_1_q8_0", "mo_vec_dot_q5_0_q8_0", "mo_vec_dot_q5_1_q8_0",
                  "mo_vec_dot_q2_k_q8_k", "mo_vec_dot_q3_k_q8_k", "mo_vec_dot_q8_1_q8_0"):
            f = getattr(L, n)
            f.restype = C.c_float
            f.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]
        L.mo_vec_dot_f16.restype = C.c_float
        L.mo_vec_dot_f16.argtypes = [C.c_int, C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t]
        L.mo_matmul_quantized.restype = C.c_int
        L.mo_matmul_quantized.argtypes = [
            C.c_int, C.c_void_p, C.c_void_p, C.c_int, C.c_size_t, C.c_size_t, C.c_size_t, C.c_void_p, C.c_void_p,
            C.c_int, C.c_int, C.c_int,
        ]
        L.mo_matmul_qkv_separate.restype = C.c_int
        L.mo_matmul_qkv_separate.argtypes = [
            C.c_int, C.POINTER(C.c_void_p), C.c_void_p, C.c_int, C.c_size_t, C.c_size_t, C.c_size_t,
            C.POINTER(C.c_void_p), C.c_int, C.POINTER(C.c_void_p),
        ]
        L.mo_matmul_qkv_separate_rope.restype = C.c_int
        L.mo_matmul_qkv_separate_rope.argtypes = L.mo_matmul_qkv_separate.argtypes + [
            C.POINTER(RopeParams), C.c_void_p, C.c_int]
        L.mo_rope_frequencies.restype = C.c_int
        L.mo_rope_frequencies.argtypes = [C.POINTER(RopeParams), C.c_size_t, C.c_void_p, C.POINTER(C.c_float)]
        L.mo_rope_resolve_head_dim.restype = C.c_size_t
        L.mo_rope_resolve_head_dim.argtypes = [C.c_size_t, C.c_uint32]
        L.mo_rope.restype = C.c_int
        L.mo_rope.argtypes = [C.c_void_p, C.c_int, C.c_size_t, C.c_size_t, C.c_size_t, C.c_size_t,
                              C.POINTER(RopeParams), C.c_void_p, C.c_int, C.c_void_p]
        L.mo_rope_rotate_row.restype = None
        L.mo_rope_rotate_row.argtypes = [C.c_void_p, C.c_size_t, C.c_size_t, C.c_float, C.c_void_p, C.c_float, C.c_int]
        L.mo_embedding_gather_quantized.restype = C.c_int
        L.mo_embedding_gather_quantized.argtypes = [
            C.c_int, C.c_void_p, C.c_size_t, C.c_size_t, C.c_void_p, C.c_int, C.c_size_t, C.c_void_p, C.c_int,
            C.c_float, C.c_int32, C.c_int, C.POINTER(C.c_size_t)]
        L.mo_topk.restype = C.c_int
        L.mo_topk.argtypes = [C.c_void_p, C.c_size_t, C.c_size_t, C.c_size_t, C.c_void_p, C.c_void_p]
        L.mo_softmax_rows.restype = None
        L.mo_softmax_rows.argtypes = [C.c_void_p, C.c_size_t, C.c_size_t, C.c_void_p]
        L.mo_rms_norm.restype = C.c_int
        L.mo_rms_norm.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_float, C.c_float, C.c_size_t, C.c_size_t,
                                  C.c_void_p]
        L.mo_glu.restype = C.c_int
        L.mo_glu.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int, C.c_void_p]
        L.mo_moe_glu.restype = C.c_int
        L.mo_moe_glu.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int, C.c_void_p]
        L.mo_moe_experts.restype = C.c_int
        L.mo_moe_experts.argtypes = [
            C.c_void_p, C.c_size_t, C.c_size_t, C.c_size_t, C.c_size_t, C.c_size_t, C.c_int, C.c_int, C.c_void_p,
            C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_float, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p,
        ]
        L.mo_f32_to_fp8_e4m3.restype = C.c_uint8
        L.mo_f32_to_fp8_e4m3.argtypes = [C.c_float]
        L.mo_fp8_e4m3_to_f32.restype = C.c_float
        L.mo_fp8_e4m3_to_f32.argtypes = [C.c_uint8]
        L.mo_paged_attention.restype = C.c_int
        L.mo_paged_attention.argtypes = [C.POINTER(PagedAttentionArgs)]
        L.mo_row_grain.restype = C.c_size_t
        L.mo_row_grain.argtypes = [C.c_size_t, C.c_size_t, C.c_size_t]
        L.mo_unary.restype = C.c_int
        L.mo_unary.argtypes = [C.c_int, C.c_void_p, C.c_int, C.c_size_t, C.c_void_p]
        L.mo_softmax.restype = C.c_int
        L.mo_softmax.argtypes = [C.c_void_p, C.c_size_t, C.c_size_t, C.c_size_t, C.c_void_p]
        L.mo_softmax_typed.restype = C.c_int
        L.mo_softmax_typed.argtypes = [C.c_int, C.c_void_p, C.c_size_t, C.c_size_t, C.c_size_t, C.c_void_p]
        L.mo_convert.restype = C.c_int
        L.mo_convert.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_int, C.c_size_t]
        L.mo_gather_rows.restype = C.c_int
        L.mo_gather_rows.argtypes = [C.c_void_p, C.c_size_t, C.c_size_t, C.c_size_t, C.c_size_t, C.c_void_p, C.c_int,
                                     C.c_size_t, C.c_size_t, C.c_void_p, C.c_size_t, C.POINTER(C.c_size_t)]
        L.mo_slice.restype = C.c_int
        L.mo_slice.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t, C.POINTER(C.c_size_t),
                               C.POINTER(C.c_size_t), C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)]

    # ---- fp16
    def f16_to_f32(self, h: int) -> float:
        return float(self.L.mo_f16_to_f32(h))

    def f32_to_f16(self, f: float) -> int:
        return int(self.L.mo_f32_to_f16(np.float32(f)))

    # ---- quantize / dequantize
    def quantize(self, kind: int, x: np.ndarray) -> np.ndarray:
        x = np.ascontiguousarray(x, dtype=np.float32)
        if x.ndim == 1:
            x = x[None, :]
        rows, k = x.shape
        out = np.zeros((rows, row_bytes(kind, k)), dtype=np.uint8)
        st = self.L.mo_quantize_rows(kind, _ptr(x), rows, k, _ptr(out))
        if st != 0:
            raise RuntimeError(f"mo_quantize_rows -> {st}")
        return out

    def dequantize(self, kind: int, blocks: np.ndarray, k: int) -> np.ndarray:
        blocks = np.ascontiguousarray(blocks, dtype=np.uint8)
        if blocks.ndim == 1:
            blocks = blocks[None, :]
        rows = blocks.shape[0]
        assert blocks.shape[1] == row_bytes(kind, k), (blocks.shape, row_bytes(kind, k))
        out = np.zeros((rows, k), dtype=np.float32)
        st = self.L.mo_dequantize_rows(kind, _ptr(blocks), rows, k, _ptr(out))
        if st != 0:
            raise RuntimeError(f"mo_dequantize_rows -> {st}")
        return out

    # ---- activation packers
    def pack(self, act_kind: int, x: np.ndarray) -> np.ndarray:
        """x: 1-D float32 or float16 row -> packed Q8_0 / Q8_K blocks (uint8)."""
        if x.dtype == np.float16:
            dt = DT_F16
        else:
            x = np.ascontiguousarray(x, dtype=np.float32)
            dt = DT_F32
        x = np.ascontiguousarray(x)
        k = x.shape[0]
        out = np.zeros(row_bytes(act_kind, k), dtype=np.uint8)
        fn = self.L.mo_pack_q8_0 if act_kind == KIND_Q8_0 else self.L.mo_pack_q8_k
        fn(_ptr(x), dt, k, _ptr(out))
        return out

    def vec_dot(self, kind: int, w: np.ndarray, a: np.ndarray, nblocks: int) -> float:
        fn = {
            KIND_Q8_0: self.L.mo_vec_dot_q8_0_q8_0,
            KIND_Q4_0: self.L.mo_vec_dot_q4_0_q8_0,
            KIND_Q4_K: self.L.mo_vec_dot_q4_k_q8_k,
            KIND_Q5_K: self.L.mo_vec_dot_q5_k_q8_k,
            KIND_Q4_1: self.L.mo_vec_dot_q4_1_q8_0,
            KIND_Q5_0: self.L.mo_vec_dot_q5_0_q8_0,
            KIND_Q5_1: self.L.mo_vec_dot_q5_1_q8_0,
            KIND_Q2_K: self.L.mo_vec_dot_q2_k_q8_k,
            KIND_Q3_K: self.L.mo_vec_dot_q3_k_q8_k,
            KIND_Q8_1: self.L.mo_vec_dot_q8_1_q8_0,
            KIND_Q6_K: self.L.mo_vec_dot_q6_k_q8_k,
        }[kind]
        w = np.ascontiguousarray(w, dtype=np.uint8)
        a = np.ascontiguousarray(a, dtype=np.uint8)
        return float(fn(_ptr(w), _ptr(a), nblocks))

    def vec_dot_f16(self, kind: int, w: np.ndarray, a: np.ndarray, k: int) -> float:
        w = np.ascontiguousarray(w, dtype=np.uint8)
        a = np.ascontiguousarray(a, dtype=np.float16)
        nb = (k + BLOCK_VALUES[kind] - 1) // BLOCK_VALUES[kind]
        return float(self.L.mo_vec_dot_f16(kind, _ptr(w), _ptr(a), nb, k))

    # ---- matmul
    def matmul(self, kind: int, weight: np.ndarray, x: np.ndarray, M: int, bias=None, out_dtype=None,
               force_pack: bool = False, threads: int = 1) -> np.ndarray:
        weight = np.ascontiguousarray(weight, dtype=np.uint8)
        if x.dtype == np.float16:
            in_dt = DT_F16
        else:
            x = x.astype(np.float32, copy=False)
            in_dt = DT_F32
        x = np.ascontiguousarray(x)
        N, K = x.shape
        assert weight.size == M * row_bytes(kind, K), (weight.size, M, K)
        if out_dtype is None:
            out_dtype = np.float32
        out = np.zeros((N, M), dtype=out_dtype)
        out_dt = DT_F16 if out.dtype == np.float16 else DT_F32
        b = None
        if bias is not None:
            b = np.ascontiguousarray(bias, dtype=np.float32)
        st = self.L.mo_matmul_quantized(
            kind, _ptr(weight), _ptr(x), in_dt, N, K, M, _ptr(b) if b is not None else None, _ptr(out), out_dt,
            1 if force_pack else 0, threads,
        )
        if st != 0:
            raise RuntimeError(f"mo_matmul_quantized -> {st}")
        return out

    def paged_attention(self, token_meta, q, k_new, v_new, kv_k, kv_v, block_table, layer_idx: int, scale: float,
                        act_bf16: bool = False, kv_bf16: bool = False, token_count=None, kv_k_scale=None,
                        kv_v_scale=None):
        """marmot_paged_attention: kv_k / kv_v ([blocks, layers, kv heads, block size, head dim]) are updated in place;
        q / k_new / v_new are [tokens, heads, head dim] arrays (views with any strides) of float32, float16, or uint16
        holding bfloat16 bits (act_bf16 / kv_bf16); a uint8 cache is FLOAT8_E4M3 with its float32 scale tensors
        [blocks, layers, kv heads], updated in place too. Returns (status, out)."""
        args, out = paged_attention_args(token_meta, q, k_new, v_new, kv_k, kv_v, block_table, layer_idx, scale, act_bf16,
                                         kv_bf16, token_count, kv_k_scale=kv_k_scale, kv_v_scale=kv_v_scale)
        st = self.L.mo_paged_attention(C.byref(args))
        return st, out

    def rope_frequencies(self, rope: "RopeParams", head_dim: int):
        """(angular frequencies [head_dim / 2], attention scale) of marmot_rope_freq_cache_ensure."""
        freqs = np.zeros(head_dim // 2, dtype=np.float32)
        scale = C.c_float(0.0)
        st = self.L.mo_rope_frequencies(C.byref(rope), head_dim, _ptr(freqs), C.byref(scale))
        if st != 0:
            raise RuntimeError(f"mo_rope_frequencies -> {st}")
        return freqs, float(scale.value)

    def rope_rotate_row(self, row: np.ndarray, head_dim: int, position: float, freqs: np.ndarray, attn_scale: float,
                        rope_type: int) -> np.ndarray:
        out = np.ascontiguousarray(row, dtype=np.float32).copy()
        freqs = np.ascontiguousarray(freqs, dtype=np.float32)
        self.L.mo_rope_rotate_row(_ptr(out), out.shape[0], head_dim, position, _ptr(freqs), attn_scale, rope_type)
        return out

    def rope(self, x: np.ndarray, positions: np.ndarray, rope: "RopeParams", dim=None, x_row_stride=None,
             out_row_stride=None):
        """marmot_rope: the last dimension of x (float32 or float16, rank >= 2) is rotated, one position (float32,
        int32 or int64) per row; `rope.head_dim` is not used. With `dim` and row strides (in elements), x is a flat
        buffer holding positions.size rows of dim values at x_row_stride and the result a flat buffer of rows at
        out_row_stride (the gaps hold NaN). Returns (status, out)."""
        assert x.dtype in (np.float32, np.float16)
        x = np.ascontiguousarray(x)
        pos = np.ascontiguousarray(positions)
        pos_dt = {np.dtype(np.float32): DT_F32, np.dtype(np.int32): DT_I32, np.dtype(np.int64): DT_I64}[pos.dtype]
        dt = DT_F16 if x.dtype == np.float16 else DT_F32
        if dim is None:
            dim = x.shape[-1]
            rows = x.size // dim if dim else 0
            out = np.full(x.shape, np.nan, dtype=x.dtype)
            xs = os_ = dim
        else:
            rows, xs, os_ = pos.size, x_row_stride, out_row_stride
            assert x.ndim == 1 and (rows == 0 or x.size >= (rows - 1) * xs + dim)
            out = np.full(max(rows - 1, 0) * os_ + dim, np.nan, dtype=x.dtype)
        st = self.L.mo_rope(_ptr(x), dt, rows, dim, xs, os_, C.byref(rope), _ptr(pos), pos_dt, _ptr(out))
        return st, out

    def matmul_qkv(self, kind: int, wq, wk, wv, x: np.ndarray, M: int, bq=None, bk=None, bv=None, rope=None,
                   positions=None):
        """marmot_matmul_qkv with separate quantized weights; returns (q, k, v) of x's dtype (float32 or float16).
        rope: RopeParams (rotary epilogue on q and/or k) with positions: N values, float32, int32 or int64."""
        ws = [np.ascontiguousarray(w, dtype=np.uint8) for w in (wq, wk, wv)]
        if x.dtype != np.float16:
            x = x.astype(np.float32, copy=False)
        x = np.ascontiguousarray(x)
        in_dt = DT_F16 if x.dtype == np.float16 else DT_F32
        N, K = x.shape
        for w in ws:
            assert w.size == M * row_bytes(kind, K), (w.size, M, K)
        biases = [None if b is None else np.ascontiguousarray(b) for b in (bq, bk, bv)]
        given = [b for b in biases if b is not None]
        assert all(b.dtype == given[0].dtype and b.dtype in (np.float32, np.float16) for b in given)
        bias_dt = DT_F16 if given and given[0].dtype == np.float16 else DT_F32
        outs = [np.zeros((N, M), dtype=x.dtype) for _ in range(3)]
        arr = C.c_void_p * 3
        pos, pos_dt = None, 0
        if rope is not None:
            pos = np.ascontiguousarray(positions)
            pos_dt = {np.dtype(np.float32): DT_F32, np.dtype(np.int32): DT_I32, np.dtype(np.int64): DT_I64}[pos.dtype]
            assert pos.shape == (N,)
        st = self.L.mo_matmul_qkv_separate_rope(
            kind, arr(*[w.ctypes.data for w in ws]), _ptr(x), in_dt, N, K, M,
            arr(*[None if b is None else b.ctypes.data for b in biases]), bias_dt, arr(*[o.ctypes.data for o in outs]),
            C.byref(rope) if rope is not None else None, _ptr(pos) if pos is not None else None, pos_dt,
        )
        if st != 0:
            raise RuntimeError(f"mo_matmul_qkv_separate_rope -> {st}")
        return tuple(outs)

    def embedding_gather(self, kind: int, table: np.ndarray, vocab: int, dim: int, ids: np.ndarray,
                         out_dtype=np.float32, scale: float = 1.0, padding_id: int = -1, bounds_check: bool = False):
        """marmot_embedding_gather with a block-quantized table; ids int32 or int64, any shape. Raises IndexError
        (with the flat position) for an out-of-range token when bounds_check is set."""
        table = np.ascontiguousarray(table, dtype=np.uint8)
        assert table.size == vocab * row_bytes(kind, dim)
        ids = np.ascontiguousarray(ids)
        ids_dt = {np.dtype(np.int32): DT_I32, np.dtype(np.int64): DT_I64}[ids.dtype]
        out = np.full(ids.shape + (dim,), np.nan, dtype=out_dtype)
        err = C.c_size_t(0)
        st = self.L.mo_embedding_gather_quantized(
            kind, _ptr(table), vocab, dim, _ptr(ids), ids_dt, ids.size, _ptr(out),
            DT_F16 if out.dtype == np.float16 else DT_F32, scale, padding_id, 1 if bounds_check else 0, C.byref(err))
        if st == -1:
            raise IndexError(int(err.value))
        if st != 0:
            raise RuntimeError(f"mo_embedding_gather_quantized -> {st}")
        return out

    # ---- MoE
    def topk(self, x: np.ndarray, k: int):
        x = np.ascontiguousarray(x, dtype=np.float32)
        rows, cols = x.shape
        vals = np.zeros((rows, k), dtype=np.float32)
        idx = np.zeros((rows, k), dtype=np.int32)
        st = self.L.mo_topk(_ptr(x), rows, cols, k, _ptr(vals), _ptr(idx))
        if st != 0:
            raise RuntimeError(f"mo_topk -> {st}")
        return vals, idx

    def softmax_rows(self, x: np.ndarray) -> np.ndarray:
        x = np.ascontiguousarray(x, dtype=np.float32)
        out = np.zeros_like(x)
        self.L.mo_softmax_rows(_ptr(x), x.shape[0], x.shape[1], _ptr(out))
        return out

    # ---- tensor operations around the linears
    UNARY_GELU, UNARY_GELU_TANH, UNARY_SILU = 0, 1, 2

    def unary(self, op: int, x: np.ndarray) -> np.ndarray:
        """x: float32 or float16 values of any shape."""
        x = np.ascontiguousarray(x)
        assert x.dtype in (np.float32, np.float16)
        out = np.zeros_like(x)
        st = self.L.mo_unary(op, _ptr(x), DT_F32 if x.dtype == np.float32 else DT_F16, x.size, _ptr(out))
        if st != 0:
            raise RuntimeError(f"mo_unary -> {st}")
        return out

    def softmax(self, x: np.ndarray, axis: int = -1) -> np.ndarray:
        x = np.ascontiguousarray(x, dtype=np.float32)
        axis = axis % x.ndim
        outer = int(np.prod(x.shape[:axis], dtype=np.int64))
        inner = int(np.prod(x.shape[axis + 1:], dtype=np.int64))
        out = np.zeros_like(x)
        st = self.L.mo_softmax(_ptr(x), outer, x.shape[axis], inner, _ptr(out))
        if st != 0:
            raise RuntimeError(f"mo_softmax -> {st}")
        return out

    def softmax_typed(self, x: np.ndarray, dtype: int, axis: int = -1) -> np.ndarray:
        """x: float32 values (dtype FLOAT32) or uint16 bit patterns of FLOAT16 (1) / BFLOAT16 (2); the result likewise."""
        x = np.ascontiguousarray(x)
        assert x.dtype == (np.float32 if dtype == DT_F32 else np.uint16)
        axis = axis % x.ndim
        outer = int(np.prod(x.shape[:axis], dtype=np.int64))
        inner = int(np.prod(x.shape[axis + 1:], dtype=np.int64))
        out = np.zeros_like(x)
        st = self.L.mo_softmax_typed(dtype, _ptr(x), outer, x.shape[axis], inner, _ptr(out))
        if st != 0:
            raise RuntimeError(f"mo_softmax_typed -> {st}")
        return out

    def convert(self, src: np.ndarray, src_dtype: int, dst_dtype: int) -> np.ndarray:
        """src: float32 values, or uint16 bit patterns for FLOAT16 (1) / BFLOAT16 (2) sources; the result likewise."""
        src = np.ascontiguousarray(src)
        assert src.dtype == (np.float32 if src_dtype == DT_F32 else np.uint16)
        out = np.zeros(src.shape, dtype=np.float32 if dst_dtype == DT_F32 else np.uint16)
        st = self.L.mo_convert(_ptr(out), dst_dtype, _ptr(src), src_dtype, src.size)
        if st != 0:
            raise RuntimeError(f"mo_convert -> {st}")
        return out

    def gather_rows(self, x: np.ndarray, idx: np.ndarray) -> np.ndarray:
        """x: 2-D array whose rows may be strided (unit column stride); idx: int32 or uint32, 1-D."""
        assert x.ndim == 2 and idx.ndim == 1 and (x.shape[1] <= 1 or x.strides[1] == x.itemsize)
        idx = np.ascontiguousarray(idx)
        assert idx.dtype in (np.int32, np.uint32)
        out = np.zeros((idx.shape[0], x.shape[1]), dtype=x.dtype)
        bad = C.c_size_t(0)
        st = self.L.mo_gather_rows(x.ctypes.data, x.shape[0], x.shape[1], x.itemsize, x.strides[0] // x.itemsize,
                                   _ptr(idx), 1 if idx.dtype == np.int32 else 0, 1, idx.shape[0], _ptr(out),
                                   x.shape[1], C.byref(bad))
        if st != 0:
            raise IndexError(int(bad.value))
        return out

    def slice(self, x: np.ndarray, starts, sizes) -> np.ndarray:
        x = np.ascontiguousarray(x)
        out = np.zeros(tuple(sizes), dtype=x.dtype)
        n = x.ndim
        arr = lambda v: (C.c_size_t * n)(*[int(i) for i in v])
        st = self.L.mo_slice(_ptr(x), _ptr(out), x.itemsize, n, arr(x.shape), arr(out.shape), arr(starts), arr(sizes))
        if st != 0:
            raise RuntimeError(f"mo_slice -> {st}")
        return out

    def rms_norm(self, x, weight=None, residual=None, eps: float = 1e-5, weight_offset: float = 0.0) -> np.ndarray:
        x = np.ascontiguousarray(x, dtype=np.float32)
        rows, cols = x.shape
        res = None if residual is None else np.ascontiguousarray(residual, dtype=np.float32)
        w = None if weight is None else np.ascontiguousarray(weight, dtype=np.float32)
        out = np.zeros_like(x)
        st = self.L.mo_rms_norm(_ptr(x), _ptr(res) if res is not None else None, _ptr(w) if w is not None else None,
                                weight_offset, eps, rows, cols, _ptr(out))
        if st != 0:
            raise RuntimeError(f"mo_rms_norm -> {st}")
        return out

    def glu(self, gate, up, geglu: bool = False) -> np.ndarray:
        gate = np.ascontiguousarray(gate, dtype=np.float32)
        up = np.ascontiguousarray(up, dtype=np.float32)
        out = np.zeros_like(gate)
        self.L.mo_glu(_ptr(gate), _ptr(up), gate.size, 1 if geglu else 0, _ptr(out))
        return out

    def moe_glu(self, gate: np.ndarray, up: np.ndarray, ffn_type: int = 0) -> np.ndarray:
        """act(gate) * up element by element, as the expert body forms it between the projections."""
        gate = np.ascontiguousarray(gate, dtype=np.float32)
        up = np.ascontiguousarray(up, dtype=np.float32)
        assert gate.shape == up.shape
        out = np.zeros_like(gate)
        st = self.L.mo_moe_glu(_ptr(gate), _ptr(up), gate.size, ffn_type, _ptr(out))
        if st != 0:
            raise RuntimeError(f"mo_moe_glu -> {st}")
        return out

    def moe_experts(self, hidden, gate, up, down, topk_ids, topk_weights, F: int, E: int, kind_gate_up: int,
                    kind_down: int, weights_scale: float = 1.0, policy: int = 1, ffn_type: int = 0,
                    force_grouped: bool = False, threads: int = 1) -> np.ndarray:
        hidden = np.ascontiguousarray(hidden, dtype=np.float32)
        T, H = hidden.shape
        ids = np.ascontiguousarray(topk_ids, dtype=np.int32)
        w = np.ascontiguousarray(topk_weights, dtype=np.float32)
        kpt = ids.shape[1]
        gate = np.ascontiguousarray(gate, dtype=np.uint8)
        up = np.ascontiguousarray(up, dtype=np.uint8)
        down = np.ascontiguousarray(down, dtype=np.uint8)
        assert gate.size == E * F * row_bytes(kind_gate_up, H)
        assert down.size == E * H * row_bytes(kind_down, F)
        out = np.zeros((T, H), dtype=np.float32)
        st = self.L.mo_moe_experts(
            _ptr(hidden), T, H, F, E, kpt, kind_gate_up, kind_down, _ptr(gate), _ptr(up), _ptr(down), _ptr(ids),
            _ptr(w), weights_scale, policy, ffn_type, 1 if force_grouped else 0, threads, _ptr(out),
        )
        if st != 0:
            raise RuntimeError(f"mo_moe_experts -> {st}")
        return out

    def row_grain(self, rows: int, cols: int, threads: int) -> int:
        return int(self.L.mo_row_grain(rows, cols, threads))


class _QuantTraits(C.Structure):
    # include/marmot/quant_traits.h:30-43
    _fields_ = [
        ("kind", C.c_int),
        ("name", C.c_char_p),
        ("block_size", C.c_uint32),
        ("block_bytes", C.c_uint32),
        ("weight_bits", C.c_uint32),
        ("has_zero_point", C.c_bool),
        ("requires_calibration", C.c_bool),
        ("layout", C.c_int),
        ("compute_params", C.c_void_p),
        ("quantize_block", C.CFUNCTYPE(C.c_int, C.c_void_p, C.c_uint32, C.c_void_p, C.c_void_p)),
        ("dequantize_block", C.CFUNCTYPE(C.c_int, C.c_void_p, C.c_uint32, C.c_void_p, C.c_void_p)),
        ("vec_dot_block", C.c_void_p),
    ]


class RefLib:
    """The reference's own leaf arithmetic (scalar build), where oracle/_ref was built."""

    @staticmethod
    def available() -> bool:
        return os.path.exists(REF_SO)

    def __init__(self):
        L = C.CDLL(REF_SO)
        self.L = L
        L.marmot_get_quant_traits.restype = C.POINTER(_QuantTraits)
        L.marmot_get_quant_traits.argtypes = [C.c_int]
        for n in ("cpu_matmul_quant_pack_q8_0_f32", "cpu_matmul_quant_pack_q8_k_f32", "cpu_matmul_quant_pack_q8_0_f16",
                  "cpu_matmul_quant_pack_q8_k_f16"):
            f = getattr(L, n)
            f.restype = None
            f.argtypes = [C.c_void_p, C.c_size_t, C.c_size_t, C.c_size_t, C.c_size_t, C.c_size_t, C.c_void_p]
        for n in ("q8_0_q8_0", "q4_0_q8_0", "q4_k_q8_k", "q5_k_q8_k", "q6_k_q8_k", "q4_1_q8_0", "q5_0_q8_0",
                  "q5_1_q8_0", "q2_k_q8_k", "q3_k_q8_k", "q8_1_q8_0"):
            f = getattr(L, f"cpu_vec_dot_{n}_scalar")
            f.restype = C.c_float
            f.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]
        for n in ("q8_0", "q4_0", "q4_k", "q5_k", "q6_k", "q4_1", "q5_0", "q5_1", "q2_k", "q3_k", "q8_1"):
            f = getattr(L, f"cpu_vec_dot_{n}_f16_scalar")
            f.restype = C.c_float
            f.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t, C.c_size_t]

    def _traits(self, kind: int) -> _QuantTraits:
        p = self.L.marmot_get_quant_traits(kind)
        if not p:
            raise RuntimeError(f"reference has no traits for kind {kind}")
        return p.contents

    def quantize(self, kind: int, x: np.ndarray) -> np.ndarray:
        x = np.ascontiguousarray(x, dtype=np.float32)
        if x.ndim == 1:
            x = x[None, :]
        rows, k = x.shape
        t = self._traits(kind)
        bv, bb = t.block_size, t.block_bytes
        nb = (k + bv - 1) // bv
        out = np.zeros((rows, nb * bb), dtype=np.uint8)
        for r in range(rows):
            for b in range(nb):
                elems = min(bv, k - b * bv)
                src = x[r, b * bv:b * bv + elems]
                src = np.ascontiguousarray(src)
                st = t.quantize_block(_ptr(src), elems, C.c_void_p(out[r].ctypes.data + b * bb), None)
                assert st == 0
        return out

    def dequantize(self, kind: int, blocks: np.ndarray, k: int) -> np.ndarray:
        blocks = np.ascontiguousarray(blocks, dtype=np.uint8)
        if blocks.ndim == 1:
            blocks = blocks[None, :]
        rows = blocks.shape[0]
        t = self._traits(kind)
        bv, bb = t.block_size, t.block_bytes
        nb = (k + bv - 1) // bv
        out = np.zeros((rows, k), dtype=np.float32)
        for r in range(rows):
            for b in range(nb):
                elems = min(bv, k - b * bv)
                st = t.dequantize_block(C.c_void_p(blocks[r].ctypes.data + b * bb), elems,
                                        C.c_void_p(out[r].ctypes.data + 4 * b * bv), None)
                assert st == 0
        return out

    def pack(self, act_kind: int, x: np.ndarray) -> np.ndarray:
        f16 = x.dtype == np.float16
        x = np.ascontiguousarray(x if f16 else x.astype(np.float32))
        k = x.shape[0]
        bv = BLOCK_VALUES[act_kind]
        nb = (k + bv - 1) // bv
        out = np.zeros(nb * BLOCK_BYTES[act_kind], dtype=np.uint8)
        name = f"cpu_matmul_quant_pack_{'q8_0' if act_kind == KIND_Q8_0 else 'q8_k'}_{'f16' if f16 else 'f32'}"
        getattr(self.L, name)(_ptr(x), 1, k, 0, k, nb, _ptr(out))
        return out

    def vec_dot(self, kind: int, w: np.ndarray, a: np.ndarray, nblocks: int) -> float:
        name = {KIND_Q8_0: "q8_0_q8_0", KIND_Q4_0: "q4_0_q8_0", KIND_Q4_K: "q4_k_q8_k", KIND_Q5_K: "q5_k_q8_k",
                KIND_Q6_K: "q6_k_q8_k", KIND_Q4_1: "q4_1_q8_0", KIND_Q5_0: "q5_0_q8_0", KIND_Q5_1: "q5_1_q8_0",
                KIND_Q2_K: "q2_k_q8_k", KIND_Q3_K: "q3_k_q8_k", KIND_Q8_1: "q8_1_q8_0"}[kind]
        w = np.ascontiguousarray(w, dtype=np.uint8)
        a = np.ascontiguousarray(a, dtype=np.uint8)
        return float(getattr(self.L, f"cpu_vec_dot_{name}_scalar")(_ptr(w), _ptr(a), nblocks))

    def vec_dot_f16(self, kind: int, w: np.ndarray, a: np.ndarray, k: int) -> float:
        name = {KIND_Q8_0: "q8_0", KIND_Q4_0: "q4_0", KIND_Q4_K: "q4_k", KIND_Q5_K: "q5_k", KIND_Q6_K: "q6_k",
                KIND_Q4_1: "q4_1", KIND_Q5_0: "q5_0", KIND_Q5_1: "q5_1", KIND_Q2_K: "q2_k", KIND_Q3_K: "q3_k",
                KIND_Q8_1: "q8_1"}[kind]
        w = np.ascontiguousarray(w, dtype=np.uint8)
        a = np.ascontiguousarray(a, dtype=np.float16)
        nb = (k + BLOCK_VALUES[kind] - 1) // BLOCK_VALUES[kind]
        return float(getattr(self.L, f"cpu_vec_dot_{name}_f16_scalar")(_ptr(w), _ptr(a), 1, nb, k))
