"""Host-side mirror of the reference's operator interface for the quantized matmul path.

Names and argument meaning follow the reference's C API: ``linear(input[N,K], weight[M,K]) -> out[N,M]``
(include/marmot/ops/matmul.h:11), ``dequantize`` (ops/quantization.h), ``topk`` / ``moe_experts``
(ops/neural.h:67,85). Everything runs through the C ABI in include/marmot_hip.h.
"""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import capi
from .capi import DT_F16, DT_F32, KIND_Q8_0, KIND_Q8_K, check, load_library

_BV = {1: 32, 2: 32, 3: 32, 4: 32, 5: 32, 6: 32, 7: 256, 8: 256, 9: 256, 10: 256, 11: 256, 12: 256}
_BB = {1: 18, 2: 20, 3: 22, 4: 24, 5: 34, 6: 36, 7: 84, 8: 110, 9: 144, 10: 176, 11: 210, 12: 292}


def block_values(kind: int) -> int:
    return _BV[kind]


def block_bytes(kind: int) -> int:
    return _BB[kind]


def row_bytes(kind: int, k: int) -> int:
    return ((k + _BV[kind] - 1) // _BV[kind]) * _BB[kind]


def _np_dtype_id(dt) -> int:
    dt = np.dtype(dt)
    if dt == np.float32:
        return DT_F32
    if dt == np.float16:
        return DT_F16
    raise TypeError(f"unsupported dtype {dt}")


class DeviceBuffer:
    """A device allocation made through marmot_hip_alloc."""

    def __init__(self, backend: "HipBackend", nbytes: int):
        self.backend = backend
        self.nbytes = int(nbytes)
        p = C.c_void_p()
        check(backend.lib.marmot_hip_alloc(backend.dev, max(self.nbytes, 1), C.byref(p)))
        self.ptr = p.value

    def upload(self, arr: np.ndarray, offset: int = 0):
        arr = np.ascontiguousarray(arr)
        assert offset + arr.nbytes <= self.nbytes
        if arr.nbytes:
            check(self.backend.lib.marmot_hip_memcpy_to_device(
                self.backend.dev, C.c_void_p(self.ptr + offset), arr.ctypes.data_as(C.c_void_p), arr.nbytes))
        return self

    def download(self, dtype, shape, offset: int = 0) -> np.ndarray:
        out = np.empty(shape, dtype=dtype)
        assert offset + out.nbytes <= self.nbytes
        if out.nbytes:
            check(self.backend.lib.marmot_hip_memcpy_from_device(
                self.backend.dev, out.ctypes.data_as(C.c_void_p), C.c_void_p(self.ptr + offset), out.nbytes))
        return out

    def free(self):
        if self.ptr:
            self.backend.lib.marmot_hip_free(self.backend.dev, C.c_void_p(self.ptr))
            self.ptr = 0

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class HipBackend:
    """One marmot_hip_device_t (one GPU, one stream)."""

    def __init__(self, device_index: int = 0):
        self.lib = load_library()
        dev = C.c_void_p()
        check(self.lib.marmot_hip_device_create(device_index, C.byref(dev)))
        self.dev = dev

    def close(self):
        if self.dev:
            self.lib.marmot_hip_device_destroy(self.dev)
            self.dev = None

    # ---- plumbing
    def alloc(self, nbytes: int) -> DeviceBuffer:
        return DeviceBuffer(self, nbytes)

    def to_device(self, arr: np.ndarray) -> DeviceBuffer:
        arr = np.ascontiguousarray(arr)
        return DeviceBuffer(self, arr.nbytes).upload(arr)

    def copy_d(self, d_dst, d_src, nbytes: int):
        check(self.lib.marmot_hip_memcpy_device(self.dev, C.c_void_p(d_dst.ptr), C.c_void_p(d_src.ptr), nbytes))

    def read_probe_d(self, d_src, nbytes: int, d_sink, offset: int = 0):
        """One launch that only reads nbytes at d_src + offset (bandwidth calibration)."""
        check(self.lib.marmot_hip_read_probe(self.dev, C.c_void_p(d_src.ptr + offset), nbytes, C.c_void_p(d_sink.ptr)))

    def synchronize(self):
        check(self.lib.marmot_hip_synchronize(self.dev))

    def caps(self) -> dict:
        c = capi.Caps()
        check(self.lib.marmot_hip_get_caps(self.dev, C.byref(c)))
        return {f: (getattr(c, f).decode() if isinstance(getattr(c, f), bytes) else getattr(c, f))
                for f, _ in capi.Caps._fields_}

    def allocator_usage(self):
        cur, peak, n = C.c_size_t(), C.c_size_t(), C.c_size_t()
        check(self.lib.marmot_hip_allocator_usage(self.dev, C.byref(cur), C.byref(peak), C.byref(n)))
        return cur.value, peak.value, n.value

    def last_route(self) -> str:
        return self.lib.marmot_hip_last_route().decode()

    def graph_capture(self, fn):
        """Records everything fn() enqueues into a HIP graph and returns the executable graph handle."""
        check(self.lib.marmot_hip_graph_begin_capture(self.dev))
        g = C.c_void_p()
        try:
            fn()
        finally:
            st = self.lib.marmot_hip_graph_end_capture(self.dev, C.byref(g))
        check(st)
        return g

    def branches(self, *fns):
        """Runs fns[0](), fns[1](), ... as the branches of one section: what they enqueue may overlap on the device, and
        whatever is enqueued afterwards starts after all of them (marmot_hip_branch_begin / _next / _join). The caller
        guarantees that no branch touches what another one writes. At most MARMOT_HIP_MAX_BRANCHES functions."""
        check(self.lib.marmot_hip_branch_begin(self.dev))
        try:
            for i, fn in enumerate(fns):
                if i > 0:
                    check(self.lib.marmot_hip_branch_next(self.dev))
                fn()
        finally:
            st = self.lib.marmot_hip_branch_join(self.dev)
        check(st)

    def graph_max_nodes(self) -> int:
        """Most nodes one captured graph may hold (graph_capture raises beyond it)."""
        return int(self.lib.marmot_hip_graph_max_nodes())

    def graph_last_capture_nodes(self) -> int:
        return int(self.lib.marmot_hip_graph_last_capture_nodes(self.dev))

    def graph_launch(self, g):
        check(self.lib.marmot_hip_graph_launch(self.dev, g))

    def graph_destroy(self, g):
        self.lib.marmot_hip_graph_destroy(self.dev, g)

    def event(self):
        e = C.c_void_p()
        check(self.lib.marmot_hip_event_create(self.dev, C.byref(e)))
        return e

    def event_destroy(self, e):
        self.lib.marmot_hip_event_destroy(self.dev, e)

    def record(self, e):
        check(self.lib.marmot_hip_event_record(self.dev, e))

    def elapsed_ms(self, a, b) -> float:
        ms = C.c_float()
        check(self.lib.marmot_hip_event_elapsed_ms(self.dev, a, b, C.byref(ms)))
        return ms.value

    # ---- device-pointer level ops (what bench.py times)
    def dequantize_d(self, kind: int, d_blocks: DeviceBuffer, rows: int, k: int, d_out: DeviceBuffer):
        check(self.lib.marmot_hip_dequantize(self.dev, kind, C.c_void_p(d_blocks.ptr), rows, k, C.c_void_p(d_out.ptr)))

    def linear_d(self, kind: int, d_weight, d_input, in_dtype: int, N: int, K: int, M: int, d_out, out_dtype: int,
                 d_bias=None, bias_dtype: int = DT_F32, flags: int = 0, weight_offset: int = 0):
        check(self.lib.marmot_hip_matmul_quantized(
            self.dev, kind, C.c_void_p(d_weight.ptr + weight_offset), C.c_void_p(d_input.ptr), in_dtype, N, K, M,
            C.c_void_p(d_bias.ptr) if d_bias is not None else None, bias_dtype, C.c_void_p(d_out.ptr), out_dtype,
            flags))

    def linear_noalloc_d(self, kind: int, d_weight, d_input, in_dtype: int, N: int, K: int, M: int, d_out,
                         out_dtype: int, d_bias=None, bias_dtype: int = DT_F32, flags: int = 0):
        """marmot_hip_matmul_quantized_noalloc: the same linear with its scratch in the library's static device array."""
        check(self.lib.marmot_hip_matmul_quantized_noalloc(
            self.dev, kind, C.c_void_p(d_weight.ptr), C.c_void_p(d_input.ptr), in_dtype, N, K, M,
            C.c_void_p(d_bias.ptr) if d_bias is not None else None, bias_dtype, C.c_void_p(d_out.ptr), out_dtype,
            flags))

    def linear_qkv_d(self, kind: int, d_wq, d_wk, d_wv, d_input, dtype: int, N: int, K: int, M: int, d_out_q, d_out_k,
                     d_out_v, d_bq=None, d_bk=None, d_bv=None, weight_offset: int = 0):
        """marmot_hip_matmul_qkv_quantized on device buffers; weight_offset applies to the three weights alike."""
        opt = lambda b: C.c_void_p(b.ptr) if b is not None else None
        check(self.lib.marmot_hip_matmul_qkv_quantized(
            self.dev, kind, C.c_void_p(d_wq.ptr + weight_offset), C.c_void_p(d_wk.ptr + weight_offset),
            C.c_void_p(d_wv.ptr + weight_offset), C.c_void_p(d_input.ptr), dtype, N, K, M, opt(d_bq), opt(d_bk),
            opt(d_bv), dtype, C.c_void_p(d_out_q.ptr), C.c_void_p(d_out_k.ptr), C.c_void_p(d_out_v.ptr), dtype))

    def packed_activation_bytes(self, kind: int, N: int, K: int) -> int:
        return int(self.lib.marmot_hip_packed_activation_bytes(kind, N, K))

    def pack_activations_d(self, kind: int, d_input, in_dtype: int, N: int, K: int, d_packed):
        check(self.lib.marmot_hip_pack_activations(self.dev, kind, C.c_void_p(d_input.ptr), in_dtype, N, K,
                                                   C.c_void_p(d_packed.ptr)))

    def linear_prepacked_d(self, kind: int, d_weight, d_packed, N: int, K: int, M: int, d_out, out_dtype: int = DT_F32,
                           d_bias=None, bias_dtype: int = DT_F32, weight_offset: int = 0):
        check(self.lib.marmot_hip_matmul_prepacked(
            self.dev, kind, C.c_void_p(d_weight.ptr + weight_offset), C.c_void_p(d_packed.ptr), N, K, M,
            C.c_void_p(d_bias.ptr) if d_bias is not None else None, bias_dtype, C.c_void_p(d_out.ptr), out_dtype))

    # ---- numpy level ops (what the parity tests call)
    def dequantize(self, kind: int, blocks: np.ndarray, k: int) -> np.ndarray:
        blocks = np.ascontiguousarray(blocks, dtype=np.uint8)
        if blocks.ndim == 1:
            blocks = blocks[None, :]
        rows = blocks.shape[0]
        if blocks.shape[1] != row_bytes(kind, k):
            raise ValueError("blocks do not match rows x row_bytes(kind, k)")
        d_in = self.to_device(blocks)
        d_out = self.alloc(rows * k * 4)
        self.dequantize_d(kind, d_in, rows, k, d_out)
        out = d_out.download(np.float32, (rows, k))
        d_in.free()
        d_out.free()
        return out

    def quantize_activations(self, act_kind: int, x: np.ndarray) -> np.ndarray:
        x = np.ascontiguousarray(x)
        if x.ndim == 1:
            x = x[None, :]
        rows, k = x.shape
        d_x = self.to_device(x)
        nbytes = rows * row_bytes(act_kind, k)
        d_out = self.alloc(nbytes)
        check(self.lib.marmot_hip_quantize_activations(self.dev, act_kind, C.c_void_p(d_x.ptr), _np_dtype_id(x.dtype),
                                                       rows, k, C.c_void_p(d_out.ptr)))
        out = d_out.download(np.uint8, (rows, row_bytes(act_kind, k)))
        d_x.free()
        d_out.free()
        return out

    def quantize_weights(self, kind: int, x: np.ndarray) -> np.ndarray:
        """fp32 rows -> Q4_K / Q5_K / Q6_K blocks on the device (the reference's K-quant quantizers, byte for byte);
        returns [rows, row_bytes] uint8."""
        x = np.ascontiguousarray(x, dtype=np.float32)
        if x.ndim == 1:
            x = x[None, :]
        rows, k = x.shape
        d_x = self.to_device(x)
        d_out = self.alloc(max(1, rows * row_bytes(kind, k)))
        try:
            check(self.lib.marmot_hip_quantize_weights(self.dev, kind, C.c_void_p(d_x.ptr), rows, k,
                                                       C.c_void_p(d_out.ptr)))
            return d_out.download(np.uint8, (rows, row_bytes(kind, k)))
        finally:
            d_x.free()
            d_out.free()

    def linear(self, x: np.ndarray, weight: np.ndarray, kind: int, M: int, bias: np.ndarray | None = None,
               out_dtype=np.float32, force_pack: bool = False) -> np.ndarray:
        """marmot_linear(input[N,K], weight[M,K] as GGUF blocks) -> out[N,M]."""
        x = np.ascontiguousarray(x)
        N, K = x.shape
        weight = np.ascontiguousarray(weight, dtype=np.uint8)
        if weight.size != M * row_bytes(kind, K):
            raise ValueError("weight bytes do not match M x row_bytes(kind, K)")
        d_w = self.to_device(weight)
        d_x = self.to_device(x)
        out_dtype = np.dtype(out_dtype)
        d_out = self.alloc(max(N * M * out_dtype.itemsize, 4))
        d_b = self.to_device(bias) if bias is not None else None
        try:
            self.linear_d(kind, d_w, d_x, _np_dtype_id(x.dtype), N, K, M, d_out, _np_dtype_id(out_dtype), d_b,
                          _np_dtype_id(bias.dtype) if bias is not None else DT_F32,
                          capi.FLAG_FORCE_PACK if force_pack else 0)
            return d_out.download(out_dtype, (N, M))
        finally:
            for b in (d_w, d_x, d_out, d_b):
                if b is not None:
                    b.free()

    def linear_dual(self, x: np.ndarray, weight_a: np.ndarray, weight_b: np.ndarray, kind: int, M: int,
                    out_dtype=np.float32, force_pack: bool = False):
        x = np.ascontiguousarray(x)
        N, K = x.shape
        d_a = self.to_device(np.ascontiguousarray(weight_a, dtype=np.uint8))
        d_b = self.to_device(np.ascontiguousarray(weight_b, dtype=np.uint8))
        d_x = self.to_device(x)
        out_dtype = np.dtype(out_dtype)
        d_oa = self.alloc(N * M * out_dtype.itemsize)
        d_ob = self.alloc(N * M * out_dtype.itemsize)
        try:
            check(self.lib.marmot_hip_matmul_quantized_dual(
                self.dev, kind, C.c_void_p(d_a.ptr), C.c_void_p(d_b.ptr), C.c_void_p(d_x.ptr), _np_dtype_id(x.dtype),
                N, K, M, C.c_void_p(d_oa.ptr), C.c_void_p(d_ob.ptr), _np_dtype_id(out_dtype),
                capi.FLAG_FORCE_PACK if force_pack else 0))
            return d_oa.download(out_dtype, (N, M)), d_ob.download(out_dtype, (N, M))
        finally:
            for b in (d_a, d_b, d_x, d_oa, d_ob):
                b.free()

    def rope_frequencies(self, M: int, head_dim: int = 0, theta: float = 10000.0, scaling_type: int = 0,
                         freq_scale: float = 1.0, ext_factor: float = 0.0, attn_factor: float = 1.0,
                         beta_fast: float = 32.0, beta_slow: float = 1.0, orig_ctx_len: int = 0):
        """(frequencies [head_dim/2] float32, attention scale, resolved head_dim) for marmot_rope_params_t fields
        (defaults of marmot_rope_params_default, include/marmot/ops/matmul.h:45-61)."""
        freqs = np.zeros(max(1, M // 2), dtype=np.float32)
        scale, hd = C.c_float(0.0), C.c_uint32(0)
        check(self.lib.marmot_hip_rope_frequencies(scaling_type, theta, freq_scale, ext_factor, attn_factor, beta_fast,
                                                   beta_slow, orig_ctx_len, head_dim, M, freqs.ctypes.data,
                                                   C.byref(scale), C.byref(hd)))
        return freqs[: hd.value // 2].copy(), float(scale.value), int(hd.value)

    def linear_qkv(self, x: np.ndarray, wq: np.ndarray, wk: np.ndarray, wv: np.ndarray, kind: int, M: int,
                   bq=None, bk=None, bv=None, rope: dict | None = None, positions=None):
        """marmot_matmul_qkv with separate quantized weights of one shape [M, K] (include/marmot/ops/matmul.h:74-95,
        CPU implementation src/backends/cpu/ops/matmul/qkv/matmul_qkv.c:749-947): returns (q, k, v), each [N, M] of
        the input dtype; biases are optional per projection and must share one dtype (float32 or float16).
        rope: keyword arguments of rope_frequencies plus rope_type, apply_to_q, apply_to_k (the rotary epilogue), with
        positions: N values of float32, int32 or int64."""
        x = np.ascontiguousarray(x)
        N, K = x.shape
        d_w = [self.to_device(np.ascontiguousarray(w, dtype=np.uint8)) for w in (wq, wk, wv)]
        d_x = self.to_device(x)
        biases = [None if b is None else np.ascontiguousarray(b) for b in (bq, bk, bv)]
        given = [b for b in biases if b is not None]
        if any(b.dtype != given[0].dtype for b in given):
            raise ValueError("q/k/v biases must share one dtype")
        d_b = [None if b is None else self.to_device(b) for b in biases]
        out_dtype = np.dtype(x.dtype)
        d_o = [self.alloc(N * M * out_dtype.itemsize) for _ in range(3)]
        extra = []
        rope_arg = None
        if rope is not None:
            kw = dict(rope)
            rope_type = kw.pop("rope_type", 0)
            aq, ak = kw.pop("apply_to_q", True), kw.pop("apply_to_k", True)
            freqs, scale, hd = self.rope_frequencies(M, **kw)
            pos = np.ascontiguousarray(positions)
            pos_dt = {np.dtype(np.float32): capi.DT_F32, np.dtype(np.int32): capi.DT_I32,
                      np.dtype(np.int64): capi.DT_I64}[pos.dtype]
            extra = [self.to_device(pos), self.to_device(freqs)]
            rope_arg = capi.Rope(extra[0].ptr, pos_dt, extra[1].ptr, scale, hd, rope_type, int(aq), int(ak))
        try:
            check(self.lib.marmot_hip_matmul_qkv_rope_quantized(
                self.dev, kind, *[C.c_void_p(w.ptr) for w in d_w], C.c_void_p(d_x.ptr), _np_dtype_id(x.dtype), N, K, M,
                *[C.c_void_p(b.ptr if b is not None else None) for b in d_b],
                _np_dtype_id(given[0].dtype) if given else 0,
                *[C.c_void_p(o.ptr) for o in d_o], _np_dtype_id(out_dtype),
                C.byref(rope_arg) if rope_arg is not None else None))
            return tuple(o.download(out_dtype, (N, M)) for o in d_o)
        finally:
            for b in d_w + [d_x] + [b for b in d_b if b is not None] + d_o + extra:
                b.free()

    def embedding_gather(self, kind: int, table: np.ndarray, vocab: int, dim: int, ids: np.ndarray,
                         out_dtype=np.float32, scale: float = 1.0, padding_id: int = -1, bounds_check: bool = False):
        """marmot_embedding_gather with a block-quantized table [vocab, dim] (include/marmot/ops_types.h:160-170,
        src/backends/cpu/ops/embedding/scalar/embedding_scalar.c): ids int32 or int64 of any shape -> ids.shape + (dim,)
        of out_dtype (float32 or float16)."""
        ids = np.ascontiguousarray(ids)
        ids_dt = {np.dtype(np.int32): capi.DT_I32, np.dtype(np.int64): capi.DT_I64}[ids.dtype]
        out_dtype = np.dtype(out_dtype)
        d_t = self.to_device(np.ascontiguousarray(table, dtype=np.uint8))
        d_i = self.to_device(ids)
        d_o = self.alloc(max(1, ids.size * dim * out_dtype.itemsize))
        try:
            check(self.lib.marmot_hip_embedding_gather_quantized(
                self.dev, kind, C.c_void_p(d_t.ptr), vocab, dim, C.c_void_p(d_i.ptr), ids_dt, ids.size,
                C.c_void_p(d_o.ptr), _np_dtype_id(out_dtype), scale, padding_id, 1 if bounds_check else 0))
            return d_o.download(out_dtype, ids.shape + (dim,))
        finally:
            for b in (d_t, d_i, d_o):
                b.free()

    def topk(self, x: np.ndarray, k: int):
        x = np.ascontiguousarray(x, dtype=np.float32)
        rows, cols = x.shape
        d_x = self.to_device(x)
        d_v = self.alloc(rows * k * 4)
        d_i = self.alloc(rows * k * 4)
        try:
            check(self.lib.marmot_hip_topk(self.dev, C.c_void_p(d_x.ptr), rows, cols, k, C.c_void_p(d_v.ptr),
                                           C.c_void_p(d_i.ptr)))
            return d_v.download(np.float32, (rows, k)), d_i.download(np.int32, (rows, k))
        finally:
            for b in (d_x, d_v, d_i):
                b.free()

    def softmax_rows(self, x: np.ndarray) -> np.ndarray:
        x = np.ascontiguousarray(x, dtype=np.float32)
        rows, k = x.shape
        d_x = self.to_device(x)
        d_o = self.alloc(rows * k * 4)
        try:
            check(self.lib.marmot_hip_softmax_rows(self.dev, C.c_void_p(d_x.ptr), rows, k, C.c_void_p(d_o.ptr)))
            return d_o.download(np.float32, (rows, k))
        finally:
            d_x.free()
            d_o.free()

    def moe_experts_d(self, d_hidden, T: int, H: int, F: int, E: int, k_per_token: int, kind_gate_up: int,
                      kind_down: int, d_gate, d_up, d_down, d_ids, d_weights, d_out, weights_scale: float = 1.0,
                      policy: int = 1, ffn_type: int = 0, gate_offset: int = 0, up_offset: int = 0,
                      down_offset: int = 0):
        """Device-pointer form of moe_experts (everything already resident; the offsets select one of several
        expert-stack copies inside the weight buffers)."""
        check(self.lib.marmot_hip_moe_experts(
            self.dev, C.c_void_p(d_hidden.ptr), T, H, F, E, k_per_token, kind_gate_up, kind_down,
            C.c_void_p(d_gate.ptr + gate_offset), C.c_void_p(d_up.ptr + up_offset),
            C.c_void_p(d_down.ptr + down_offset), C.c_void_p(d_ids.ptr), C.c_void_p(d_weights.ptr), weights_scale,
            policy, ffn_type, C.c_void_p(d_out.ptr)))

    # ---- ops between the linears (host-array conveniences over the device-pointer ABI)
    def rms_norm(self, x: np.ndarray, weight=None, residual=None, eps: float = 1e-5, weight_offset: float = 0.0,
                 pack_for_kind: int = 0, want_f32: bool = True):
        """Rows of x normalized; with pack_for_kind also (or only) as packed activations: returns out, or
        (out or None, packed uint8 image)."""
        x = np.ascontiguousarray(x, dtype=np.float32)
        rows, cols = x.shape
        bufs = [self.to_device(x)]
        d_res = d_w = None
        if residual is not None:
            d_res = self.to_device(np.ascontiguousarray(residual, dtype=np.float32))
            bufs.append(d_res)
        if weight is not None:
            d_w = self.to_device(np.ascontiguousarray(weight, dtype=np.float32))
            bufs.append(d_w)
        d_out = self.alloc(rows * cols * 4) if want_f32 else None
        d_packed = self.alloc(self.packed_activation_bytes(pack_for_kind, rows, cols)) if pack_for_kind else None
        bufs += [b for b in (d_out, d_packed) if b is not None]
        opt = lambda b: C.c_void_p(b.ptr) if b is not None else None
        try:
            if pack_for_kind:
                check(self.lib.marmot_hip_rms_norm_pack(self.dev, C.c_void_p(bufs[0].ptr), opt(d_res), opt(d_w),
                                                        weight_offset, eps, rows, cols, pack_for_kind, opt(d_out),
                                                        C.c_void_p(d_packed.ptr)))
                out = d_out.download(np.float32, (rows, cols)) if want_f32 else None
                return out, d_packed.download(np.uint8, (d_packed.nbytes,))
            check(self.lib.marmot_hip_rms_norm(self.dev, C.c_void_p(bufs[0].ptr), opt(d_res), opt(d_w), weight_offset,
                                               eps, rows, cols, C.c_void_p(d_out.ptr)))
            return d_out.download(np.float32, (rows, cols))
        finally:
            for b in bufs:
                b.free()

    def glu(self, gate: np.ndarray, up: np.ndarray, ffn_type: int = 0) -> np.ndarray:
        gate = np.ascontiguousarray(gate, dtype=np.float32)
        up = np.ascontiguousarray(up, dtype=np.float32)
        rows, cols = gate.shape
        bufs = [self.to_device(gate), self.to_device(up), self.alloc(rows * cols * 4)]
        try:
            check(self.lib.marmot_hip_glu(self.dev, ffn_type, C.c_void_p(bufs[0].ptr), C.c_void_p(bufs[1].ptr), rows,
                                          cols, cols, cols, cols, C.c_void_p(bufs[2].ptr)))
            return bufs[2].download(np.float32, (rows, cols))
        finally:
            for b in bufs:
                b.free()

    def swiglu_pack(self, gate: np.ndarray, up: np.ndarray, kind: int) -> np.ndarray:
        gate = np.ascontiguousarray(gate, dtype=np.float32)
        up = np.ascontiguousarray(up, dtype=np.float32)
        rows, cols = gate.shape
        bufs = [self.to_device(gate), self.to_device(up), self.alloc(self.packed_activation_bytes(kind, rows, cols))]
        try:
            check(self.lib.marmot_hip_swiglu_pack(self.dev, C.c_void_p(bufs[0].ptr), C.c_void_p(bufs[1].ptr), rows,
                                                  cols, kind, C.c_void_p(bufs[2].ptr)))
            return bufs[2].download(np.uint8, (bufs[2].nbytes,))
        finally:
            for b in bufs:
                b.free()

    # ---- tensor operations around the linears
    UNARY_GELU, UNARY_GELU_TANH, UNARY_SILU = 0, 1, 2

    def unary(self, op: int, x: np.ndarray, in_place: bool = False) -> np.ndarray:
        """GELU (erf form), GELU (tanh form) or SiLU of float32 / float16 values (cpu_unary_gelu / _gelu_tanh / _silu,
        src/backends/cpu/ops/unary/scalar/unary_scalar.c:201-218)."""
        x = np.ascontiguousarray(x)
        dt = {np.dtype(np.float32): capi.DT_F32, np.dtype(np.float16): capi.DT_F16}[x.dtype]
        d_x = self.to_device(x) if x.size else None
        d_out = d_x if in_place or not x.size else self.alloc(x.nbytes)
        try:
            if x.size:
                check(self.lib.marmot_hip_unary(self.dev, op, C.c_void_p(d_x.ptr), dt, x.size, C.c_void_p(d_out.ptr)))
                return d_out.download(x.dtype, x.shape)
            return x.copy()
        finally:
            for b_ in {id(d_x): d_x, id(d_out): d_out}.values():
                if b_ is not None:
                    b_.free()

    def softmax(self, x: np.ndarray, axis: int = -1, in_place: bool = False, dtype: int = DT_F32) -> np.ndarray:
        """marmot_softmax of a contiguous tensor along one axis (cpu_softmax_impl,
        src/backends/cpu/ops/softmax/softmax_dispatch.c:67-103). dtype FLOAT32: float32 values; FLOAT16 (1) /
        BFLOAT16 (2): uint16 bit patterns in, uint16 bit patterns out."""
        np_type = np.float32 if dtype == DT_F32 else np.uint16
        x = np.ascontiguousarray(x, dtype=np_type) if dtype == DT_F32 else np.ascontiguousarray(x)
        assert x.dtype == np_type
        axis = axis % x.ndim
        outer = int(np.prod(x.shape[:axis], dtype=np.int64))
        inner = int(np.prod(x.shape[axis + 1:], dtype=np.int64))
        if x.size == 0:
            return x.copy()
        d_x = self.to_device(x)
        d_out = d_x if in_place else self.alloc(x.nbytes)
        try:
            check(self.lib.marmot_hip_softmax_typed(self.dev, dtype, C.c_void_p(d_x.ptr), outer, x.shape[axis], inner,
                                                    C.c_void_p(d_out.ptr)))
            return d_out.download(np_type, x.shape)
        finally:
            d_x.free()
            if d_out is not d_x:
                d_out.free()

    def convert(self, src: np.ndarray, src_dtype: int, dst_dtype: int) -> np.ndarray:
        """marmot_convert between FLOAT32 (float32 arrays), FLOAT16 and BFLOAT16 (uint16 bit patterns)
        (src/backends/cpu/ops/convert/dtype_convert.c:17-130)."""
        src = np.ascontiguousarray(src)
        assert src.dtype == (np.float32 if src_dtype == capi.DT_F32 else np.uint16)
        out_np = np.float32 if dst_dtype == capi.DT_F32 else np.uint16
        if src.size == 0:
            return np.zeros(src.shape, out_np)
        d_src = self.to_device(src)
        d_dst = self.alloc(src.size * np.dtype(out_np).itemsize)
        try:
            check(self.lib.marmot_hip_convert(self.dev, C.c_void_p(d_dst.ptr), dst_dtype, C.c_void_p(d_src.ptr),
                                              src_dtype, src.size))
            return d_dst.download(out_np, src.shape)
        finally:
            d_src.free()
            d_dst.free()

    def gather_rows(self, x: np.ndarray, idx: np.ndarray, out_stride: int | None = None) -> np.ndarray:
        """marmot_gather_rows (cpu_gather_rows, src/backends/cpu/ops/tensor_ops/tensor_ops.c:464-547): x is a 2-D array
        whose rows may be a strided view (unit column stride), idx int32 or uint32. With out_stride (elements) the
        rows land that far apart in a buffer filled with 0xFF bytes, which is returned whole as [rows, out_stride]."""
        assert x.ndim == 2 and idx.ndim == 1 and (x.shape[1] <= 1 or x.strides[1] == x.itemsize)
        idx = np.ascontiguousarray(idx)
        idt = {np.dtype(np.int32): capi.DT_I32, np.dtype(np.uint32): capi.DT_U32}[idx.dtype]
        rows_in, cols = x.shape
        in_stride = x.strides[0] // x.itemsize if rows_in > 1 else cols
        span = ((rows_in - 1) * in_stride + cols) if rows_in else 0
        flat = np.lib.stride_tricks.as_strided(x, shape=(span,), strides=(x.itemsize,)) if span else x.reshape(-1)
        ostride = cols if out_stride is None else out_stride
        n_out = idx.shape[0]
        if n_out == 0 or cols == 0:
            return np.zeros((n_out, ostride), x.dtype)
        out_host = np.full((n_out, ostride), 0xFF, np.uint8).repeat(x.itemsize, axis=1).view(x.dtype)
        bufs = [self.to_device(np.ascontiguousarray(flat)), self.to_device(idx), self.to_device(out_host)]
        try:
            check(self.lib.marmot_hip_gather_rows(self.dev, C.c_void_p(bufs[0].ptr), rows_in, cols * x.itemsize,
                                                  in_stride * x.itemsize, C.c_void_p(bufs[1].ptr), idt, 1, n_out,
                                                  C.c_void_p(bufs[2].ptr), ostride * x.itemsize))
            return bufs[2].download(x.dtype, (n_out, ostride))
        finally:
            for b_ in bufs:
                b_.free()

    def slice(self, x: np.ndarray, starts, sizes) -> np.ndarray:
        """marmot_slice (cpu_slice, tensor_ops.c:401-462): the box [starts, starts + sizes) of a contiguous array."""
        x = np.ascontiguousarray(x)
        n = x.ndim
        out = np.zeros(tuple(int(v) for v in sizes), x.dtype)
        arr = lambda v: (C.c_size_t * n)(*[int(i) for i in v])
        d_x = self.to_device(x) if x.size else self.alloc(16)
        d_out = self.alloc(max(out.nbytes, 16))
        try:
            check(self.lib.marmot_hip_slice(self.dev, C.c_void_p(d_x.ptr), x.itemsize, n, arr(x.shape), arr(starts),
                                            arr(sizes), C.c_void_p(d_out.ptr)))
            return d_out.download(x.dtype, out.shape) if out.size else out
        finally:
            d_x.free()
            d_out.free()

    def add(self, a: np.ndarray, b: np.ndarray) -> np.ndarray:
        a = np.ascontiguousarray(a, dtype=np.float32)
        b = np.ascontiguousarray(b, dtype=np.float32)
        bufs = [self.to_device(a), self.to_device(b), self.alloc(a.size * 4)]
        try:
            check(self.lib.marmot_hip_add(self.dev, C.c_void_p(bufs[0].ptr), C.c_void_p(bufs[1].ptr), a.size,
                                          C.c_void_p(bufs[2].ptr)))
            return bufs[2].download(np.float32, a.shape)
        finally:
            for b_ in bufs:
                b_.free()

    def rope(self, x: np.ndarray, positions: np.ndarray, rope_type: int = 0, dim=None, x_row_stride=None,
             out_row_stride=None, in_place: bool = False, **freq_kw) -> np.ndarray:
        """marmot_rope (include/marmot/ops/rope.h; CPU implementation src/backends/cpu/ops/rope/rope_dispatch.c): the
        last dimension of x (float32 or float16, rank >= 2) is rotated, one position (float32, int32 or int64) per row;
        freq_kw are the keyword arguments of rope_frequencies (head_dim is the rotated dimension). With `dim` and row
        strides (in elements), x is a flat buffer of positions.size rows of dim values at x_row_stride and the result
        a flat buffer of rows at out_row_stride (its gaps keep the NaN they are filled with)."""
        x = np.ascontiguousarray(x)
        pos = np.ascontiguousarray(positions)
        pos_dt = {np.dtype(np.float32): capi.DT_F32, np.dtype(np.int32): capi.DT_I32,
                  np.dtype(np.int64): capi.DT_I64}[pos.dtype]
        if dim is None:
            dim = x.shape[-1]
            rows = x.size // dim
            xs = os_ = dim
            out_shape, out_size = x.shape, x.size
        else:
            rows, xs, os_ = pos.size, x_row_stride, out_row_stride
            out_size = (rows - 1) * os_ + dim
            out_shape = (out_size,)
        freq_kw.pop("head_dim", None)
        freqs, scale, hd = self.rope_frequencies(dim, head_dim=dim, **freq_kw)
        d_x, d_p, d_f = self.to_device(x), self.to_device(pos), self.to_device(freqs)
        d_o = d_x if in_place else self.to_device(np.full(out_size, np.nan, dtype=x.dtype))
        arg = capi.Rope(d_p.ptr, pos_dt, d_f.ptr, scale, hd, rope_type, 0, 0)
        try:
            check(self.lib.marmot_hip_rope(self.dev, C.c_void_p(d_x.ptr), _np_dtype_id(x.dtype), rows, dim, xs, os_,
                                           C.byref(arg), C.c_void_p(d_o.ptr)))
            return d_o.download(x.dtype, out_shape)
        finally:
            for b in {d_x, d_p, d_f, d_o}:
                b.free()

    def paged_attention_args(self, dev_ptr, token_meta, q, k_new, v_new, kv_k, kv_v, block_table, out, layer_idx: int,
                             scale: float, act_bf16: bool = False, kv_bf16: bool = False, token_count=None,
                             kv_k_scale=None, kv_v_scale=None):
        """marmot_hip_paged_attention_t over numpy arrays (shapes, dtypes and element strides) whose device addresses
        dev_ptr(array) gives; bfloat16 tensors travel as uint16 bits."""
        def code(a, bf16):
            if bf16:
                assert a.dtype == np.uint16
                return capi.DT_BF16
            return _np_dtype_id(a.dtype)

        def strides(a):
            return [st // a.itemsize for st in a.strides]

        p = capi.PagedAttention()
        p.token_count = q.shape[0] if token_count is None else token_count
        p.layer_idx, p.scale = layer_idx, scale
        p.num_q_heads, p.num_kv_heads, p.head_dim, p.block_size = q.shape[1], k_new.shape[1], q.shape[2], kv_k.shape[3]
        p.act_dtype = code(q, act_bf16)
        if kv_k.dtype == np.uint8:  # FLOAT8_E4M3 cache with float32 scales [blocks, layers, kv heads]
            p.kv_dtype = capi.DT_F8_E4M3
        else:
            p.kv_dtype = code(kv_k, kv_bf16)
        if kv_k_scale is not None:
            assert kv_k_scale.dtype == np.float32 and kv_k_scale.strides == kv_v_scale.strides
            p.d_kv_k_scale, p.d_kv_v_scale = dev_ptr(kv_k_scale), dev_ptr(kv_v_scale)
            p.scale_stride = (C.c_size_t * 3)(*strides(kv_k_scale))
        p.d_token_meta, p.meta_stride = dev_ptr(token_meta), (C.c_size_t * 2)(*strides(token_meta))
        p.d_q, p.d_k_new, p.d_v_new = dev_ptr(q), dev_ptr(k_new), dev_ptr(v_new)
        p.q_stride = (C.c_size_t * 3)(*strides(q))
        p.k_stride = (C.c_size_t * 3)(*strides(k_new))
        p.v_stride = (C.c_size_t * 3)(*strides(v_new))
        p.d_kv_k, p.d_kv_v, p.kv_stride = dev_ptr(kv_k), dev_ptr(kv_v), (C.c_size_t * 5)(*strides(kv_k))
        p.kv_blocks, p.kv_layers = kv_k.shape[0], kv_k.shape[1]
        p.d_block_table, p.table_stride = dev_ptr(block_table), (C.c_size_t * 2)(*strides(block_table))
        p.max_seqs, p.max_blocks_per_seq = block_table.shape
        p.d_out, p.out_stride = dev_ptr(out), (C.c_size_t * 3)(*strides(out))
        return p

    def paged_attention(self, token_meta, q, k_new, v_new, kv_k, kv_v, block_table, layer_idx: int, scale: float,
                        act_bf16: bool = False, kv_bf16: bool = False, token_count=None, validate: bool = True,
                        kv_k_scale=None, kv_v_scale=None):
        """marmot_paged_attention (include/marmot/ops/paged_attention.h; CPU implementation
        src/backends/cpu/ops/paged_attention/paged_attention_ref.c): token_meta [tokens, 4] uint32 (seq_slot, pos,
        kv_slot, flags), q [tokens, q heads, head dim], k_new / v_new [tokens, kv heads, head dim] (float32, float16 or
        uint16 holding bfloat16 bits; views with any strides), kv_k / kv_v [blocks, layers, kv heads, block size, head
        dim] (updated in place; uint8 = FLOAT8_E4M3 with the float32 scale tensors kv_k_scale / kv_v_scale [blocks,
        layers, kv heads], updated in place too), block_table [sequences, blocks per sequence] uint32. Returns out
        like q."""
        out = np.zeros(q.shape, dtype=q.dtype)
        arrays = [token_meta, q, k_new, v_new, kv_k, kv_v, block_table, out]
        scales = [a for a in (kv_k_scale, kv_v_scale) if a is not None]
        arrays += scales
        roots = {}

        def root_of(a):
            while a.base is not None and isinstance(a.base, np.ndarray):
                a = a.base
            return a

        for a in arrays:
            r = root_of(a)
            if id(r) not in roots:
                assert r.flags.c_contiguous, "views must come from contiguous arrays"
                roots[id(r)] = (r, self.to_device(r.reshape(-1).view(np.uint8)))

        def dev_ptr(a):
            r, d = roots[id(root_of(a))]
            return d.ptr + (a.ctypes.data - r.ctypes.data)

        p = self.paged_attention_args(dev_ptr, token_meta, q, k_new, v_new, kv_k, kv_v, block_table, out, layer_idx,
                                      scale, act_bf16, kv_bf16, token_count, kv_k_scale, kv_v_scale)
        try:
            check(self.lib.marmot_hip_paged_attention(self.dev, C.byref(p), 1 if validate else 0))
            for a in [kv_k, kv_v, out] + scales:
                r, d = roots[id(root_of(a))]
                flat = r.reshape(-1).view(np.uint8)
                flat[...] = d.download(np.uint8, (flat.size,))
            return out
        finally:
            for _, d in roots.values():
                d.free()

    def packed_activation_layout(self, kind: int, N: int, K: int) -> "capi.PackedLayout":
        lay = capi.PackedLayout()
        check(self.lib.marmot_hip_packed_activation_layout(kind, N, K, C.byref(lay)))
        return lay

    def moe_experts_probe(self, hidden, gate, up, down, topk_ids, topk_weights, F: int, E: int, kind_gate_up: int,
                          kind_down: int, weights_scale: float = 1.0, policy: int = 1, ffn_type: int = 0,
                          fused_override: np.ndarray = None) -> dict:
        """moe_experts with every stage read back: {"out", "sorted_tokens", "route_pos", "gate_out", "up_out",
        "fused_packed" (uint8 image, see packed_activation_layout)}. `fused_override`, a packed image of the same
        size, replaces the activations the down projection reads."""
        hidden = np.ascontiguousarray(hidden, dtype=np.float32)
        T, H = hidden.shape
        ids = np.ascontiguousarray(topk_ids, dtype=np.int32)
        w = np.ascontiguousarray(topk_weights, dtype=np.float32)
        kpt = ids.shape[1]
        routes = T * kpt
        packed_bytes = self.packed_activation_bytes(kind_down, routes, F)
        ins = [self.to_device(a) for a in (hidden, np.ascontiguousarray(gate, dtype=np.uint8),
                                           np.ascontiguousarray(up, dtype=np.uint8),
                                           np.ascontiguousarray(down, dtype=np.uint8), ids, w)]
        outs = [self.alloc(n) for n in (T * H * 4, routes * 4, routes * 4, routes * F * 4, routes * F * 4,
                                        packed_bytes)]
        if fused_override is not None:
            fused_override = np.ascontiguousarray(fused_override, dtype=np.uint8)
            assert fused_override.size == packed_bytes
            ins.append(self.to_device(fused_override))
        try:
            probe = capi.MoeProbe(outs[1].ptr, outs[2].ptr, outs[3].ptr, outs[4].ptr, outs[5].ptr,
                                  ins[6].ptr if fused_override is not None else None)
            check(self.lib.marmot_hip_moe_experts_probe(
                self.dev, C.c_void_p(ins[0].ptr), T, H, F, E, kpt, kind_gate_up, kind_down, C.c_void_p(ins[1].ptr),
                C.c_void_p(ins[2].ptr), C.c_void_p(ins[3].ptr), C.c_void_p(ins[4].ptr), C.c_void_p(ins[5].ptr),
                weights_scale, policy, ffn_type, C.c_void_p(outs[0].ptr), C.byref(probe)))
            return {"out": outs[0].download(np.float32, (T, H)),
                    "sorted_tokens": outs[1].download(np.uint32, (routes,)),
                    "route_pos": outs[2].download(np.int32, (T, kpt)),
                    "gate_out": outs[3].download(np.float32, (routes, F)),
                    "up_out": outs[4].download(np.float32, (routes, F)),
                    "fused_packed": outs[5].download(np.uint8, (packed_bytes,))}
        finally:
            for b in ins + outs:
                b.free()

    def moe_experts(self, hidden, gate, up, down, topk_ids, topk_weights, F: int, E: int, kind_gate_up: int,
                    kind_down: int, weights_scale: float = 1.0, policy: int = 1, ffn_type: int = 0) -> np.ndarray:
        hidden = np.ascontiguousarray(hidden, dtype=np.float32)
        T, H = hidden.shape
        ids = np.ascontiguousarray(topk_ids, dtype=np.int32)
        w = np.ascontiguousarray(topk_weights, dtype=np.float32)
        kpt = ids.shape[1]
        bufs = [self.to_device(a) for a in (hidden, np.ascontiguousarray(gate, dtype=np.uint8),
                                            np.ascontiguousarray(up, dtype=np.uint8),
                                            np.ascontiguousarray(down, dtype=np.uint8), ids, w)]
        d_out = self.alloc(T * H * 4)
        try:
            check(self.lib.marmot_hip_moe_experts(
                self.dev, C.c_void_p(bufs[0].ptr), T, H, F, E, kpt, kind_gate_up, kind_down, C.c_void_p(bufs[1].ptr),
                C.c_void_p(bufs[2].ptr), C.c_void_p(bufs[3].ptr), C.c_void_p(bufs[4].ptr), C.c_void_p(bufs[5].ptr),
                weights_scale, policy, ffn_type, C.c_void_p(d_out.ptr)))
            return d_out.download(np.float32, (T, H))
        finally:
            for b in bufs + [d_out]:
                b.free()
