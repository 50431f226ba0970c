"""CPU tests of the marmot_tensor_t-level backend layer: ABI layout against the reference's headers, exported
tables, kernel query rules, bytecode immediates, kernel DSL files. No device work happens here."""
import ctypes as C
import os
import re
import struct
import subprocess

import pytest

from marmot_amd import capi
from marmot_amd import tensor_abi as ta

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLDEN = os.path.join(ROOT, "tests", "golden")
REFERENCE = "/root/reference"


def _facts(text):
    out = {}
    for line in text.splitlines():
        name, value = line.rsplit(" ", 1)
        out[name] = int(value)
    return out


@pytest.fixture(scope="module")
def golden_layout():
    with open(os.path.join(GOLDEN, "abi_layout.txt")) as f:
        return _facts(f.read())


@pytest.fixture(scope="module")
def lib():
    return ta.bind(capi.load_library())


def test_mirror_header_matches_reference_layout(tmp_path, golden_layout):
    exe = tmp_path / "abi_mirror"
    subprocess.run(["gcc", "-std=c11", f"-I{ROOT}/include", "-o", str(exe), os.path.join(GOLDEN, "abi_probe.c")],
                   check=True)
    mine = _facts(subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout)
    assert mine == golden_layout
    assert len(mine) > 150


@pytest.mark.skipif(not os.path.isdir(REFERENCE), reason="reference tree not present")
def test_layout_fixture_is_current(golden_layout):
    import importlib.util
    spec = importlib.util.spec_from_file_location("make_abi_layout", os.path.join(GOLDEN, "make_abi_layout.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    assert _facts(mod.reference_layout()) == golden_layout


def test_ctypes_structs_match_layout(golden_layout):
    pairs = {
        "marmot_shape_t": ta.Shape, "marmot_tensor_t": ta.Tensor, "marmot_matmul_epilogue_t": ta.Epilogue,
        "marmot_topk_desc_t": ta.TopkDesc, "marmot_moe_experts_desc_t": ta.MoeDesc,
        "marmot_rmsnorm_desc_t": ta.RmsNormDesc, "marmot_softmax_desc_t": ta.SoftmaxDesc,
        "marmot_activation_params_t": ta.ActivationParams,
        "marmot_op_signature_t": ta.OpSignature, "marmot_kernel_selection_t": ta.KernelSelection,
        "marmot_device_caps_t": ta.DeviceCaps, "marmot_device_ops_t": ta.DeviceOps,
        "marmot_bc_exec_ctx_t": ta.BcExecCtx, "marmot_bc_tables_t": ta.BcTables,
        "marmot_allocator_usage_t": ta.AllocatorUsage, "marmot_context_policy_t": ta.ContextPolicy,
        "marmot_backend_preferences_t": ta.BackendPreferences, "marmot_matmul_dims_t": ta.MatmulDims,
        "marmot_quant_block_t": ta.QuantBlock, "marmot_rope_params_t": ta.RopeParams,
        "marmot_matmul_qkv_desc_t": ta.QkvDesc, "marmot_matmul_qkv_separate_t": ta.QkvSeparate,
        "marmot_embedding_gather_desc_t": ta.EmbeddingGatherDesc,
        "marmot_paged_attention_desc_t": ta.PagedAttentionDesc,
        "marmot_paged_attention_kv_scale_ext_t": ta.PagedAttentionKvScaleExt,
    }
    checked = 0
    for cname, cls in pairs.items():
        assert C.sizeof(cls) == golden_layout[f"sizeof({cname})"], cname
        for key, off in golden_layout.items():
            m = re.fullmatch(rf"offsetof\({cname},(\w+)\)", key)
            if m:
                assert getattr(cls, m.group(1)).offset == off, key
                checked += 1
    assert checked >= 114
    assert ta.OP_MATMUL == golden_layout["MARMOT_OP_MATMUL"]
    assert ta.OP_MOE_EXPERTS == golden_layout["MARMOT_OP_MOE_EXPERTS"]
    assert ta.OP_TOPK == golden_layout["MARMOT_OP_TOPK"]
    assert ta.OP_EMBEDDING == golden_layout["MARMOT_OP_EMBEDDING"]
    assert ta.DTYPE_I64 == golden_layout["MARMOT_DTYPE_INT64"]
    assert (ta.PREFERENCE_ENABLE, ta.PREFERENCE_DISABLE) == (
        golden_layout["MARMOT_PREFERENCE_ENABLE"], golden_layout["MARMOT_PREFERENCE_DISABLE"])
    assert ta.QSCHEME_OF_KIND[ta.KIND_Q4_K] == golden_layout["MARMOT_QSCHEME_Q4_K"]
    assert ta.QSCHEME_OF_KIND[ta.KIND_Q6_K] == golden_layout["MARMOT_QSCHEME_Q6_K"]
    assert ta.QSCHEME_OF_KIND[ta.KIND_Q5_K] == golden_layout["MARMOT_QSCHEME_Q5_K"]
    assert ta.KIND_Q5_K == golden_layout["MARMOT_QUANT_KIND_Q5_K"]
    for name in ("Q4_1", "Q5_0", "Q5_1", "Q2_K", "Q3_K", "Q8_1"):
        kind = getattr(ta, f"KIND_{name}")
        assert kind == golden_layout[f"MARMOT_QUANT_KIND_{name}"]
        assert ta.QSCHEME_OF_KIND[kind] == golden_layout[f"MARMOT_QSCHEME_{name}"]
    assert ta.KIND_Q8_K == golden_layout["MARMOT_QUANT_KIND_Q8_K"]
    assert ta.NOT_IMPLEMENTED == golden_layout["MARMOT_ERROR_NOT_IMPLEMENTED"]
    assert ta.BACKEND_HIP == golden_layout["MARMOT_BACKEND_CUDA"] + 1


def test_backend_symbols_declared_and_exported(lib):
    header = open(os.path.join(ROOT, "include", "marmot_hip_backend.h")).read()
    for name in ta.BACKEND_SYMBOLS:
        assert re.search(rf"\b{name}\s*\(", header), f"{name} not declared in marmot_hip_backend.h"
        assert getattr(lib, name) is not None
    declared = set(re.findall(r"\b((?:marmot_get_hip|marmot_hip_|hip_)\w+)\s*\(", header))
    assert declared == set(ta.BACKEND_SYMBOLS)


def test_vtable_is_complete(lib):
    ops = lib.marmot_get_hip_ops().contents
    for name, _ in ta.DeviceOps._fields_:
        assert getattr(ops, name), f"vtable entry {name} is null"
    # same table on every call
    assert C.addressof(lib.marmot_get_hip_ops().contents) == C.addressof(ops)


def _sig(op=ta.OP_MATMUL, kind=ta.KIND_Q4_K, inp=ta.DTYPE_F32, out=ta.DTYPE_F32, N=1, K=4096, M=14336):
    s = ta.OpSignature()
    s.op_id = op
    s.profile_id = ta.PROFILE_SCALAR
    s.matmul_layout = ta.MATMUL_LAYOUT_NT
    s.input_dtype, s.weight_dtype, s.output_dtype, s.accum_dtype = inp, ta.DTYPE_U8, out, ta.DTYPE_F32
    s.qscheme_id = ta.QSCHEME_OF_KIND.get(kind, 0)
    s.weight_layout = ta.WEIGHT_LAYOUT_SEPARATE
    s.dims.matmul.N, s.dims.matmul.K, s.dims.matmul.M = N, K, M
    return s


def _caps():
    c = ta.DeviceCaps()
    c.mem_bw_gbps = 8000.0
    c.peak_flops_tflops_fp16 = 2500.0
    c.launch_overhead_us = 2.0
    return c


def _query(lib, sig):
    caps = _caps()
    return lib.marmot_hip_query_kernel(C.byref(sig), C.byref(caps))


def test_query_kernel_matmul_rules(lib):
    expect_op = {ta.KIND_Q4_0: 1, ta.KIND_Q8_0: 2, ta.KIND_Q4_K: 3, ta.KIND_Q6_K: 4, ta.KIND_Q5_K: 20, ta.KIND_Q4_1: 24,
                 ta.KIND_Q5_0: 28, ta.KIND_Q5_1: 32, ta.KIND_Q2_K: 36, ta.KIND_Q3_K: 40,
                 ta.KIND_Q8_1: 44}
    for kind, op in expect_op.items():
        sel = _query(lib, _sig(kind=kind))
        assert sel.supported and sel.op_index == op and sel.kernel_id == 0x4000 + op
        assert sel.fallback_reason is None
    # profile is a wildcard
    s = _sig()
    for profile in (0, 1, 2, 3, 4):
        s.profile_id = profile
        assert _query(lib, s).supported
    # LINEAR resolves like MATMUL
    assert _query(lib, _sig(op=ta.OP_LINEAR)).op_index == 3
    # dtype pairs: f32->f32, f16->f32, f16->f16 yes; f32->f16 no
    assert _query(lib, _sig(inp=ta.DTYPE_F16, out=ta.DTYPE_F32)).supported
    assert _query(lib, _sig(inp=ta.DTYPE_F16, out=ta.DTYPE_F16)).supported
    assert not _query(lib, _sig(inp=ta.DTYPE_F32, out=ta.DTYPE_F16)).supported
    # every weight scheme takes fp16 activations (the K-quants as the reference's fp16 direct dots compute them)
    for kind in (ta.KIND_Q2_K, ta.KIND_Q3_K, ta.KIND_Q5_K, ta.KIND_Q6_K):
        assert _query(lib, _sig(kind=kind, inp=ta.DTYPE_F16)).supported
    sel = _query(lib, _sig(kind=ta.KIND_Q8_K))
    assert not sel.supported and sel.op_index == 0xFFFF and sel.fallback_reason
    # unsupported scheme, layout, weight layout, stride mode, epilogue, variant
    assert not _query(lib, _sig(kind=ta.KIND_Q8_K)).supported
    s = _sig(); s.qscheme_id = 13  # beyond the enumeration
    assert not _query(lib, s).supported
    s = _sig(); s.matmul_layout = 1
    assert not _query(lib, s).supported
    s = _sig(); s.weight_layout = 2
    assert not _query(lib, s).supported
    s = _sig(); s.stride_mode = 3
    assert not _query(lib, s).supported
    s = _sig(); s.stride_mode = 1
    assert _query(lib, s).supported
    s = _sig(); s.epilogue_flags = ta.EPILOGUE_BIAS
    assert _query(lib, s).supported
    s = _sig(); s.epilogue_flags = ta.EPILOGUE_BIAS | 2
    assert not _query(lib, s).supported
    s = _sig(); s.variant_flags = 1
    assert not _query(lib, s).supported
    s = _sig(); s.accum_dtype = ta.DTYPE_F16
    assert not _query(lib, s).supported
    # null arguments
    sel = lib.marmot_hip_query_kernel(None, None)
    assert not sel.supported


def test_query_kernel_cost_model(lib):
    # decode matvec is priced by bytes over HBM bandwidth, prefill by flops over the MFMA peak
    decode = _query(lib, _sig(N=1, K=4096, M=14336))
    nbytes = 14336 * 16 * 144 + 4096 * 4 + 14336 * 4
    assert decode.estimated_us == pytest.approx(2.0 + nbytes / 8000e3, rel=1e-6)
    prefill = _query(lib, _sig(inp=ta.DTYPE_F16, N=512, K=4096, M=4096))
    assert prefill.estimated_us == pytest.approx(2.0 + 2 * 512 * 4096 * 4096 / 2500e6, rel=1e-6)
    assert decode.est_workspace_mb > 0 and prefill.est_workspace_mb == 0


def test_query_kernel_other_ops(lib):
    for kind, op in {ta.KIND_Q4_0: 5, ta.KIND_Q8_0: 6, ta.KIND_Q4_K: 7, ta.KIND_Q6_K: 8, ta.KIND_Q5_K: 21,
                     ta.KIND_Q4_1: 25, ta.KIND_Q5_0: 29, ta.KIND_Q5_1: 33, ta.KIND_Q2_K: 37,
                     ta.KIND_Q3_K: 41, ta.KIND_Q8_1: 45}.items():
        assert _query(lib, _sig(op=ta.OP_MOE_EXPERTS, kind=kind)).op_index == op
    assert not _query(lib, _sig(op=ta.OP_MOE_EXPERTS, inp=ta.DTYPE_F16, out=ta.DTYPE_F16)).supported
    assert _query(lib, _sig(op=ta.OP_TOPK)).op_index == 9
    assert _query(lib, _sig(op=ta.OP_QUANTIZE, kind=ta.KIND_Q8_K)).op_index == 10
    assert _query(lib, _sig(op=ta.OP_QUANTIZE, kind=ta.KIND_Q8_0, inp=ta.DTYPE_F16)).op_index == 10
    # weight formats with the K-quant searches on the device: FLOAT32 input only
    assert _query(lib, _sig(op=ta.OP_QUANTIZE, kind=ta.KIND_Q4_K)).op_index == 10
    assert _query(lib, _sig(op=ta.OP_QUANTIZE, kind=ta.KIND_Q6_K)).op_index == 10
    assert not _query(lib, _sig(op=ta.OP_QUANTIZE, kind=ta.KIND_Q4_K, inp=ta.DTYPE_F16)).supported
    assert not _query(lib, _sig(op=ta.OP_QUANTIZE, kind=ta.KIND_Q4_0)).supported
    assert _query(lib, _sig(op=ta.OP_DEQUANTIZE, kind=ta.KIND_Q6_K)).op_index == 11
    # rope: rows and result of one type, FLOAT32 or FLOAT16
    assert _query(lib, _sig(op=ta.OP_ROPE, kind=ta.KIND_GENERIC)).op_index == ta.BC_OP_ROPE
    assert _query(lib, _sig(op=ta.OP_ROPE, kind=ta.KIND_GENERIC, inp=ta.DTYPE_F16, out=ta.DTYPE_F16)).op_index == 53
    assert not _query(lib, _sig(op=ta.OP_ROPE, kind=ta.KIND_GENERIC, inp=ta.DTYPE_F16, out=ta.DTYPE_F32)).supported
    assert not _query(lib, _sig(op=12345)).supported


def test_query_kernel_qkv_rules(lib, golden_layout):
    """cpu/kernels/matmul_qkv.def:19-36, 54-71 with this backend's schemes; outputs carry the activation dtype."""
    assert (ta.OP_QKV_PROJECTION, ta.OP_QKV_SHARED_INPUT, ta.OP_QKV_ROPE) == tuple(
        golden_layout[k] for k in ("MARMOT_OP_QKV_PROJECTION", "MARMOT_OP_QKV_SHARED_INPUT", "MARMOT_OP_QKV_ROPE"))
    assert ta.EPILOGUE_ROPE == golden_layout["MARMOT_EPILOGUE_ROPE"]
    for op_id in (ta.OP_QKV_PROJECTION, ta.OP_QKV_SHARED_INPUT, ta.OP_QKV_ROPE):
        for kind, op in {ta.KIND_Q4_0: 12, ta.KIND_Q8_0: 13, ta.KIND_Q4_K: 14, ta.KIND_Q6_K: 15,
                         ta.KIND_Q5_K: 22, ta.KIND_Q4_1: 26, ta.KIND_Q5_0: 30, ta.KIND_Q5_1: 34,
                         ta.KIND_Q2_K: 38, ta.KIND_Q3_K: 42, ta.KIND_Q8_1: 46}.items():
            for dt in (ta.DTYPE_F32, ta.DTYPE_F16):
                sel = _query(lib, _sig(op=op_id, kind=kind, inp=dt, out=dt, N=4, K=4096, M=4096))
                assert sel.supported and sel.op_index == op and sel.kernel_id == 0x4000 + op
    s = _sig(op=ta.OP_QKV_SHARED_INPUT, inp=ta.DTYPE_F16, out=ta.DTYPE_F32)
    assert not _query(lib, s).supported  # outputs must have the activation dtype
    s = _sig(op=ta.OP_QKV_SHARED_INPUT); s.epilogue_flags = ta.EPILOGUE_BIAS
    assert _query(lib, s).supported
    s = _sig(op=ta.OP_QKV_SHARED_INPUT); s.epilogue_flags = ta.EPILOGUE_BIAS | ta.EPILOGUE_ROPE
    assert _query(lib, s).supported
    s = _sig(op=ta.OP_QKV_SHARED_INPUT); s.epilogue_flags = ta.EPILOGUE_ROPE | 2  # activation epilogue
    sel = _query(lib, s)
    assert not sel.supported and b"rotary" in sel.fallback_reason
    assert not _query(lib, _sig(op=ta.OP_QKV_SHARED_INPUT, kind=ta.KIND_Q8_K)).supported
    s = _sig(op=ta.OP_QKV_SHARED_INPUT); s.weight_layout = 2
    assert not _query(lib, s).supported
    # three weight streams, one activation read, three outputs
    sel = _query(lib, _sig(op=ta.OP_QKV_SHARED_INPUT, N=1, K=4096, M=4096))
    nbytes = 3 * 4096 * 16 * 144 + 4096 * 4 + 3 * 4096 * 4
    assert sel.estimated_us == pytest.approx(2.0 + nbytes / 8000e3, rel=1e-6) and sel.est_workspace_mb > 0


def test_default_caps_and_preferences(lib):
    caps = lib.marmot_hip_detect_default_caps()
    assert caps.mem_bw_gbps == pytest.approx(8000.0)
    assert caps.peak_flops_tflops_fp16 == pytest.approx(2500.0)
    assert caps.simd_width == 64 and caps.num_compute_units >= 1 and caps.has_tensor_cores
    prefs = ta.BackendPreferences()
    assert lib.marmot_hip_default_preferences(C.byref(caps), C.byref(prefs))
    assert prefs.routing_policy == 1 and not prefs.policy.matmul_requires_temp_tensors
    assert not prefs.policy.matmul_prefer_packed_weights
    assert not lib.marmot_hip_default_preferences(None, C.byref(prefs))


def test_query_kernel_embedding_rules(lib):
    """cpu/kernels/embedding.def:19-30 with this backend's schemes, index and output types."""
    def sig(kind=ta.KIND_Q4_K, ids=ta.DTYPE_I32, out=ta.DTYPE_F32):
        s = ta.OpSignature()
        s.op_id, s.input_dtype, s.weight_dtype, s.output_dtype = ta.OP_EMBEDDING, ids, ta.DTYPE_U8, out
        s.qscheme_id = ta.QSCHEME_OF_KIND.get(kind, 0)
        s.weight_layout = ta.WEIGHT_LAYOUT_SEPARATE
        return s
    for kind, op in ((ta.KIND_Q4_0, 16), (ta.KIND_Q8_0, 17), (ta.KIND_Q4_K, 18), (ta.KIND_Q6_K, 19),
                     (ta.KIND_Q5_K, 23), (ta.KIND_Q4_1, 27), (ta.KIND_Q5_0, 31), (ta.KIND_Q5_1, 35), (ta.KIND_Q2_K, 39), (ta.KIND_Q3_K, 43),
                     (ta.KIND_Q8_1, 47)):
        for ids in (ta.DTYPE_I32, ta.DTYPE_I64):
            for out in (ta.DTYPE_F32, ta.DTYPE_F16):
                sel = _query(lib, sig(kind, ids, out))
                assert sel.supported and sel.op_index == op
    assert not _query(lib, sig(kind=ta.KIND_Q8_K)).supported
    assert not _query(lib, sig(kind=ta.KIND_GENERIC)).supported
    assert not _query(lib, sig(ids=ta.DTYPE_F32)).supported
    assert not _query(lib, sig(out=ta.DTYPE_I32)).supported


def test_query_kernel_paged_attention_rules(lib):
    """cpu/kernels/paged_attention.def:3-22: activations and result of one float type, the cache type (FLOAT8_E4M3
    included) as the weight type."""
    def sig(act=ta.DTYPE_F32, kv=ta.DTYPE_F16, out=None):
        s = ta.OpSignature()
        s.op_id, s.input_dtype, s.weight_dtype = ta.OP_PAGED_ATTENTION, act, kv
        s.output_dtype = act if out is None else out
        s.accum_dtype = ta.DTYPE_F32
        return s
    for act in (ta.DTYPE_F32, ta.DTYPE_F16, ta.DTYPE_BF16):
        for kv in (ta.DTYPE_F32, ta.DTYPE_F16, ta.DTYPE_BF16):
            sel = _query(lib, sig(act, kv))
            assert sel.supported and sel.op_index == ta.BC_OP_PAGED_ATTENTION
    assert _query(lib, sig(kv=ta.DTYPE_F8_E4M3)).supported
    assert not _query(lib, sig(kv=ta.DTYPE_I32)).supported
    assert not _query(lib, sig(act=ta.DTYPE_I32)).supported
    assert not _query(lib, sig(out=ta.DTYPE_F16)).supported


def test_bytecode_tables(lib, golden_layout):
    t = ta.BcTables()
    assert lib.marmot_hip_bc_get_tables(C.byref(t))
    assert not lib.marmot_hip_bc_get_tables(None)
    assert t.op_count == 64
    assert not t.exec_table[0] and t.imm_size[0] == 0  # opcode 0 is END
    schema = [t.schema_id[i] for i in range(t.op_count)]
    assert schema[1:5] == [golden_layout["MARMOT_BC_SCHEMA_MATMUL"]] * 4
    assert schema[5:9] == [golden_layout["MARMOT_BC_SCHEMA_MOE_EXPERTS"]] * 4
    assert schema[9] == golden_layout["MARMOT_BC_SCHEMA_TOPK"]
    assert schema[10] == golden_layout["MARMOT_BC_SCHEMA_QUANTIZE"]
    assert schema[11] == golden_layout["MARMOT_BC_SCHEMA_DEQUANTIZE"]
    assert schema[12:16] == [golden_layout["MARMOT_BC_SCHEMA_QKV"]] * 4
    assert schema[16:20] == [golden_layout["MARMOT_BC_SCHEMA_EMBEDDING"]] * 4
    # immediate sizes equal what the encoders of tensor_abi.Program emit (opcode excluded)
    sizes = [t.imm_size[i] for i in range(t.op_count)]
    assert sizes[1:5] == [struct.calcsize("<HHHIH")] * 4
    assert sizes[5:9] == [struct.calcsize("<7HIfI")] * 4
    assert sizes[9] == struct.calcsize("<HHHII")
    assert sizes[10] == struct.calcsize("<HIHII")
    assert sizes[11] == struct.calcsize("<HHII")
    assert sizes[12:16] == [struct.calcsize("<7HII3H")] * 4
    assert sizes[16:20] == [struct.calcsize("<3HIfI3B")] * 4 == [21] * 4
    # Q5_K was added behind the four original kinds: one op per family
    # kinds added behind the four original ones (Q5_K, Q4_1, Q5_0, Q5_1, Q2_K, Q3_K, Q8_1): four consecutive ops
    # each
    for base in (20, 24, 28, 32, 36, 40, 44):
        assert schema[base:base + 4] == [golden_layout[f"MARMOT_BC_SCHEMA_{n}"]
                                         for n in ("MATMUL", "MOE_EXPERTS", "QKV", "EMBEDDING")]
        assert sizes[base:base + 4] == [sizes[1], sizes[5], sizes[12], sizes[16]]
    # the FLOAT32 ops between the linears: two normalizations, three binary ops
    assert schema[48:50] == [golden_layout["MARMOT_BC_SCHEMA_RMS_NORM"]] * 2
    assert schema[50:53] == [golden_layout["MARMOT_BC_SCHEMA_BINARY"]] * 3
    assert sizes[48:50] == [struct.calcsize("<4Hf")] * 2 and sizes[50:53] == [struct.calcsize("<3H")] * 3
    assert (ta.BC_OP_RMS_NORM_F32, ta.BC_OP_RMS_NORM_GEMMA_F32, ta.BC_OP_SWIGLU_F32, ta.BC_OP_GEGLU_F32,
            ta.BC_OP_ADD_F32) == (48, 49, 50, 51, 52)
    # the rotary embedding: input, output and positions registers, parameter offset, n_past, n_rot
    assert schema[53] == golden_layout["MARMOT_BC_SCHEMA_ROPE"] and sizes[53] == struct.calcsize("<3H3I") == 18
    assert ta.BC_OP_ROPE == 53 and ta.OP_ROPE == golden_layout["MARMOT_OP_ROPE"]
    # paged attention: ten tensor registers, six u32 and the scale
    assert schema[54] == golden_layout["MARMOT_BC_SCHEMA_PAGED_ATTENTION"]
    assert sizes[54] == struct.calcsize("<10H6If") == 48
    assert ta.BC_OP_PAGED_ATTENTION == 54 and ta.OP_PAGED_ATTENTION == golden_layout["MARMOT_OP_PAGED_ATTENTION"]
    assert (ta.DTYPE_BF16, ta.DTYPE_U32, ta.DTYPE_F8_E4M3) == (
        golden_layout["MARMOT_DTYPE_BFLOAT16"], golden_layout["MARMOT_DTYPE_UINT32"],
        golden_layout["MARMOT_DTYPE_FLOAT8_E4M3"])
    # the remaining nodes of a model graph: three unary activations, softmax, reshape, view, slice, gather_rows, convert
    assert schema[55:58] == [golden_layout["MARMOT_BC_SCHEMA_UNARY"]] * 3 and sizes[55:58] == [struct.calcsize("<2HI")] * 3
    assert schema[58] == golden_layout["MARMOT_BC_SCHEMA_SOFTMAX"] and sizes[58] == struct.calcsize("<2HI")
    assert schema[59] == golden_layout["MARMOT_BC_SCHEMA_RESHAPE"] and sizes[59] == struct.calcsize("<2HIQ") == 16
    assert schema[60] == golden_layout["MARMOT_BC_SCHEMA_VIEW"] and sizes[60] == struct.calcsize("<2HQ") == 12
    assert schema[61] == golden_layout["MARMOT_BC_SCHEMA_SLICE"] and sizes[61] == struct.calcsize("<2H2I") == 12
    assert schema[62] == golden_layout["MARMOT_BC_SCHEMA_GATHER_ROWS"] and sizes[62] == struct.calcsize("<3H")
    assert schema[63] == golden_layout["MARMOT_BC_SCHEMA_CONVERT"] and sizes[63] == struct.calcsize("<2IQ2I") == 24
    assert (ta.BC_OP_GELU, ta.BC_OP_GELU_TANH, ta.BC_OP_SILU, ta.BC_OP_SOFTMAX_F32, ta.BC_OP_RESHAPE, ta.BC_OP_VIEW,
            ta.BC_OP_SLICE, ta.BC_OP_GATHER_ROWS, ta.BC_OP_CONVERT) == tuple(range(55, 64))
    assert (ta.OP_GELU, ta.OP_GELU_TANH, ta.OP_SILU, ta.OP_SOFTMAX, ta.OP_RESHAPE, ta.OP_VIEW, ta.OP_SLICE,
            ta.OP_GATHER_ROWS, ta.OP_CONVERT) == tuple(
        golden_layout["MARMOT_OP_" + n] for n in ("GELU", "GELU_TANH", "SILU", "SOFTMAX", "RESHAPE", "VIEW", "SLICE",
                                                 "GATHER_ROWS", "CONVERT"))
    for i in range(1, t.op_count):
        assert t.exec_table[i], f"exec entry {i} missing"


def test_exec_entries_reject_null_arguments(lib):
    t = ta.BcTables()
    lib.marmot_hip_bc_get_tables(C.byref(t))
    imm = (C.c_uint8 * 32)()
    for i in range(1, t.op_count):
        assert t.exec_table[i](None, None, imm, None) == ta.INVALID_ARGUMENT
    detail = C.c_char_p()
    assert lib.marmot_hip_backend_last_error(C.byref(detail)) == ta.INVALID_ARGUMENT
    assert b"Null bytecode exec arguments" in detail.value
    # impl functions with a null device context
    assert lib.hip_matmul_quantized_q4_k(None, None, None, None, None) == ta.INVALID_ARGUMENT
    assert lib.hip_moe_experts_impl(None, None) == ta.INVALID_ARGUMENT
    assert lib.hip_matmul_qkv_q4_k(None, None) == ta.INVALID_ARGUMENT
    assert lib.hip_topk_impl(None, None) == ta.INVALID_ARGUMENT
    assert lib.hip_embedding_gather(None, None) == ta.INVALID_ARGUMENT
    assert lib.hip_paged_attention_impl(None, None) == ta.INVALID_ARGUMENT


def test_program_encoding_matches_reference_immediates():
    import numpy as np
    x = ta.HostTensor.dense(np.zeros((2, 256), np.float32))
    w = ta.HostTensor.quantized(np.zeros(4 * 144, np.uint8), (4, 256), ta.KIND_Q4_K)
    y = ta.HostTensor.empty((2, 4), ta.DTYPE_F32)
    b = ta.HostTensor.dense(np.zeros(4, np.float32))
    p = ta.Program()
    p.matmul(3, x, w, y)
    assert bytes(p.code) == struct.pack("<HHHHIH", 3, 0, 1, 0xFFFF, 0xFFFFFFFF, 2)
    p.matmul(3, x, w, y, bias=b)
    op, ri, rw, rb, off, ro = struct.unpack_from("<HHHHIH", p.code, 14)
    assert (op, ri, rw, rb, ro) == (3, 0, 1, 3, 2) and off == 0 and len(p.const_pool) == C.sizeof(ta.Epilogue)
    assert len(p.regs) == 4
    # QKV: seven tensor registers (absent biases 0xFFFF), epilogue and rope offsets, three outputs
    q = ta.Program()
    outs = [ta.HostTensor.empty((2, 4), ta.DTYPE_F32) for _ in range(3)]
    q.qkv(14, x, w, w, w, *outs, bk=b)
    assert bytes(q.code) == struct.pack("<H7HII3H", 14, 0, 1, 1, 1, 0xFFFF, 2, 0xFFFF, 0xFFFFFFFF, 0xFFFFFFFF, 3, 4, 5)
    rp = ta.RopeParams()
    rp.theta, rp.apply_to_q = 10000.0, True
    q.qkv(14, x, w, w, w, *outs, rope=rp)
    assert struct.unpack_from("<I", q.code, 30 + 2 + 14 + 4)[0] == 0 and len(q.const_pool) == C.sizeof(ta.RopeParams)
    # ROPE: input, output, positions register (absent: the tensor the parameters name), offset, n_past, n_rot
    r = ta.Program()
    r.rope(53, x, y, rp)
    assert bytes(r.code) == struct.pack("<HHHHIII", 53, 0, 1, 0xFFFF, 0, 0, 0)
    r.rope(53, x, y, rp, positions=b, n_past=7, n_rot=64)
    assert struct.unpack_from("<HHHHIII", r.code, 20) == (53, 0, 1, 2, C.sizeof(ta.RopeParams), 7, 64)
    # EMBEDDING: table, ids, out; output dtype, scale, padding id, three flag bytes
    e = ta.Program()
    ids = ta.HostTensor.dense(np.zeros((2, 3), np.int64))
    eo = ta.HostTensor.empty((2, 3, 256), ta.DTYPE_F16)
    e.embedding(18, w, ids, eo, scale=0.5, padding_id=-1, bounds_check=True)
    assert bytes(e.code) == struct.pack("<H3HIfI3B", 18, 0, 1, 2, ta.DTYPE_F16, 0.5, 0xFFFFFFFF, 1, 0, 1)
    # tensor strides are row-major element strides, as marmot_tensor_create fills them
    assert list(x.t.shape.strides[:2]) == [256, 1] and x.t.shape.ndim == 2


def test_kernel_def_files_name_exported_impls(lib):
    ddir = os.path.join(ROOT, "marmot_amd", "kernels_def")
    families = {}
    for fn in sorted(os.listdir(ddir)):
        text = open(os.path.join(ddir, fn)).read()
        for name, body in re.findall(r"KERNEL_FAMILY\((\w+)\)\s*\{(.*?)\n\}", text, re.S):
            fields = dict(re.findall(r"^\s*([A-Z_]+(?:\(\w+\))?):\s*(.+?),?\s*$", body, re.M))
            families[name] = fields
    qkv = {f"{op}_quantized_hip_{dt}" for op in ("qkv_shared_input", "qkv_projection") for dt in ("f16", "f32")}
    assert set(families) == {"matmul_quantized_hip", "topk_hip",
                             "moe_experts_quantized_hip", "quantize_block_hip", "dequantize_block_hip",
                             "embedding_quantized_hip", "rms_norm_hip", "rms_norm_gemma_hip", "glu_hip",
                             "add_hip", "rope_hip", "paged_attention_hip", "unary_hip", "softmax_hip",
                             "tensor_ops_hip", "convert_hip"} | qkv
    for name in qkv:
        f = families[name]
        assert f["INPUT_DTYPE"] == f["OUTPUT_DTYPE"] and f["EPILOGUE"] == "[BIAS, ROPE]" and f["OP"] in name
    for name, f in families.items():
        impl = f["IMPL_FUNCTION"].strip('"')
        schemes = re.findall(r"Q\d_[01K]", f.get("AXIS(scheme)", "")) or [""]
        ops = re.findall(r"\w+", f.get("AXIS(op)", "")) or [""]
        for s in schemes:
            for o in ops:
                sym = impl.replace("{scheme:lower}", s.lower()).replace("{op}", o)
                assert hasattr(lib, sym), f"{name}: {sym} not exported"
        assert f["PLATFORM"] == "HIP" and f["PROFILE"] == ("NONE" if f["OP"] == "embedding" else "ANY")
    mm = families["matmul_quantized_hip"]
    assert mm["OP"] == "matmul" and mm["MATMUL_LAYOUT"] == "NT" and mm["WEIGHT_LAYOUT"] == "SEPARATE"
    assert mm["EPILOGUE"] == "[BIAS]" and mm["ACCUM_DTYPE"] == "FLOAT32" and mm["STRIDE_MODE"] == "CONTIGUOUS"
    assert mm["AXIS(scheme)"] == "[Q4_0, Q4_1, Q5_0, Q5_1, Q8_0, Q8_1, Q2_K, Q3_K, Q4_K, Q5_K, Q6_K]"
    assert mm["INPUT_DTYPE"] == "[FLOAT16, FLOAT32]"
