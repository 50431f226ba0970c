"""GPU parity: marmot_matmul_qkv with separate quantized weights (one launch over q, k and v, activations quantized
once) against the CPU oracle, through the C ABI: every quant kind, the fused-quantization matvec (N <= 4), the packed
matvec, the small-batch MFMA route with and without K split, per-projection biases of either dtype, float16 in/out with
the op's single rounding, the reference's own test case, error codes."""
import ctypes as C

import numpy as np
import pytest

from marmot_amd import capi
from oracle.pyoracle import KIND_Q8_1, KIND_Q2_K, KIND_Q3_K, KIND_Q4_0, KIND_Q4_1, KIND_Q5_0, KIND_Q5_1, KIND_Q4_K, KIND_Q5_K, KIND_Q6_K, KIND_Q8_0
from tests.util import assert_matmul_parity, gaussian

pytestmark = pytest.mark.gpu

KINDS = {"q4_0": KIND_Q4_0, "q8_0": KIND_Q8_0, "q4_k": KIND_Q4_K, "q5_k": KIND_Q5_K, "q6_k": KIND_Q6_K,
         "q4_1": KIND_Q4_1, "q5_0": KIND_Q5_0, "q5_1": KIND_Q5_1, "q2_k": KIND_Q2_K, "q3_k": KIND_Q3_K,
         "q8_1": KIND_Q8_1}


@pytest.fixture(scope="module")
def hip():
    from marmot_amd import HipBackend

    b = HipBackend(0)
    yield b
    b.close()


def _weights(oracle, kind, M, K, seed):
    return [oracle.quantize(kind, gaussian(seed + i, (M, K), 0.02)) for i in range(3)]


@pytest.mark.parametrize("name", ["Q4_0", "Q4_1", "Q5_0", "Q5_1", "Q8_0", "Q8_1", "Q2_K", "Q3_K", "Q4_K", "Q5_K", "Q6_K"])
def test_reference_qkv_test_case(hip, ref_goldens, name):
    """tests/backend/test_backend_matmul.c:936-1032: the matmul golden weight as q, k and v."""
    kind, N, K, M = (int(v) for v in ref_goldens[f"matmul_{name}_dims"])
    w = ref_goldens[f"matmul_{name}_weight"]
    x = ref_goldens[f"matmul_{name}_input_f32"].reshape(N, K)
    exp = ref_goldens[f"matmul_{name}_expected_f32"].reshape(N, M)
    for out in hip.linear_qkv(x, w, w, w, kind, M):
        assert np.all(np.abs(out - exp) <= 2e-5 + 5e-5 * np.abs(exp)), np.abs(out - exp).max()


@pytest.mark.parametrize("name", ["q4_0", "q4_1", "q5_0", "q5_1", "q8_0", "q8_1", "q2_k", "q3_k", "q4_k", "q5_k", "q6_k"])
@pytest.mark.parametrize("N", [1, 2, 4, 5, 8, 16, 33])
def test_qkv_fp32_all_routes(hip, oracle, name, N):
    kind = KINDS[name]
    M, K = 32 * 5 + 7, 2048
    ws = _weights(oracle, kind, M, K, 600)
    x = gaussian(610 + N, (N, K))
    biases = [gaussian(620, (M,)), None, gaussian(621, (M,))]
    ref = oracle.matmul_qkv(kind, *ws, x, M, bq=biases[0], bv=biases[2])
    got = hip.linear_qkv(x, *ws, kind, M, bq=biases[0], bv=biases[2])
    route = hip.last_route()
    if name in ("q8_0", "q4_0") and N >= 9:  # three weights through the tiled int8 GEMM, K split across workgroups
        assert route == f"gemm_{name}_q8_0_mfma_tile", route
    for g, r, what in zip(got, ref, "qkv"):
        assert g.dtype == np.float32
        assert_matmul_parity(g, r, what=f"{name} N={N} {what} {route}")


@pytest.mark.parametrize("name", ["q4_k", "q6_k"])
@pytest.mark.parametrize("M,K", [(64, 14336), (4096, 4096)])
def test_qkv_split_k_and_model_shape(hip, oracle, name, M, K):
    """Few row groups and long rows (K split over workgroups, ordered reduction per projection) and the shape of a
    4096-wide attention block, at decode and at small-batch size."""
    kind = KINDS[name]
    ws = _weights(oracle, kind, M, K, 630)
    bias = [gaussian(640 + i, (M,)) for i in range(3)]
    for N in (1, 7):
        x = gaussian(650 + N, (N, K))
        ref = oracle.matmul_qkv(kind, *ws, x, M, bq=bias[0], bk=bias[1], bv=bias[2])
        got = hip.linear_qkv(x, *ws, kind, M, bq=bias[0], bk=bias[1], bv=bias[2])
        for g, r, what in zip(got, ref, "qkv"):
            assert_matmul_parity(g, r, what=f"{name} {M}x{K} N={N} {what} {hip.last_route()}")


@pytest.mark.parametrize("name", ["q8_0", "q2_k", "q3_k", "q4_k", "q5_k", "q6_k"])
@pytest.mark.parametrize("N", [1, 3, 9])
@pytest.mark.parametrize("bias_dtype", [np.float16, np.float32])
def test_qkv_fp16_in_out(hip, oracle, name, N, bias_dtype):
    """float16 activations are packed (no direct float16 route in this op); outputs are float16 of bias + dot with
    one rounding, so they may differ from the oracle by one float16 step where the fp32 sums differ in the last bits."""
    kind = KINDS[name]
    M, K = 96, 1024
    ws = _weights(oracle, kind, M, K, 660)
    x = gaussian(670 + N, (N, K)).astype(np.float16)
    bias = [gaussian(680 + i, (M,)).astype(bias_dtype) for i in range(3)]
    ref = oracle.matmul_qkv(kind, *ws, x, M, bq=bias[0], bk=bias[1], bv=bias[2])
    got = hip.linear_qkv(x, *ws, kind, M, bq=bias[0], bk=bias[1], bv=bias[2])
    for g, r in zip(got, ref):
        assert g.dtype == np.float16
        g32, r32 = g.astype(np.float32), r.astype(np.float32)
        assert np.max(np.abs(g32 - r32)) <= 1e-3 * np.abs(r32).max()
        assert np.mean(g.view(np.uint16) == r.view(np.uint16)) > 0.98


def test_qkv_error_codes(hip, oracle):
    kind, M, K = KIND_Q4_K, 32, 256
    w = oracle.quantize(kind, gaussian(690, (M, K), 0.02))
    d_w = hip.to_device(w)
    d_x = hip.to_device(gaussian(691, (1, K)))
    d_o = hip.alloc(M * 4)
    p = lambda b: C.c_void_p(b.ptr)
    none = C.c_void_p(None)
    try:
        call = lambda kind_, in_dt, out_dt, wq=p(d_w): hip.lib.marmot_hip_matmul_qkv_quantized(
            hip.dev, kind_, wq, p(d_w), p(d_w), p(d_x), in_dt, 1, K, M, none, none, none, 0, p(d_o), p(d_o), p(d_o),
            out_dt)
        assert call(kind, capi.DT_F32, capi.DT_F32) == 0
        # MARMOT_HIP_ERROR_NOT_IMPLEMENTED = -8, MARMOT_HIP_ERROR_INVALID_ARGUMENT = -1
        assert call(kind, capi.DT_F32, capi.DT_F16) == -8  # outputs must have the input dtype
        assert call(kind, 7, 7) == -8
        assert call(capi.KIND_Q8_K, capi.DT_F32, capi.DT_F32) == -8
        assert call(kind, capi.DT_F32, capi.DT_F32, wq=none) == -1
    finally:
        for b in (d_w, d_x, d_o):
            b.free()


# ---------------------------------------------------------------- rotary epilogue
@pytest.mark.parametrize("name", ["q8_0", "q2_k", "q3_k", "q4_k", "q5_k", "q6_k"])
@pytest.mark.parametrize("N", [1, 4, 6, 19])
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_qkv_rope_epilogue(hip, oracle, name, N, dtype):
    """q and/or k rotated in fp32 before the store, v untouched; NORM and NEOX pairs; int32, int64 and float32
    positions; a head dimension that splits the row into heads and one that does not divide it (whole row = one
    head, as cpu_matmul_qkv_resolve_head_dim decides)."""
    from oracle.pyoracle import RopeParams

    kind = KINDS[name]
    M, K = 256, 1024
    ws = _weights(oracle, kind, M, K, 700)
    x = gaussian(710 + N, (N, K)).astype(dtype)
    bias = [gaussian(720 + i, (M,)).astype(dtype) for i in range(3)]
    rng = np.random.default_rng(730 + N)
    cases = [
        (dict(head_dim=64, theta=500000.0), 0, True, True, rng.integers(0, 8192, N).astype(np.int32)),
        (dict(head_dim=128, theta=10000.0), 1, True, False, rng.integers(0, 4096, N).astype(np.int64)),
        (dict(head_dim=96, theta=10000.0, scaling_type=1, freq_scale=0.25, attn_factor=1.25), 1, False, True,
         (rng.random(N) * 100).astype(np.float32)),
    ]
    for kw, rope_type, aq, ak, pos in cases:
        rope = RopeParams.default(rope_type=rope_type, apply_to_q=int(aq), apply_to_k=int(ak), **kw)
        ref = oracle.matmul_qkv(kind, *ws, x, M, bq=bias[0], bk=bias[1], bv=bias[2], rope=rope, positions=pos)
        got = hip.linear_qkv(x, *ws, kind, M, bq=bias[0], bk=bias[1], bv=bias[2], positions=pos,
                             rope=dict(kw, rope_type=rope_type, apply_to_q=aq, apply_to_k=ak))
        for g, r, what in zip(got, ref, "qkv"):
            assert g.dtype == dtype
            g32, r32 = g.astype(np.float32), r.astype(np.float32)
            if dtype == np.float32:
                assert_matmul_parity(g32, r32, what=f"{name} N={N} rope case {kw} {what}")
            else:
                assert np.max(np.abs(g32 - r32)) <= 1e-3 * np.abs(r32).max()
                assert np.mean(g.view(np.uint16) == r.view(np.uint16)) > 0.97
    # the frequencies come from the host with the reference's formula: same bits as the oracle's
    f_hip, a_hip, hd = hip.rope_frequencies(M, head_dim=64, theta=500000.0)
    f_ref, a_ref = oracle.rope_frequencies(RopeParams.default(head_dim=64, theta=500000.0), 64)
    assert hd == 64 and a_hip == a_ref and np.array_equal(f_hip, f_ref)


def test_qkv_rope_errors(hip, oracle):
    kind, M, K = KIND_Q4_K, 64, 256
    ws = _weights(oracle, kind, M, K, 740)
    x = gaussian(741, (2, K))
    pos = np.array([1, 2], np.int32)
    # the YaRN ramp: frequencies and attention scale are the oracle's bits (host code, the reference's formulas)
    from oracle.pyoracle import RopeParams as RP
    yarn = dict(scaling_type=2, ext_factor=1.0, freq_scale=0.5, orig_ctx_len=4096, beta_fast=32.0, beta_slow=1.0)
    f_hip, a_hip, hd = hip.rope_frequencies(M, head_dim=64, theta=10000.0, **yarn)
    f_ref, a_ref = oracle.rope_frequencies(RP.default(head_dim=64, theta=10000.0, **yarn), 64)
    assert hd == 64 and a_hip == a_ref and np.array_equal(f_hip, f_ref) and a_ref > 1.0
    q, k_, _ = hip.linear_qkv(x, *ws, kind, M, positions=pos, rope=dict(theta=10000.0, head_dim=64, **yarn))
    rq, rk, _ = oracle.matmul_qkv(kind, *ws, x, M, positions=pos, rope=RP.default(theta=10000.0, head_dim=64, **yarn))
    assert_matmul_parity(q, rq, what="yarn q")
    assert_matmul_parity(k_, rk, what="yarn k")
    # YaRN parameters without an original context length degenerate to linear scaling (rope.c:85-93)
    q, _, _ = hip.linear_qkv(x, *ws, kind, M, positions=pos, rope=dict(scaling_type=2, ext_factor=1.0, freq_scale=0.5))
    from oracle.pyoracle import RopeParams
    rq, _, _ = oracle.matmul_qkv(kind, *ws, x, M, positions=pos,
                                 rope=RopeParams.default(scaling_type=2, ext_factor=1.0, freq_scale=0.5))
    assert_matmul_parity(q, rq, what="degenerate yarn")
    d = [hip.to_device(w) for w in ws] + [hip.to_device(x), hip.alloc(2 * M * 4)]
    try:
        bad = capi.Rope(None, capi.DT_I32, None, 1.0, 64, 0, 1, 1)
        st = hip.lib.marmot_hip_matmul_qkv_rope_quantized(
            hip.dev, kind, *[C.c_void_p(b.ptr) for b in d[:3]], C.c_void_p(d[3].ptr), capi.DT_F32, 2, K, M, None, None,
            None, 0, *[C.c_void_p(d[4].ptr)] * 3, capi.DT_F32, C.byref(bad))
        assert st == -1  # positions / frequencies missing
        bad = capi.Rope(d[3].ptr, capi.DT_I32, d[3].ptr, 1.0, 48, 0, 1, 1)
        st = hip.lib.marmot_hip_matmul_qkv_rope_quantized(
            hip.dev, kind, *[C.c_void_p(b.ptr) for b in d[:3]], C.c_void_p(d[3].ptr), capi.DT_F32, 2, K, M, None, None,
            None, 0, *[C.c_void_p(d[4].ptr)] * 3, capi.DT_F32, C.byref(bad))
        assert st == -1  # head dimension does not divide M
    finally:
        for b in d:
            b.free()
