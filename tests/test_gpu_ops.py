"""GPU parity: the fp32 operations between the quantized linears (RMS normalization, gated products, residual add) and
their fused forms that emit packed activations, against the CPU oracle and against the unfused chain on the GPU."""
import numpy as np
import pytest

from marmot_amd import capi
from oracle.pyoracle import KIND_Q4_K, KIND_Q6_K, KIND_Q8_0, KIND_Q8_K
from tests.test_oracle_ops import GLU_GATE, GLU_UP, RMSNORM_EXPECTED, RMSNORM_INPUT, RMSNORM_WEIGHT
from tests.util import assert_matmul_parity, assert_moe_parity, bits, gaussian

pytestmark = pytest.mark.gpu

# expf / tanhf are the device's (a few units in the last place), and the sum of squares of a row is added by 256
# threads as a tree where the scalar CPU loop adds sequentially: over n terms the sequential fp32 sum itself carries a
# relative error of about sqrt(n) * 2^-24 (5e-6 at 14336 columns), half of which reaches 1 / sqrt. Against float64
# the tree is the closer one (checked below).
OPS_RTOL = 1e-5


@pytest.fixture(scope="module")
def hip():
    from marmot_amd import HipBackend

    b = HipBackend(0)
    yield b
    b.close()


def same_packed(lay, rows, a, b):
    """The three arrays of two packed images agree (the alignment gaps between them are not written)."""
    return all(np.array_equal(a[lo:lo + n], b[lo:lo + n])
               for lo, n in ((lay.values_offset, rows * lay.values_per_row),
                             (lay.scales_offset, rows * lay.blocks_per_row * 4),
                             (lay.sums_offset, rows * lay.blocks_per_row * lay.sums_per_block * 2)))


def close(got, ref, what, rtol=OPS_RTOL, atol=1e-9):
    got64, ref64 = np.asarray(got, np.float64), np.asarray(ref, np.float64)
    err = np.abs(got64 - ref64) - (atol + rtol * np.abs(ref64))
    assert np.all(np.isfinite(got64)) and err.max() <= 0, f"{what}: {np.abs(got64 - ref64).max():.3e}"


def test_rms_norm_reference_golden_and_oracle(hip, oracle):
    assert np.max(np.abs(hip.rms_norm(RMSNORM_INPUT, RMSNORM_WEIGHT, eps=1e-5) - RMSNORM_EXPECTED)) <= 1e-6
    for rows, cols in ((1, 4096), (16, 4096), (3, 14336), (7, 1000), (2, 33), (64, 2048)):
        x = gaussian(720 + cols, (rows, cols))
        w = gaussian(721 + cols, (cols,), 0.5) + np.float32(1.0)
        r = gaussian(722 + cols, (rows, cols))
        close(hip.rms_norm(x, w), oracle.rms_norm(x, w), f"rms_norm {rows}x{cols}")
        close(hip.rms_norm(x, None, eps=1e-6), oracle.rms_norm(x, None, eps=1e-6), f"no weight {rows}x{cols}")
        close(hip.rms_norm(x, w, residual=r, weight_offset=1.0),
              oracle.rms_norm(x, w, residual=r, weight_offset=1.0), f"residual + gemma {rows}x{cols}")
    # against the definition in float64 the GPU result is at least as close as the sequential fp32 loop
    x, w = gaussian(725, (4, 14336)), gaussian(726, (14336,), 0.5) + np.float32(1.0)
    v = x.astype(np.float64)
    exact = v / np.sqrt(np.mean(v * v, axis=1, keepdims=True) + 1e-5) * w.astype(np.float64)
    err_gpu = np.abs(hip.rms_norm(x, w) - exact).max()
    err_cpu = np.abs(oracle.rms_norm(x, w) - exact).max()
    assert err_gpu <= err_cpu + 1e-7, (err_gpu, err_cpu)
    assert hip.rms_norm(np.zeros((0, 16), np.float32)).shape == (0, 16)  # no work


@pytest.mark.parametrize("kind", [KIND_Q4_K, KIND_Q8_0])
def test_rms_norm_pack_equals_unfused_chain(hip, oracle, kind):
    """The fused kernel's packed rows are the bits that packing its own fp32 output gives (same arithmetic), its fp32
    output is the unfused kernel's, and a linear on the packed rows agrees with the oracle's whole chain."""
    for rows, cols, M in ((1, 4096, 64), (16, 4096, 96), (5, 1000, 40), (3, 14336, 32)):
        if kind == KIND_Q4_K and cols % 256 != 0:
            continue
        x = gaussian(730 + cols, (rows, cols))
        w = gaussian(731 + cols, (cols,), 0.5) + np.float32(1.0)
        r = gaussian(732 + cols, (rows, cols))
        plain = hip.rms_norm(x, w, residual=r)
        out, image = hip.rms_norm(x, w, residual=r, pack_for_kind=kind)
        assert np.array_equal(bits(out), bits(plain))
        lay = hip.packed_activation_layout(kind, rows, cols)
        only, image2 = hip.rms_norm(x, w, residual=r, pack_for_kind=kind, want_f32=False)
        assert only is None and same_packed(lay, rows, image, image2)
        d_plain = hip.to_device(plain)
        d_p = hip.alloc(hip.packed_activation_bytes(kind, rows, cols))
        hip.pack_activations_d(kind, d_plain, capi.DT_F32, rows, cols, d_p)
        unfused = d_p.download(np.uint8, (lay.total_bytes,))
        assert same_packed(lay, rows, image, unfused), (rows, cols)
        # linear on the packed rows against the oracle: rms_norm -> quantize -> matmul
        blocks = oracle.quantize(kind, gaussian(733 + cols, (M, cols), 0.02))
        d_w, d_out = hip.to_device(blocks), hip.alloc(rows * M * 4)
        d_p.upload(image)
        hip.linear_prepacked_d(kind, d_w, d_p, rows, cols, M, d_out)
        got = d_out.download(np.float32, (rows, M))
        # the linear itself at the matmul bound, on the fp32 rows the GPU normalized (their packed bits are the input)
        assert_matmul_parity(got, oracle.matmul(kind, blocks, plain, M),
                             what=f"rms_norm_pack -> linear kind={kind} {rows}x{cols}")
        # the whole chain against the oracle's: a last-place difference of 1 / sqrt moves a few int8 codes of a long
        # row by one step, so the bound is taken against the output scale (as for the MoE re-quantization)
        ref = oracle.matmul(kind, blocks, oracle.rms_norm(x, w, residual=r), M)
        assert_moe_parity(got, ref, what=f"rms_norm -> quantize -> linear chain kind={kind} {rows}x{cols}")
        for b in (d_plain, d_p, d_w, d_out):
            b.free()


def test_glu_add_and_swiglu_pack(hip, oracle):
    g64, u64 = GLU_GATE.astype(np.float64), GLU_UP.astype(np.float64)
    silu = g64 / (1.0 + np.exp(-g64))
    gelu = 0.5 * g64 * (1.0 + np.tanh(0.7978845608028654 * (g64 + 0.044715 * g64 ** 3)))
    assert np.max(np.abs(hip.glu(GLU_GATE[None, :], GLU_UP[None, :])[0] - silu * u64)) <= 1e-6
    assert np.max(np.abs(hip.glu(GLU_GATE[None, :], GLU_UP[None, :], 2)[0] - gelu * u64)) <= 1e-6
    gate, up = gaussian(740, (16, 14336), 2.0), gaussian(741, (16, 14336))
    close(hip.glu(gate, up), oracle.glu(gate, up), "swiglu", atol=1e-7)
    close(hip.glu(gate, up, 2), oracle.glu(gate, up, geglu=True), "geglu", atol=1e-7)
    a, b = gaussian(742, (9, 777)), gaussian(743, (9, 777))
    assert np.array_equal(bits(hip.add(a, b)), bits((a + b).astype(np.float32)))
    # swiglu straight into packed activations == packing the fp32 product (same expression, same rounding)
    for kind in (KIND_Q6_K, KIND_Q8_0):
        rows, cols = 5, 2048
        image = hip.swiglu_pack(gate[:rows, :cols], up[:rows, :cols], kind)
        d_f = hip.to_device(hip.glu(gate[:rows, :cols], up[:rows, :cols]))
        d_p = hip.alloc(hip.packed_activation_bytes(kind, rows, cols))
        hip.pack_activations_d(kind, d_f, capi.DT_F32, rows, cols, d_p)
        lay = hip.packed_activation_layout(kind, rows, cols)
        unfused = d_p.download(np.uint8, (lay.total_bytes,))
        assert same_packed(lay, rows, image, unfused), kind
        d_f.free()
        d_p.free()


def test_ops_argument_errors(hip):
    d = hip.alloc(1024)
    lib, dev = hip.lib, hip.dev
    assert lib.marmot_hip_rms_norm(dev, None, None, None, 0.0, 1e-5, 1, 8, d.ptr) == -1
    assert lib.marmot_hip_rms_norm(dev, d.ptr, None, None, 0.0, 1e-5, 1, 8, None) == -1
    assert lib.marmot_hip_rms_norm_pack(dev, d.ptr, None, None, 0.0, 1e-5, 1, 8, KIND_Q4_K, None, d.ptr + 16) == -1
    assert lib.marmot_hip_rms_norm_pack(dev, d.ptr, None, None, 0.0, 1e-5, 1, 8, KIND_Q8_K, None, d.ptr) == -8
    assert lib.marmot_hip_glu(dev, 1, d.ptr, d.ptr, 1, 8, 8, 8, 8, d.ptr) == -8      # plain GELU FFN: not a gated product
    assert lib.marmot_hip_glu(dev, 0, d.ptr, d.ptr, 2, 8, 4, 8, 8, d.ptr) != 0       # stride shorter than a row
    assert lib.marmot_hip_add(dev, d.ptr, None, 4, d.ptr) == -1
    d.free()


# ---------------------------------------------------------------- stand-alone rotary embedding
# The device's sincosf and the C library's sinf / cosf agree to a few units in the last place of sin and cos, which
# reach a result as |x| * 2^-23 each; a FLOAT16 result can then round to the neighbouring half value.
def rope_close(got, ref, x, what):
    g, r = np.asarray(got, np.float64), np.asarray(ref, np.float64)
    scale = np.abs(np.asarray(x, np.float64)).max()
    tol = 2e-6 * scale if np.asarray(got).dtype == np.float32 else 1.1e-3 * np.maximum(np.abs(r), 1e-3)
    assert np.all(np.isfinite(g)) and np.all(np.abs(g - r) <= tol), f"{what}: {np.abs(g - r).max():.3e}"


def test_rope_reference_test_cases(hip, oracle):
    """The cases of the reference's own test (tests/backend/test_rope.c) at its tolerances."""
    from tests.test_oracle_ops import rope_closed_form, rope_test_inputs
    x, pos = rope_test_inputs()
    for dtype, tol in ((np.float32, 1e-5), (np.float16, 4e-3)):
        for rope_type in (0, 1):
            got = hip.rope(x.astype(dtype), pos, rope_type=rope_type, theta=10000.0)
            want = rope_closed_form(x.astype(dtype), pos, 10000.0, rope_type)
            assert got.dtype == dtype and np.max(np.abs(got.astype(np.float64) - want)) <= tol, (dtype, rope_type)
    ipos = np.rint(pos).astype(np.int32)
    for p in (ipos, ipos.astype(np.int64)):
        assert np.max(np.abs(hip.rope(x, p, theta=10000.0) - rope_closed_form(x, p, 10000.0, 0))) <= 1e-5
    y = np.cos(np.arange(32, dtype=np.float32) * np.float32(0.09), dtype=np.float32).reshape(1, 4, 8)
    assert np.array_equal(hip.rope(y, np.zeros((1, 4), np.float32), theta=10000.0), y)  # zero positions: identity


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_rope_matches_oracle(hip, oracle, dtype):
    from oracle.pyoracle import RopeParams
    x = gaussian(1200, (4, 33, 128)).astype(dtype)
    cases = [(dict(theta=500000.0), np.arange(132, dtype=np.int32).reshape(4, 33) * 61),
             (dict(theta=10000.0, scaling_type=1, freq_scale=0.25, attn_factor=1.5),
              (np.arange(132, dtype=np.int64).reshape(4, 33) * 997) % 8192),
             (dict(theta=10000.0, scaling_type=2, ext_factor=1.0, freq_scale=0.5, orig_ctx_len=4096, beta_fast=32.0,
                   beta_slow=1.0), gaussian(1201, (4, 33), 300.0))]
    for kw, pos in cases:
        for rope_type in (0, 1):
            st, ref = oracle.rope(x, pos, RopeParams.default(rope_type=rope_type, **kw))
            assert st == 0
            rope_close(hip.rope(x, pos, rope_type=rope_type, **kw), ref, x, f"{dtype.__name__} {kw} type {rope_type}")
    # in place, and an odd number of rows of a width that is not a multiple of the workgroup
    x2 = gaussian(1202, (7, 6)).astype(dtype)
    p2 = np.array([0, 1, 5, 17, 4096, 100000, 3], np.int32)
    st, ref = oracle.rope(x2, p2, RopeParams.default())
    rope_close(hip.rope(x2, p2, in_place=True), ref, x2, "in place")
    # row strides: input rows 160 apart, output rows 144 apart (even: paired accesses) and 145 / 131 apart (odd:
    # single-element accesses); the gaps of the output keep their contents
    rows = 21
    xr = gaussian(1203, (rows, 128)).astype(dtype)
    pr = (np.arange(rows, dtype=np.int32) * 37)
    for xs, os_ in ((160, 144), (145, 131)):
        flat = np.full((rows - 1) * xs + 128, 7.0, dtype)
        for r in range(rows):
            flat[r * xs:r * xs + 128] = xr[r]
        for rope_type in (0, 1):
            rp = RopeParams.default(theta=500000.0, rope_type=rope_type)
            st, ref = oracle.rope(flat, pr, rp, dim=128, x_row_stride=xs, out_row_stride=os_)
            got = hip.rope(flat, pr, rope_type=rope_type, theta=500000.0, dim=128, x_row_stride=xs, out_row_stride=os_)
            assert st == 0 and np.array_equal(np.isnan(got), np.isnan(ref))
            live = ~np.isnan(ref)
            rope_close(got[live], ref[live], xr, f"strides {xs}/{os_} type {rope_type}")


def test_rope_prefill_shape_and_invariants(hip, oracle):
    """512 tokens x 32 heads x 128: the q rows of a prefill step, rotated in one launch; against the oracle on a slice
    and through what a rotation fixes on the whole (pair norms kept, the inverse rotation restores the rows)."""
    from oracle.pyoracle import RopeParams
    T, Hh, D = 512, 32, 128
    x = gaussian(1210, (T, Hh, D))
    pos = np.repeat(np.arange(T, dtype=np.int32)[:, None] + 1000, Hh, axis=1)
    for rope_type in (0, 1):
        y = hip.rope(x, pos, rope_type=rope_type, theta=500000.0)
        st, ref = oracle.rope(x[:16], pos[:16], RopeParams.default(theta=500000.0, rope_type=rope_type))
        rope_close(y[:16], ref, x, f"prefill type {rope_type}")
        pairs = (lambda v: np.stack([v[..., :D // 2], v[..., D // 2:]], -1)) if rope_type == 1 else \
            (lambda v: v.reshape(v.shape[:-1] + (D // 2, 2)))
        nx = np.linalg.norm(pairs(x.astype(np.float64)), axis=-1)
        ny = np.linalg.norm(pairs(y.astype(np.float64)), axis=-1)
        assert np.allclose(nx, ny, rtol=1e-5, atol=1e-6)
        back = hip.rope(y, -pos, rope_type=rope_type, theta=500000.0)
        assert np.max(np.abs(back - x)) <= 1e-5


def test_rope_argument_errors(hip):
    d = hip.to_device(np.zeros(1024, np.float32))
    lib, dev = hip.lib, hip.dev
    r = capi.Rope(d.ptr, capi.DT_I32, d.ptr, 1.0, 8, 0, 0, 0)
    import ctypes as C
    call = lambda *a: lib.marmot_hip_rope(dev, *a)
    assert call(C.c_void_p(d.ptr), capi.DT_F32, 2, 8, 8, 8, C.byref(r), C.c_void_p(d.ptr)) == 0
    assert call(None, capi.DT_F32, 2, 8, 8, 8, C.byref(r), C.c_void_p(d.ptr)) == -1
    assert call(C.c_void_p(d.ptr), capi.DT_F32, 2, 8, 8, 8, None, C.c_void_p(d.ptr)) == -1
    assert call(C.c_void_p(d.ptr), capi.DT_I32, 2, 8, 8, 8, C.byref(r), C.c_void_p(d.ptr)) == -6
    assert call(C.c_void_p(d.ptr), capi.DT_F32, 2, 7, 8, 8, C.byref(r), C.c_void_p(d.ptr)) == -7   # odd dimension
    assert call(C.c_void_p(d.ptr), capi.DT_F32, 0, 8, 8, 8, C.byref(r), C.c_void_p(d.ptr)) == -1   # empty
    assert call(C.c_void_p(d.ptr), capi.DT_F32, 2, 8, 6, 8, C.byref(r), C.c_void_p(d.ptr)) == -7   # stride < row
    assert call(C.c_void_p(d.ptr), capi.DT_F32, 2, 16, 16, 16, C.byref(r), C.c_void_p(d.ptr)) == -1  # 4 freqs for dim 16
    r.positions_dtype = capi.DT_F16
    assert call(C.c_void_p(d.ptr), capi.DT_F32, 2, 8, 8, 8, C.byref(r), C.c_void_p(d.ptr)) == -6
    r.positions_dtype, r.d_positions = capi.DT_I32, None
    assert call(C.c_void_p(d.ptr), capi.DT_F32, 2, 8, 8, 8, C.byref(r), C.c_void_p(d.ptr)) == -1
    hip.synchronize()
    d.free()
