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
