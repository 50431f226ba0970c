"""CPU: the oracle's RMS normalization and gated products pinned against the reference's own golden vectors and test
values, and against what the mathematics fixes (closed forms, scaling laws, float64 evaluation)."""
import numpy as np

from tests.util import gaussian

# tests/backend/golden_data.h:503-518 (g_rmsnorm): 2 x 4 input, weight, eps, expected
RMSNORM_INPUT = np.array([[0.5, -1, 2, -4], [1.5, -3, 6, -2]], dtype=np.float32)
RMSNORM_WEIGHT = np.array([0.5, 1, 1.5, 2], dtype=np.float32)
RMSNORM_EXPECTED = np.array([[0.1084651268, -0.4338605073, 1.301581522, -3.470884058],
                             [0.209529007, -0.8381160279, 2.514348084, -1.117488037]], dtype=np.float32)
# tests/backend/test_backend_elementwise.c:47-75 (check_glu_float32): gate, up; expected = act(gate) * up at 1e-6
GLU_GATE = np.array([-1.0, -0.25, 0.0, 0.75, 1.5], dtype=np.float32)
GLU_UP = np.array([0.5, -1.25, 2.0, -0.25, 0.75], dtype=np.float32)


def test_rms_norm_reference_golden(oracle):
    got = oracle.rms_norm(RMSNORM_INPUT, RMSNORM_WEIGHT, eps=1e-5)
    assert np.max(np.abs(got - RMSNORM_EXPECTED)) <= 1e-6  # the reference's own tolerance class for this vector


def test_rms_norm_closed_forms(oracle):
    # a constant row c: mean square c^2, out = c / sqrt(c^2 + eps) * w, one rounding chain that float64 reproduces
    for c, eps in ((3.0, 1e-5), (-0.125, 1e-6), (0.75, 0.0)):  # c * c * k is exact in fp32 for k <= 64
        x = np.full((1, 64), c, dtype=np.float32)
        w = np.linspace(0.5, 2.0, 64, dtype=np.float32)
        got = oracle.rms_norm(x, w, eps=eps)
        inv = np.float32(1.0) / np.sqrt(np.float32(np.float32(c) * np.float32(c)) + np.float32(eps), dtype=np.float32)
        want = (np.float32(c) * inv) * w
        assert np.array_equal(got[0], want.astype(np.float32)), (c, eps)
    # without weight the output has unit mean square (up to eps); the Gemma offset adds one to the weight
    x = gaussian(700, (5, 2048))
    y = oracle.rms_norm(x, eps=0.0)
    assert np.allclose(np.mean(y.astype(np.float64) ** 2, axis=1), 1.0, rtol=1e-5)
    w = gaussian(701, (2048,), 0.1)
    assert np.array_equal(oracle.rms_norm(x, w, weight_offset=1.0), oracle.rms_norm(x, (w + np.float32(1.0)).astype(np.float32)))
    # residual: the same as normalizing the fp32 sum
    r = gaussian(702, (5, 2048))
    assert np.array_equal(oracle.rms_norm(x, w, residual=r), oracle.rms_norm((x + r).astype(np.float32), w))
    # scale invariance with eps = 0: rms_norm(2^k x) == rms_norm(x) exactly (powers of two commute with rounding)
    assert np.array_equal(oracle.rms_norm(x * np.float32(8.0), w, eps=0.0), oracle.rms_norm(x, w, eps=0.0))
    # float64 evaluation of the definition
    v = (x + r).astype(np.float64)
    want = v / np.sqrt(np.mean(v * v, axis=1, keepdims=True) + 1e-5) * w.astype(np.float64)
    assert np.allclose(oracle.rms_norm(x, w, residual=r, eps=1e-5), want, rtol=2e-6, atol=1e-7)
    # a dropped eps, a mean over the wrong count or a missing square root would fail the golden vector above


def test_glu_reference_values_and_closed_forms(oracle):
    g64, u64 = GLU_GATE.astype(np.float64), GLU_UP.astype(np.float64)
    silu = g64 / (1.0 + np.exp(-g64))
    gelu = 0.5 * g64 * (1.0 + np.tanh(0.7978845608028654 * (g64 + 0.044715 * g64 ** 3)))
    assert np.max(np.abs(oracle.glu(GLU_GATE, GLU_UP) - silu * u64)) <= 1e-6
    assert np.max(np.abs(oracle.glu(GLU_GATE, GLU_UP, geglu=True) - gelu * u64)) <= 1e-6
    # silu(0) = 0, silu(x) -> x for large x, -> 0 for very negative x; gelu_tanh is odd-symmetric around x / 2
    big = np.array([0.0, 30.0, -30.0, 100.0, -100.0], dtype=np.float32)
    ones = np.ones_like(big)
    got = oracle.glu(big, ones)
    assert got[0] == 0.0 and got[1] == 30.0 and abs(got[2]) < 1e-11 and got[3] == 100.0 and got[4] == 0.0
    x = gaussian(710, (1000,), 2.0)
    a, b = oracle.glu(x, np.ones_like(x), geglu=True), oracle.glu(-x, np.ones_like(x), geglu=True)
    assert np.allclose(a.astype(np.float64) - b.astype(np.float64), x.astype(np.float64), rtol=0, atol=2e-6)
    # silu(x) - silu(-x) = x as well
    a, b = oracle.glu(x, np.ones_like(x)), oracle.glu(-x, np.ones_like(x))
    assert np.allclose(a.astype(np.float64) - b.astype(np.float64), x.astype(np.float64), rtol=0, atol=2e-6)
    # the MoE body's SwiGLU is the same expression
    u = gaussian(711, (1000,))
    assert np.array_equal(oracle.glu(x, u), oracle.moe_glu(x, u, 0))
