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


# ---------------------------------------------------------------- stand-alone rotary embedding
# The reference's own test (tests/backend/test_rope.c) builds its inputs and its expectation from closed forms:
# input[i] = sin(0.137 i) + 0.01 i over 2 x 5 x 8, position = seq_index + 0.125 (token % 3), freq_i = theta^(-2i/dim),
# a plane rotation of pair i by position * freq_i (:5-42, 64-70), tolerance 1e-5 for FLOAT32, 4e-3 for FLOAT16
# (:122-149), INT32 positions rounded with lrintf (:80-83), NEOX pairs (i, i + dim/2) (:181-184), zero positions are
# the identity (:186-234), two thetas give different results (:236-320). Evaluated here in float64.
def rope_test_inputs(batch=2, seq_len=5, dim=8):
    n = batch * seq_len * dim
    x = (np.sin(np.arange(n, dtype=np.float32) * np.float32(0.137), dtype=np.float32)
         + np.float32(0.01) * np.arange(n, dtype=np.float32)).astype(np.float32).reshape(batch, seq_len, dim)
    token = np.arange(batch * seq_len)
    pos = ((token % seq_len).astype(np.float32) + np.float32(0.125) * (token % 3).astype(np.float32)).astype(np.float32)
    return x, pos.reshape(batch, seq_len)


def rope_closed_form(x, pos, theta, rope_type, freq_scale=1.0, attn=1.0):
    dim = x.shape[-1]
    half = dim // 2
    rows = x.astype(np.float64).reshape(-1, dim)
    ang = pos.astype(np.float64).reshape(-1, 1) * freq_scale * theta ** (-(2.0 * np.arange(half)) / dim)
    c, s = np.cos(ang) * attn, np.sin(ang) * attn
    out = np.empty_like(rows)
    if rope_type == 1:
        e, o = rows[:, :half], rows[:, half:]
        out[:, :half], out[:, half:] = e * c - o * s, e * s + o * c
    else:
        e, o = rows[:, 0::2], rows[:, 1::2]
        out[:, 0::2], out[:, 1::2] = e * c - o * s, e * s + o * c
    return out.reshape(x.shape)


def test_rope_reference_test_cases(oracle):
    from oracle.pyoracle import RopeParams
    x, pos = rope_test_inputs()
    for dtype, tol in ((np.float32, 1e-5), (np.float16, 4e-3)):
        for rope_type in (0, 1):
            st, got = oracle.rope(x.astype(dtype), pos, RopeParams.default(theta=10000.0, rope_type=rope_type))
            assert st == 0 and got.dtype == dtype
            want = rope_closed_form(x.astype(dtype), pos, 10000.0, rope_type)
            assert np.max(np.abs(got.astype(np.float64) - want)) <= tol, (dtype, rope_type)
    ipos = np.rint(pos).astype(np.int32)  # lrintf: ties to even
    for p in (ipos, ipos.astype(np.int64)):
        st, got = oracle.rope(x, p, RopeParams.default(theta=10000.0))
        assert st == 0 and np.max(np.abs(got - rope_closed_form(x, p, 10000.0, 0))) <= 1e-5
    # zero positions: the identity, bit for bit (cos 0 = 1, sin 0 = 0)
    y = np.cos(np.arange(32, dtype=np.float32) * np.float32(0.09), dtype=np.float32).reshape(1, 4, 8)
    st, got = oracle.rope(y, np.zeros((1, 4), np.float32), RopeParams.default(theta=10000.0))
    assert st == 0 and np.array_equal(got, y)
    # two bases: each matches its own closed form and they differ by more than 1e-4
    xa, pa = rope_test_inputs(1, 6, 16)
    pa = np.arange(6, dtype=np.float32).reshape(1, 6)
    outs = []
    for theta in (10000.0, 500000.0):
        st, got = oracle.rope(xa, pa, RopeParams.default(theta=theta))
        assert st == 0 and np.max(np.abs(got - rope_closed_form(xa, pa, theta, 0))) <= 1e-5
        outs.append(got)
    assert np.max(np.abs(outs[0] - outs[1])) > 1e-4


def test_rope_invariants_strides_and_errors(oracle):
    from oracle.pyoracle import RopeParams
    x = gaussian(760, (3, 7, 128))
    pos = np.arange(21, dtype=np.int32).reshape(3, 7) * 37
    for rope_type in (0, 1):
        rp = RopeParams.default(theta=500000.0, rope_type=rope_type)
        st, y = oracle.rope(x, pos, rp)
        assert st == 0
        # a rotation keeps the norm of every pair; with an attention factor every pair is scaled by it
        pairs = (lambda v: np.stack([v[..., :64], v[..., 64:]], -1)) if rope_type == 1 else \
            (lambda v: v.reshape(v.shape[:-1] + (64, 2)))
        nx, ny = np.linalg.norm(pairs(x.astype(np.float64)), axis=-1), np.linalg.norm(pairs(y.astype(np.float64)), axis=-1)
        assert np.allclose(nx, ny, rtol=1e-5, atol=1e-6)
        # rotating back by the negated positions restores the rows
        st, back = oracle.rope(y, -pos, rp)
        assert st == 0 and np.max(np.abs(back - x)) <= 1e-5
        # the same rows as the Q/K/V epilogue's rotation with one head of the full width
        f, a = oracle.rope_frequencies(rp, 128)
        row = oracle.rope_rotate_row(x[1, 3], 128, float(pos[1, 3]), f, a, rope_type)
        assert np.array_equal(row, y[1, 3])
        # linear scaling and an attention factor enter through the frequencies and the scale
        rs = RopeParams.default(theta=500000.0, rope_type=rope_type, scaling_type=1, freq_scale=0.25, attn_factor=1.5)
        st, ys = oracle.rope(x, pos, rs)
        want = rope_closed_form(x, pos, 500000.0, rope_type, freq_scale=0.25, attn=1.5)
        assert st == 0 and np.max(np.abs(ys - want)) <= 3e-4  # angles up to 740 * 0.25 rad in fp32
    # head_dim of the parameters plays no part: the frequencies are those of the last dimension
    st, y1 = oracle.rope(x, pos, RopeParams.default(theta=500000.0, head_dim=64))
    st2, y2 = oracle.rope(x, pos, RopeParams.default(theta=500000.0))
    assert st == 0 and st2 == 0 and np.array_equal(y1, y2)
    # row strides: rows 160 apart in, 144 apart out; the gaps of the output are not written
    flat = np.full(20 * 160 + 128, 7.0, np.float32)
    for r in range(21):
        flat[r * 160:r * 160 + 128] = x.reshape(21, 128)[r]
    st, out = oracle.rope(flat, pos.reshape(-1), RopeParams.default(theta=500000.0), dim=128, x_row_stride=160,
                          out_row_stride=144)
    assert st == 0
    for r in range(21):
        assert np.array_equal(out[r * 144:r * 144 + 128], y2.reshape(21, 128)[r])
        if r < 20:
            assert np.all(np.isnan(out[r * 144 + 128:(r + 1) * 144]))
    # errors in the reference's order: odd dimension, empty input, stride shorter than a row
    assert oracle.rope(np.zeros((2, 7), np.float32), np.zeros(2, np.float32), RopeParams.default())[0] == -7
    assert oracle.rope(np.zeros((0, 8), np.float32), np.zeros(0, np.float32), RopeParams.default())[0] == -1
    assert oracle.rope(np.zeros(64, np.float32), np.zeros(2, np.float32), RopeParams.default(), dim=16, x_row_stride=8,
                       out_row_stride=16)[0] == -7
