"""CPU: the oracle's restatement of marmot_matmul_qkv with separate quantized weights
(src/backends/cpu/ops/matmul/qkv/matmul_qkv.c:749-947), pinned by
  * the reference's own test of this op (tests/backend/test_backend_matmul.c:936-1032): the matmul golden weight used
    for q, k and v, every output equal to the matmul golden (tolerance of the matmul golden test,
    tests/backend/test_matmul_quantized.c:166-177: the goldens come from another implementation's summation order);
  * the block dots and packers it is built from, which the vec-dot and quantization goldens pin separately: every
    output is recomputed here from oracle.pack / oracle.vec_dot with the accumulator started from the bias and ONE
    rounding at the store, including a float16 case in which the matmul epilogue's order (round, then add the bias)
    gives different bits."""
import numpy as np
import pytest

from oracle.pyoracle import BLOCK_BYTES, BLOCK_VALUES, KIND_Q4_0, KIND_Q4_K, KIND_Q6_K, KIND_Q8_0, KIND_Q8_K
from tests.util import bits, gaussian


@pytest.mark.parametrize("name", ["Q4_0", "Q8_0", "Q4_K", "Q6_K"])
def test_reference_qkv_test_case(oracle, ref_goldens, name):
    kind, N, K, M = (int(v) for v in ref_goldens[f"matmul_{name}_dims"])
    w = ref_goldens[f"matmul_{name}_weight"]
    x = ref_goldens[f"matmul_{name}_input_f32"].reshape(N, K)
    exp = ref_goldens[f"matmul_{name}_expected_f32"].reshape(N, M)
    for out in oracle.matmul_qkv(kind, w, w, w, x, M):
        assert out.dtype == np.float32
        assert np.all(np.abs(out - exp) <= 2e-5 + 5e-5 * np.abs(exp)), np.abs(out - exp).max()


def _expected(oracle, kind, weights, x, M, biases):
    """bias + whole-row block dot, recomputed per element from the pinned leaf functions."""
    N, K = x.shape
    act_kind = KIND_Q8_K if BLOCK_VALUES[kind] == 256 else KIND_Q8_0
    nb = (K + BLOCK_VALUES[kind] - 1) // BLOCK_VALUES[kind]
    rb = nb * BLOCK_BYTES[kind]
    outs = [np.zeros((N, M), dtype=np.float32) for _ in range(3)]
    for n in range(N):
        act = oracle.pack(act_kind, x[n])
        for i, (w, b) in enumerate(zip(weights, biases)):
            w = np.ascontiguousarray(w, dtype=np.uint8).reshape(M, rb)
            for m in range(M):
                acc = np.float32(0.0) if b is None else np.float32(b[m])
                outs[i][n, m] = np.float32(acc + np.float32(oracle.vec_dot(kind, w[m], act, nb)))
    return outs


@pytest.mark.parametrize("kind,K", [(KIND_Q4_K, 70 * 256), (KIND_Q6_K, 512), (KIND_Q8_0, 96), (KIND_Q4_0, 160)])
def test_qkv_fp32_is_bias_plus_whole_row_dot(oracle, kind, K):
    """K = 70 blocks: the q/k/v op dots the whole row in one call, it does not chunk K by 64 blocks as the matmul
    driver does (matmul_qkv.c:902-914 against matmul_quant_compute.c:1032-1112)."""
    M, N = 6, 3
    ws = [oracle.quantize(kind, gaussian(500 + i, (M, K), 0.02)) for i in range(3)]
    x = gaussian(510, (N, K))
    bq, bv = gaussian(511, (M,)), gaussian(512, (M,)).astype(np.float16)
    q, k, v = oracle.matmul_qkv(kind, *ws, x, M, bq=bq)
    eq, ek, ev = _expected(oracle, kind, ws, x, M, [bq, None, None])
    assert np.array_equal(bits(q), bits(eq)) and np.array_equal(bits(k), bits(ek)) and np.array_equal(bits(v), bits(ev))
    # float16 bias values are widened exactly before they start the accumulator
    _, _, v16 = oracle.matmul_qkv(kind, *ws, x, M, bv=bv)
    _, _, ev16 = _expected(oracle, kind, ws, x, M, [None, None, bv.astype(np.float32)])
    assert np.array_equal(bits(v16), bits(ev16))
    # without bias and within one 64-block chunk each projection is the plain quantized matmul
    if K // BLOCK_VALUES[kind] <= 64:
        for w, out in zip(ws, oracle.matmul_qkv(kind, *ws, x, M)):
            assert np.array_equal(bits(out), bits(oracle.matmul(kind, w, x, M)))


def test_qkv_fp16_packs_the_activations_and_rounds_once(oracle):
    kind, M, K, N = KIND_Q4_K, 64, 512, 4
    ws = [oracle.quantize(kind, gaussian(520 + i, (M, K), 0.02)) for i in range(3)]
    x = gaussian(523, (N, K)).astype(np.float16)
    bias = [gaussian(524 + i, (M,)).astype(np.float16) for i in range(3)]
    outs = oracle.matmul_qkv(kind, *ws, x, M, bq=bias[0], bk=bias[1], bv=bias[2])
    exp32 = _expected(oracle, kind, ws, x, M, [b.astype(np.float32) for b in bias])
    differs = 0
    for out, e32, w, b in zip(outs, exp32, ws, bias):
        assert out.dtype == np.float16
        assert np.array_equal(out.view(np.uint16), e32.astype(np.float16).view(np.uint16))
        # the matmul epilogue's order on the same packed dot: round to float16, then add the bias in float16
        mm = oracle.matmul(kind, w, x, M, bias=b.astype(np.float32), out_dtype=np.float16, force_pack=True)
        differs += int(np.count_nonzero(mm.view(np.uint16) != out.view(np.uint16)))
    assert differs > 0  # the two rounding orders are distinguishable on this input


def test_qkv_rejects_other_input_types(oracle):
    kind, M, K = KIND_Q8_0, 4, 64
    w = oracle.quantize(kind, gaussian(530, (M, K), 0.02))
    import ctypes as C
    from oracle.pyoracle import DT_F32

    arr = C.c_void_p * 3
    x = gaussian(531, (1, K))
    outs = [np.zeros((1, M), dtype=np.float32) for _ in range(3)]
    st = oracle.L.mo_matmul_qkv_separate(kind, arr(*[w.ctypes.data] * 3), x.ctypes.data, 99, 1, K, M,
                                         arr(None, None, None), DT_F32, arr(*[o.ctypes.data for o in outs]))
    assert st == -8  # MARMOT_ERROR_NOT_IMPLEMENTED (matmul_qkv.c:761-763)


# ---------------------------------------------------------------- rotary epilogue
# Pinned by the closed form the reference's own rope test uses as its expectation (tests/backend/test_rope.c:5-42:
# freq_i = theta^(-2i/dim), angle = position * freq_i, a plane rotation of each pair), evaluated here in float64,
# and by what the mathematics fixes: rotations preserve the norm of every pair, position 0 is the identity,
# rotating by p then by -p restores the row, NORM and NEOX are the same rotation under a permutation of the columns.

def _rope_f64(row, head_dim, pos, theta, rope_type, freq_scale=1.0, attn=1.0):
    row = row.astype(np.float64).copy()
    half = head_dim // 2
    i = np.arange(half, dtype=np.float64)
    ang = pos * freq_scale * theta ** (-(2.0 * i) / head_dim)
    c, s = np.cos(ang) * attn, np.sin(ang) * attn
    for h in range(row.shape[0] // head_dim):
        seg = row[h * head_dim:(h + 1) * head_dim]
        if rope_type == 1:
            e, o = seg[:half].copy(), seg[half:].copy()
            seg[:half], seg[half:] = e * c - o * s, e * s + o * c
        else:
            e, o = seg[0::2].copy(), seg[1::2].copy()
            seg[0::2], seg[1::2] = e * c - o * s, e * s + o * c
    return row


def test_rope_frequencies_and_rotation_closed_form(oracle):
    from oracle.pyoracle import ROPE_SCALING_LINEAR, ROPE_SCALING_YARN, RopeParams

    for head_dim, theta in ((64, 10000.0), (128, 500000.0)):
        f, a = oracle.rope_frequencies(RopeParams.default(theta=theta), head_dim)
        want = theta ** (-(2.0 * np.arange(head_dim // 2)) / head_dim)
        assert a == 1.0 and np.allclose(f, want, rtol=2e-6, atol=0) and f[0] == 1.0
        # without a scaling type the scale factors are ignored; linear scaling multiplies every frequency
        f2, _ = oracle.rope_frequencies(RopeParams.default(theta=theta, freq_scale=0.25), head_dim)
        assert np.array_equal(f2, f)
        f3, a3 = oracle.rope_frequencies(
            RopeParams.default(theta=theta, freq_scale=0.25, attn_factor=1.5, scaling_type=ROPE_SCALING_LINEAR), head_dim)
        assert np.array_equal(f3, f * np.float32(0.25)) and a3 == 1.5
    # YaRN (rope.c:28-59, 95-126). Known correction range for 128 dims, 4096 original context, base 10000,
    # beta_fast 32, beta_slow 1: pairs 0..20 keep their frequency (ramp 1 up to floor(20.9)), pairs from 46 = ceil(45.04)
    # on are interpolated by freq_scale (ramp 0), linear in between; attention scale attn_factor * (1 + 0.1 ln(1/s)).
    yarn = RopeParams.default(theta=10000.0, scaling_type=ROPE_SCALING_YARN, ext_factor=1.0, freq_scale=0.25,
                              attn_factor=1.0, orig_ctx_len=4096, beta_fast=32.0, beta_slow=1.0)
    f, a = oracle.rope_frequencies(yarn, 128)
    base = (10000.0 ** (-(2.0 * np.arange(64)) / 128)).astype(np.float64)
    d, lo, hi = 128, 4096 / (32 * 2 * np.pi), 4096 / (1 * 2 * np.pi)
    low = max(0.0, np.floor(d * np.log(lo) / (2 * np.log(10000.0))))
    high = min(d - 1.0, np.ceil(d * np.log(hi) / (2 * np.log(10000.0))))
    assert (low, high) == (20.0, 46.0)
    ramp = 1.0 - np.clip((np.arange(64) - low) / (high - low), 0.0, 1.0)
    want = base * (0.25 + ramp * (1.0 - 0.25))
    assert np.allclose(f, want, rtol=3e-6, atol=0)
    assert np.allclose(f[:21], base[:21], rtol=3e-6) and np.allclose(f[46:], base[46:] * 0.25, rtol=3e-6)
    assert abs(a - (1.0 + 0.1 * np.log(4.0))) < 1e-6
    # half the extrapolation factor mixes half-way; no original context length degenerates to linear scaling
    half = RopeParams.default(theta=10000.0, scaling_type=ROPE_SCALING_YARN, ext_factor=0.5, freq_scale=0.25,
                              orig_ctx_len=4096, beta_fast=32.0, beta_slow=1.0)
    f_half, _ = oracle.rope_frequencies(half, 128)
    assert np.allclose(f_half, base * (0.25 + 0.5 * ramp * 0.75), rtol=3e-6, atol=0)
    lin = RopeParams.default(theta=10000.0, scaling_type=ROPE_SCALING_YARN, ext_factor=1.0, freq_scale=0.25)
    f_lin, a_lin = oracle.rope_frequencies(lin, 128)
    assert np.allclose(f_lin, base * 0.25, rtol=3e-6, atol=0) and a_lin == 1.0
    assert oracle.L.mo_rope_resolve_head_dim(512, 128) == 128
    for bad in (0, 1024, 96, 7):  # absent, larger than the row, not a divisor, odd
        assert oracle.L.mo_rope_resolve_head_dim(512, bad) == 512

    rng = np.random.default_rng(540)
    row = rng.standard_normal(256).astype(np.float32)
    for rope_type in (0, 1):
        for head_dim in (64, 256):
            f, a = oracle.rope_frequencies(RopeParams.default(), head_dim)
            for pos in (0.0, 1.0, 37.0, 4095.0):
                got = oracle.rope_rotate_row(row, head_dim, pos, f, a, rope_type)
                want = _rope_f64(row, head_dim, pos, 10000.0, rope_type)
                # fp32 frequencies and angles: the angle is off by up to ~2^-23 * position radians
                assert np.max(np.abs(got - want)) <= (1e-6 + 1.5e-7 * pos) * np.abs(row).max()
                if pos == 0.0:
                    assert np.array_equal(got, row)
                # pair norms are preserved
                pairs = (lambda v: v.reshape(-1, 2, head_dim // 2).transpose(0, 2, 1)) if rope_type == 1 else \
                    (lambda v: v.reshape(-1, head_dim // 2, 2))
                assert np.allclose(np.linalg.norm(pairs(got), axis=-1), np.linalg.norm(pairs(row), axis=-1), rtol=1e-5)
                back = oracle.rope_rotate_row(got, head_dim, -pos, f, a, rope_type)
                assert np.allclose(back, row, atol=1e-5)
    # NEOX = NORM on columns permuted (2i, 2i+1) -> (i, i + half)
    head_dim = 64
    f, a = oracle.rope_frequencies(RopeParams.default(), head_dim)
    perm = np.concatenate([np.arange(0, head_dim, 2), np.arange(1, head_dim, 2)])
    full = np.concatenate([perm + h * head_dim for h in range(4)])
    norm = oracle.rope_rotate_row(row, head_dim, 11.0, f, a, 0)
    neox = oracle.rope_rotate_row(row[full], head_dim, 11.0, f, a, 1)
    assert np.array_equal(neox, norm[full])


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_qkv_rope_epilogue_is_projection_then_rotation(oracle, dtype):
    from oracle.pyoracle import RopeParams

    kind, M, K, N = KIND_Q4_K, 128, 512, 5
    ws = [oracle.quantize(kind, gaussian(550 + i, (M, K), 0.02)) for i in range(3)]
    x = gaussian(553, (N, K)).astype(dtype)
    bias = [gaussian(554 + i, (M,)).astype(dtype) for i in range(3)]
    plain = _expected(oracle, kind, ws, x, M, [b.astype(np.float32) for b in bias])  # fp32, before any rounding
    for pos in (np.array([0, 1, 2, 3, 900], np.int32), np.array([5, 4, 3, 2, 1], np.int64),
                np.array([0.5, 7.0, 8.0, 9.0, 10.0], np.float32)):
        for rope_type in (0, 1):
            for aq, ak in ((1, 1), (1, 0), (0, 1), (0, 0)):
                rope = RopeParams.default(head_dim=64, rope_type=rope_type, apply_to_q=aq, apply_to_k=ak,
                                          theta=500000.0)
                q, k, v = oracle.matmul_qkv(kind, *ws, x, M, bq=bias[0], bk=bias[1], bv=bias[2], rope=rope,
                                            positions=pos)
                f, a = oracle.rope_frequencies(rope, 64)
                for out, base, rot in ((q, plain[0], aq), (k, plain[1], ak), (v, plain[2], 0)):
                    want = base.copy()
                    if rot:
                        for n in range(N):
                            want[n] = oracle.rope_rotate_row(base[n], 64, float(np.float32(pos[n])), f, a, rope_type)
                    assert out.dtype == dtype
                    assert np.array_equal(bits(out), bits(want.astype(dtype)))  # one rounding, after the rotation
