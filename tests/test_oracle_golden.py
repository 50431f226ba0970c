"""Pins the CPU oracle (oracle/marmot_oracle.c) before anything trusts it.

Three independent anchors:
  1. the golden vectors the reference's own tests hold (tests/backend/golden_quant_llama.h,
     golden_vec_dot_llama.h, golden_matmul_llama.h), transcribed into reference_goldens.npz;
  2. outputs of the reference's own leaf code (scalar build) on seeded Gaussian rows
     (ref_gaussian.npz, and live against oracle/_ref where it is built);
  3. what the arithmetic fixes: float64 brute force of the block dots, closed forms of the
     dequantizers written independently in numpy, invariants of the packers.
"""
import numpy as np
import pytest

from oracle.pyoracle import (BLOCK_BYTES, BLOCK_VALUES, KIND_Q2_K, KIND_Q3_K, KIND_Q4_0, KIND_Q4_1, KIND_Q4_K, KIND_Q5_0, KIND_Q5_1, KIND_Q5_K,
                             KIND_Q6_K, KIND_Q8_0, KIND_Q8_1, KIND_Q8_K,
                             row_bytes)

KINDS = {"q4_0": KIND_Q4_0, "q8_0": KIND_Q8_0, "q4_k": KIND_Q4_K, "q5_k": KIND_Q5_K, "q6_k": KIND_Q6_K,
         "q4_1": KIND_Q4_1, "q5_0": KIND_Q5_0, "q5_1": KIND_Q5_1, "q2_k": KIND_Q2_K, "q3_k": KIND_Q3_K,
         "q8_1": KIND_Q8_1}


def bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


# ---------------------------------------------------------------- independent numpy decoders
def np_dequant_q4_k(blocks: np.ndarray) -> np.ndarray:
    """Independent vectorised decoder of Q4_K blocks [nb,144] -> float64 [nb,256] (exact arithmetic)."""
    nb = blocks.shape[0]
    d = blocks[:, 0:2].copy().view(np.float16).astype(np.float64)[:, 0]
    dmin = blocks[:, 2:4].copy().view(np.float16).astype(np.float64)[:, 0]
    s = blocks[:, 4:16].astype(np.int64)
    sc = np.zeros((nb, 8), dtype=np.int64)
    mn = np.zeros((nb, 8), dtype=np.int64)
    for j in range(8):
        if j < 4:
            sc[:, j] = s[:, j] & 63
            mn[:, j] = s[:, j + 4] & 63
        else:
            sc[:, j] = (s[:, j + 4] & 0xF) | ((s[:, j - 4] >> 6) << 4)
            mn[:, j] = (s[:, j + 4] >> 4) | ((s[:, j] >> 6) << 4)
    qs = blocks[:, 16:144].astype(np.int64).reshape(nb, 4, 32)
    q = np.zeros((nb, 8, 32), dtype=np.int64)
    q[:, 0::2, :] = qs & 0xF
    q[:, 1::2, :] = qs >> 4
    y = (d[:, None, None] * sc[:, :, None]) * q - (dmin[:, None, None] * mn[:, :, None])
    return y.reshape(nb, 256), q.reshape(nb, 256), sc, mn, d, dmin


def np_q6_k_ints(blocks: np.ndarray):
    nb = blocks.shape[0]
    ql = blocks[:, 0:128].astype(np.int64).reshape(nb, 2, 64)
    qh = blocks[:, 128:192].astype(np.int64).reshape(nb, 2, 32)
    sc = blocks[:, 192:208].copy().view(np.int8).astype(np.int64)
    d = blocks[:, 208:210].copy().view(np.float16).astype(np.float64)[:, 0]
    q = np.zeros((nb, 2, 4, 32), dtype=np.int64)
    q[:, :, 0, :] = (ql[:, :, 0:32] & 0xF) | (((qh >> 0) & 3) << 4)
    q[:, :, 1, :] = (ql[:, :, 32:64] & 0xF) | (((qh >> 2) & 3) << 4)
    q[:, :, 2, :] = (ql[:, :, 0:32] >> 4) | (((qh >> 4) & 3) << 4)
    q[:, :, 3, :] = (ql[:, :, 32:64] >> 4) | (((qh >> 6) & 3) << 4)
    q = q.reshape(nb, 256) - 32
    return q, sc, d


# ---------------------------------------------------------------- 1. reference-held goldens
@pytest.mark.parametrize("name", ["q4_0", "q8_0", "q4_k", "q5_k", "q6_k", "q4_1", "q5_0", "q5_1", "q2_k", "q3_k", "q8_1"])
def test_quantizer_bytes_match_reference_golden(oracle, ref_goldens, name):
    kind = KINDS[name]
    src = ref_goldens["g_llama_test_input"]
    if BLOCK_VALUES[kind] == 256:
        x = np.array([src[i % 96] for i in range(256)], dtype=np.float32)  # test_backend_quantization.c:209-215
    else:
        x = src
    got = oracle.quantize(kind, x)[0]
    exp = ref_goldens[f"g_llama_{name}"]
    assert got.size == exp.size
    assert np.array_equal(got, exp), f"{name}: {(got != exp).sum()} bytes differ"


def test_q8_k_bytes_match_reference_golden(oracle, ref_goldens):
    src = ref_goldens["g_llama_test_input"]
    x = np.array([src[i % 96] for i in range(256)], dtype=np.float32)
    got = oracle.pack(KIND_Q8_K, x)
    assert np.array_equal(got, ref_goldens["g_llama_q8_k"])
    assert np.array_equal(oracle.quantize(KIND_Q8_K, x)[0], ref_goldens["g_llama_q8_k"])


@pytest.mark.parametrize("name,tol", [("q4_0", 5e-4), ("q8_0", 5e-4), ("q4_k", 6e-4), ("q5_k", 6e-4), ("q6_k", 6e-4), ("q4_1", 5e-4), ("q5_0", 5e-4),
                                      ("q5_1", 5e-4), ("q2_k", 6e-4), ("q3_k", 6e-4), ("q8_1", 5e-4)])
def test_dequant_matches_reference_golden(oracle, ref_goldens, name, tol):
    kind = KINDS[name]
    exp = ref_goldens[f"g_llama_{name}_dequant"]
    got = oracle.dequantize(kind, ref_goldens[f"g_llama_{name}"], exp.size)[0]
    # the reference's own tolerance for these llama.cpp floats (test_backend_quantization.c:107-339);
    # observed error is at the 1e-9 print precision of the header
    assert np.max(np.abs(got - exp)) <= tol
    assert np.max(np.abs(got - exp)) <= 1e-6 * max(1.0, np.max(np.abs(exp)))


@pytest.mark.parametrize("name", ["q4_0", "q8_0", "q4_k", "q5_k", "q6_k", "q4_1", "q5_0", "q5_1", "q2_k", "q3_k", "q8_1"])
def test_vec_dot_matches_reference_golden(oracle, ref_goldens, name):
    kind = KINDS[name]
    act = ref_goldens["g_vec_dot_q8_k_activations" if BLOCK_VALUES[kind] == 256 else "g_vec_dot_q8_0_activations"]
    w = ref_goldens[f"g_vec_dot_{name}_weights"]
    nb = 256 // BLOCK_VALUES[kind]
    got = oracle.vec_dot(kind, w, act, nb)
    exp = float(ref_goldens[f"g_vec_dot_{name}_q8_{'k' if nb == 1 else '0'}_expected"][0])
    assert abs(got - exp) <= 1e-5 + 2e-5 * abs(exp)  # tests/backend/test_vec_dot.c:134-165


def test_activation_packers_match_reference_golden(oracle, ref_goldens):
    x = ref_goldens["g_vec_dot_test_vec2"]
    got_k = oracle.pack(KIND_Q8_K, x)
    exp_k = ref_goldens["g_vec_dot_q8_k_activations"]
    # int8 values and the 16 group sums are exact; the fp32 scale in this llama.cpp-made golden is one ulp away
    # from 1/(-127/max) evaluated in IEEE fp32 (which is what the reference's own packer computes: see the
    # *_equals_reference_code_* tests and g_llama_q8_k above, both byte-exact)
    assert np.array_equal(got_k[4:], exp_k[4:])
    assert abs(int(got_k[:4].view(np.uint32)[0]) - int(exp_k[:4].view(np.uint32)[0])) <= 1
    got = oracle.pack(KIND_Q8_0, x)
    exp = ref_goldens["g_vec_dot_q8_0_activations"]
    # ggml rounds ties to even, the scalar reference build rounds ties away from zero: allow +-1 on exact ties only
    g = got.reshape(8, 34)
    e = exp.reshape(8, 34)
    assert np.array_equal(g[:, :2], e[:, :2])  # fp16 scales
    dq = g[:, 2:].view(np.int8).astype(int) - e[:, 2:].view(np.int8).astype(int)
    scale = g[:, :2].copy().view(np.float16).astype(np.float32)
    inv = 1.0 / (np.abs(x.reshape(8, 32)).max(axis=1) / np.float32(127.0))
    frac = np.abs(x.reshape(8, 32) * inv[:, None].astype(np.float32))
    ties = np.isclose(frac - np.floor(frac), 0.5, atol=1e-4)
    assert np.all((dq == 0) | ties), "Q8_0 packer differs from golden away from rounding ties"
    assert scale.shape == (8, 1)


@pytest.mark.parametrize("name", ["Q4_0", "Q8_0", "Q4_K", "Q5_K", "Q6_K", "Q4_1", "Q5_0", "Q5_1", "Q2_K", "Q3_K", "Q8_1"])
@pytest.mark.parametrize("fp16_input", [False, True])
def test_matmul_matches_reference_golden(oracle, ref_goldens, name, fp16_input):
    kind, N, K, M = (int(v) for v in ref_goldens[f"matmul_{name}_dims"])
    w = ref_goldens[f"matmul_{name}_weight"]
    if fp16_input:
        x = ref_goldens[f"matmul_{name}_input_f16"].view(np.float16).reshape(N, K)
        exp = ref_goldens[f"matmul_{name}_expected_f16"].reshape(N, M)
    else:
        x = ref_goldens[f"matmul_{name}_input_f32"].reshape(N, K)
        exp = ref_goldens[f"matmul_{name}_expected_f32"].reshape(N, M)
    # Q6_K with fp16 activations: the golden is a snapshot of the reference's own cpu_vec_dot_q6_k_f16
    # (vec_dot_impl.h:1082-1128), whose index pattern differs from its Q6_K dequantizer; the oracle restates it
    # as written and therefore matches the snapshot.
    got = oracle.matmul(kind, w, x, M)
    # the reference's own tolerance (tests/backend/test_matmul_quantized.c:166-177)
    assert np.all(np.abs(got - exp) <= 2e-5 + 5e-5 * np.abs(exp)), (got, exp)


# ---------------------------------------------------------------- 2. reference leaf code on Gaussian rows
@pytest.mark.parametrize("name", ["q4_0", "q8_0", "q4_k", "q5_k", "q6_k", "q4_1", "q5_0", "q5_1", "q2_k", "q3_k", "q8_1"])
def test_oracle_equals_reference_code_on_gaussian_fixture(oracle, ref_gaussian, name):
    kind = KINDS[name]
    g = ref_gaussian
    K = g[f"{name}_w"].shape[1]
    blocks = oracle.quantize(kind, g[f"{name}_w"])
    assert np.array_equal(blocks, g[f"{name}_blocks"]), "quantizer bytes differ from the reference's code"
    deq = oracle.dequantize(kind, g[f"{name}_blocks"], K)
    assert np.array_equal(bits(deq), bits(g[f"{name}_dequant"])), "dequantizer not bit-exact"
    act_kind = KIND_Q8_K if BLOCK_VALUES[kind] == 256 else KIND_Q8_0
    assert np.array_equal(oracle.pack(act_kind, g[f"{name}_x"]), g[f"{name}_act"])
    assert np.array_equal(oracle.pack(act_kind, g[f"{name}_x"].astype(np.float16)), g[f"{name}_act_from_f16"])
    nb = K // BLOCK_VALUES[kind]
    dots = np.array([oracle.vec_dot(kind, g[f"{name}_blocks"][r], g[f"{name}_act"], nb)
                     for r in range(blocks.shape[0])], dtype=np.float32)
    assert np.array_equal(bits(dots), bits(g[f"{name}_dots"]))
    dots16 = np.array([oracle.vec_dot_f16(kind, g[f"{name}_blocks"][r], g[f"{name}_x"].astype(np.float16), K)
                       for r in range(blocks.shape[0])], dtype=np.float32)
    assert np.array_equal(bits(dots16), bits(g[f"{name}_dots_f16"]))
    # ragged K (zero-padded tail blocks)
    k = g[f"{name}_tail_w"].shape[1]
    assert np.array_equal(oracle.quantize(kind, g[f"{name}_tail_w"]), g[f"{name}_tail_blocks"])
    assert np.array_equal(bits(oracle.dequantize(kind, g[f"{name}_tail_blocks"], k)), bits(g[f"{name}_tail_dequant"]))
    assert np.array_equal(oracle.pack(act_kind, g[f"{name}_tail_x"]), g[f"{name}_tail_act"])


@pytest.mark.parametrize("name", ["q4_0", "q8_0", "q4_k", "q5_k", "q6_k", "q4_1", "q5_0", "q5_1", "q2_k", "q3_k", "q8_1"])
@pytest.mark.parametrize("seed,scale", [(7, 0.02), (42, 1.0), (123, 30.0), (1337, 1e-4)])
def test_oracle_equals_reference_code_live(oracle, reflib, name, seed, scale):
    kind = KINDS[name]
    rng = np.random.default_rng(seed)
    K = 768
    w = (rng.standard_normal((6, K)) * scale).astype(np.float32)
    blocks = oracle.quantize(kind, w)
    assert np.array_equal(blocks, reflib.quantize(kind, w))
    assert np.array_equal(bits(oracle.dequantize(kind, blocks, K)), bits(reflib.dequantize(kind, blocks, K)))
    x = rng.standard_normal(K).astype(np.float32) * (1.0 if seed != 123 else 50.0)
    act_kind = KIND_Q8_K if BLOCK_VALUES[kind] == 256 else KIND_Q8_0
    act = oracle.pack(act_kind, x)
    assert np.array_equal(act, reflib.pack(act_kind, x))
    nb = K // BLOCK_VALUES[kind]
    for r in range(6):
        assert oracle.vec_dot(kind, blocks[r], act, nb) == reflib.vec_dot(kind, blocks[r], act, nb)
        assert oracle.vec_dot_f16(kind, blocks[r], x.astype(np.float16), K) == \
            reflib.vec_dot_f16(kind, blocks[r], x.astype(np.float16), K)


def test_random_bytes_dequant_equals_reference_code_live(oracle, reflib):
    """Arbitrary block bytes (not produced by a quantizer): every 6-bit scale / nibble pattern."""
    rng = np.random.default_rng(5)
    for name, kind in KINDS.items():
        nb = 64
        raw = rng.integers(0, 256, size=(1, nb * BLOCK_BYTES[kind]), dtype=np.uint8)
        # keep the fp16 scale fields finite
        blk = raw.reshape(nb, BLOCK_BYTES[kind])
        for off in {"q4_0": [0], "q8_0": [0], "q4_k": [0, 2], "q5_k": [0, 2], "q6_k": [208], "q4_1": [0, 2], "q5_0": [0],
                    "q5_1": [0, 2], "q2_k": [80, 82], "q3_k": [108], "q8_1": [0, 2]}[name]:
            h = blk[:, off:off + 2].copy().view(np.uint16)
            h &= 0xBBFF  # clear the top exponent bit: |value| < 2
            blk[:, off:off + 2] = h.view(np.uint8)
        k = nb * BLOCK_VALUES[kind]
        assert np.array_equal(bits(oracle.dequantize(kind, raw, k)), bits(reflib.dequantize(kind, raw, k)))


# ---------------------------------------------------------------- 3. what the arithmetic fixes
def test_fp16_conversions_exhaustive(oracle):
    hs = np.arange(65536, dtype=np.uint16)
    exp = hs.view(np.float16).astype(np.float32)
    got = np.array([oracle.f16_to_f32(int(h)) for h in hs], dtype=np.float32)
    ok = (bits(got) == bits(exp)) | (np.isnan(got) & np.isnan(exp))
    assert ok.all()
    finite = np.isfinite(exp)
    back = np.array([oracle.f32_to_f16(float(v)) for v in exp[finite]], dtype=np.uint16)
    assert np.array_equal(back, hs[finite])
    rng = np.random.default_rng(3)
    xs = np.concatenate([rng.standard_normal(4000).astype(np.float32) * np.float32(s)
                         for s in (1e-8, 6e-8, 1e-5, 1e-3, 1.0, 100.0, 65000.0)])
    # add exact ties between adjacent halves
    h = rng.integers(1, 0x7bff, size=2000).astype(np.uint16)
    lo = h.view(np.float16).astype(np.float64)
    hi = (h + 1).astype(np.uint16).view(np.float16).astype(np.float64)
    xs = np.concatenate([xs, ((lo + hi) / 2).astype(np.float32)])
    with np.errstate(over="ignore"):
        exp16 = xs.astype(np.float16).view(np.uint16)
    got16 = np.array([oracle.f32_to_f16(float(v)) for v in xs], dtype=np.uint16)
    assert np.array_equal(got16, exp16)


def test_q4_k_dequant_closed_form_and_dot_brute_force(oracle):
    rng = np.random.default_rng(11)
    K = 2048
    w = (rng.standard_normal((8, K)) * 0.02).astype(np.float32)
    blocks = oracle.quantize(KIND_Q4_K, w)
    blk = blocks.reshape(-1, 144)
    y64, q, sc, mn, d, dmin = np_dequant_q4_k(blk)
    deq = oracle.dequantize(KIND_Q4_K, blocks, K).reshape(-1, 256)
    # fp32 evaluation with the reference's op order, written independently in numpy (each op rounds to fp32)
    d32, m32 = d.astype(np.float32), dmin.astype(np.float32)
    d1 = (d32[:, None] * sc.astype(np.float32)).astype(np.float32)
    m1 = (m32[:, None] * mn.astype(np.float32)).astype(np.float32)
    exp = (np.repeat(d1, 32, axis=1) * q.astype(np.float32)).astype(np.float32) - np.repeat(m1, 32, axis=1)
    assert np.array_equal(bits(deq), bits(exp.astype(np.float32)))
    assert np.max(np.abs(deq - y64)) < 1e-6
    # quantization error is bounded by half a step of the coarsest sub-block (sanity that bytes mean what we think)
    assert np.max(np.abs(deq.reshape(8, K) - w)) < 0.02
    # block dot vs float64 brute force on the dequantized values
    x = rng.standard_normal(K).astype(np.float32)
    act = oracle.pack(KIND_Q8_K, x)
    a = act.reshape(-1, 292)
    ad = a[:, 0:4].copy().view(np.float32)[:, 0].astype(np.float64)
    aq = a[:, 4:260].copy().view(np.int8).astype(np.float64)
    xq = (ad[:, None] * aq).reshape(-1)
    for r in range(8):
        got = oracle.vec_dot(KIND_Q4_K, blocks[r], act, K // 256)
        brute = float(np.dot(y64.reshape(8, K)[r], xq))
        assert abs(got - brute) <= 2e-6 * np.sum(np.abs(y64.reshape(8, K)[r] * xq)) + 1e-7


def test_q6_k_dequant_closed_form_and_dot_brute_force(oracle):
    rng = np.random.default_rng(12)
    K = 2048
    w = (rng.standard_normal((8, K)) * 0.02).astype(np.float32)
    blocks = oracle.quantize(KIND_Q6_K, w)
    q, sc, d = np_q6_k_ints(blocks.reshape(-1, 210))
    deq = oracle.dequantize(KIND_Q6_K, blocks, K).reshape(-1, 256)
    ds = (d.astype(np.float32)[:, None] * sc.astype(np.float32)).astype(np.float32)  # (d*sc) first
    exp = (np.repeat(ds, 16, axis=1) * q.astype(np.float32)).astype(np.float32)
    assert np.array_equal(bits(deq), bits(exp))
    assert np.max(np.abs(deq.reshape(8, K) - w)) < 0.005
    x = rng.standard_normal(K).astype(np.float32)
    act = oracle.pack(KIND_Q8_K, x)
    a = act.reshape(-1, 292)
    ad = a[:, 0:4].copy().view(np.float32)[:, 0].astype(np.float64)
    aq = a[:, 4:260].copy().view(np.int8).astype(np.float64)
    xq = (ad[:, None] * aq).reshape(-1)
    y64 = (d[:, None] * np.repeat(sc, 16, axis=1) * q).reshape(8, K)
    for r in range(8):
        got = oracle.vec_dot(KIND_Q6_K, blocks[r], act, K // 256)
        brute = float(np.dot(y64[r], xq))
        assert abs(got - brute) <= 2e-6 * np.sum(np.abs(y64[r] * xq)) + 1e-7


def test_q8_0_and_q4_0_closed_forms(oracle):
    rng = np.random.default_rng(13)
    K = 512
    w = (rng.standard_normal((4, K)) * 0.02).astype(np.float32)
    b8 = oracle.quantize(KIND_Q8_0, w).reshape(-1, 34)
    sc = b8[:, :2].copy().view(np.float16).astype(np.float32)[:, 0]
    q = b8[:, 2:].copy().view(np.int8).astype(np.float32)
    exp = (q * sc[:, None]).astype(np.float32)
    assert np.array_equal(bits(oracle.dequantize(KIND_Q8_0, b8.reshape(4, -1), K).reshape(-1, 32)), bits(exp))
    # amax maps to +-127 and the scale is amax/127 rounded to fp16
    amax = np.abs(w.reshape(-1, 32)).max(axis=1)
    assert np.array_equal(sc, (amax / np.float32(127.0)).astype(np.float16).astype(np.float32))
    assert np.all(np.abs(q).max(axis=1) == 127)
    b4 = oracle.quantize(KIND_Q4_0, w).reshape(-1, 18)
    s4 = b4[:, :2].copy().view(np.float16).astype(np.float32)[:, 0]
    lo = (b4[:, 2:] & 0xF).astype(np.float32) - 8
    hi = (b4[:, 2:] >> 4).astype(np.float32) - 8
    exp4 = np.concatenate([lo, hi], axis=1) * s4[:, None]
    assert np.array_equal(bits(oracle.dequantize(KIND_Q4_0, b4.reshape(4, -1), K).reshape(-1, 32)), bits(exp4))
    x = rng.standard_normal(K).astype(np.float32)
    act = oracle.pack(KIND_Q8_0, x).reshape(-1, 34)
    asc = act[:, :2].copy().view(np.float16).astype(np.float64)[:, 0]
    aq = act[:, 2:].copy().view(np.int8).astype(np.float64)
    xq = (aq * asc[:, None]).reshape(-1)
    for r in range(4):
        got = oracle.vec_dot(KIND_Q8_0, b8.reshape(4, -1)[r], act.reshape(-1), K // 32)
        brute = float(np.dot(exp.astype(np.float64).reshape(4, K)[r], xq))
        assert abs(got - brute) <= 2e-6 * np.sum(np.abs(exp.reshape(4, K)[r] * xq)) + 1e-7
        got4 = oracle.vec_dot(KIND_Q4_0, b4.reshape(4, -1)[r], act.reshape(-1), K // 32)
        brute4 = float(np.dot(exp4.astype(np.float64).reshape(4, K)[r], xq))
        assert abs(got4 - brute4) <= 2e-6 * np.sum(np.abs(exp4.reshape(4, K)[r] * xq)) + 1e-7


def test_q8_k_packer_invariants(oracle):
    rng = np.random.default_rng(14)
    x = rng.standard_normal(1024).astype(np.float32)
    x[256:512] = 0.0  # an all-zero block
    x[512] = -9.0  # block whose max-magnitude value is negative
    blk = oracle.pack(KIND_Q8_K, x).reshape(4, 292)
    d = blk[:, :4].copy().view(np.float32)[:, 0]
    q = blk[:, 4:260].copy().view(np.int8).astype(int)
    bs = blk[:, 260:].copy().view(np.int16).astype(int)
    assert np.array_equal(bs, q.reshape(4, 16, 16).sum(axis=2))
    assert d[1] == 0.0 and not q[1].any() and not bs[1].any()
    for b in (0, 2, 3):
        xb = x[b * 256:(b + 1) * 256]
        i = int(np.argmax(np.abs(xb)))
        assert q[b, i] == -127 and np.abs(q[b]).max() <= 127
        assert d[b] == np.float32(1.0) / (np.float32(-127.0) / xb[i])
        assert np.max(np.abs(q[b] * d[b] - xb)) <= abs(d[b]) * 0.5001


def test_matmul_driver_against_blockwise_dots(oracle):
    """The driver = packer + per-(row, col) block dot in chunks of 64 blocks, output [N, M], tiles of 16 columns."""
    rng = np.random.default_rng(15)
    for kind, K in ((KIND_Q4_K, 64 * 256 + 512), (KIND_Q8_0, 64 * 32 + 96), (KIND_Q6_K, 512)):
        M, N = 5, 19  # N > 16 crosses a column tile
        w = (rng.standard_normal((M, K)) * 0.02).astype(np.float32)
        blocks = oracle.quantize(kind, w)
        x = rng.standard_normal((N, K)).astype(np.float32)
        out = oracle.matmul(kind, blocks, x, M)
        act_kind = KIND_Q8_K if BLOCK_VALUES[kind] == 256 else KIND_Q8_0
        nb = K // BLOCK_VALUES[kind]
        bb, ab = BLOCK_BYTES[kind], BLOCK_BYTES[act_kind]
        for n in (0, 7, 16, 18):
            act = oracle.pack(act_kind, x[n])
            for m in range(M):
                acc = np.float32(0.0)
                for kb in range(0, nb, 64):
                    c = min(64, nb - kb)
                    acc = np.float32(acc + np.float32(
                        oracle.vec_dot(kind, blocks[m, kb * bb:(kb + c) * bb], act[kb * ab:(kb + c) * ab], c)))
                assert out[n, m] == acc
        # threads do not change any value
        assert np.array_equal(bits(out), bits(oracle.matmul(kind, blocks, x, M, threads=3)))
        # bias is added after the store
        bias = rng.standard_normal(M).astype(np.float32)
        assert np.array_equal(bits(oracle.matmul(kind, blocks, x, M, bias=bias)), bits(out + bias[None, :]))


def test_matmul_fp16_direct_and_forced_pack(oracle):
    rng = np.random.default_rng(16)
    K, M, N = 512, 6, 3
    w = (rng.standard_normal((M, K)) * 0.02).astype(np.float32)
    x = rng.standard_normal((N, K)).astype(np.float16)
    for kind in (KIND_Q4_K, KIND_Q8_0, KIND_Q4_0):
        blocks = oracle.quantize(kind, w)
        out = oracle.matmul(kind, blocks, x, M)
        deq = oracle.dequantize(kind, blocks, K).astype(np.float64)
        ref = x.astype(np.float64) @ deq.T
        assert np.max(np.abs(out - ref)) <= 1e-5 * np.max(np.abs(ref)) + 1e-6
        for n in range(N):
            for m in range(M):
                assert out[n, m] == np.float32(oracle.vec_dot_f16(kind, blocks[m], x[n], K))
        out16 = oracle.matmul(kind, blocks, x, M, out_dtype=np.float16)
        assert np.array_equal(out16, out.astype(np.float16))
        forced = oracle.matmul(kind, blocks, x, M, force_pack=True)
        assert np.array_equal(bits(forced), bits(oracle.matmul(kind, blocks, x.astype(np.float32), M)))
    with pytest.raises(RuntimeError):
        oracle.matmul(KIND_Q4_K, oracle.quantize(KIND_Q4_K, w), x.astype(np.float32), M, out_dtype=np.float16)


def test_row_grain_rule(oracle):
    # matmul_quant_compute.c:1222-1240
    assert oracle.row_grain(4096, 1, 1) == 512  # ceil(4096/8)=512
    assert oracle.row_grain(14336, 1, 8) == 224
    assert oracle.row_grain(14336, 4, 8) == 152  # ceil(14336/96)=150 -> 152
    assert oracle.row_grain(14336, 16, 8) == 64
    assert oracle.row_grain(100, 1, 4) == 64
    assert oracle.row_grain(10 ** 6, 1, 1) == 4096
