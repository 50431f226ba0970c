"""GPU parity, part 1: dequantizers and activation quantizers are bit-exact against the CPU oracle."""
import numpy as np
import pytest

from oracle.pyoracle import (BLOCK_BYTES, BLOCK_VALUES, KIND_Q8_1, KIND_Q2_K, KIND_Q3_K, KIND_Q4_0, KIND_Q4_1, KIND_Q5_0, KIND_Q5_1, KIND_Q4_K, KIND_Q5_K, KIND_Q6_K, KIND_Q8_0, KIND_Q8_K,
                             row_bytes)
from tests.util import bits, gaussian, quantize_weights, random_valid_blocks

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


def test_device_is_gfx950(hip):
    caps = hip.caps()
    print("device:", caps, flush=True)
    assert caps["arch"].startswith("gfx950")
    assert caps["wavefront_size"] == 64
    assert caps["num_compute_units"] >= 200


@pytest.mark.parametrize("name", ["q4_0", "q4_1", "q5_0", "q5_1", "q8_0", "q8_1", "q2_k", "q3_k", "q4_k", "q5_k", "q6_k"])
@pytest.mark.parametrize("rows,k", [(3, 1024), (2, 300), (1, 70), (64, 4096)])
def test_dequantize_bit_exact_quantized_gaussian(hip, oracle, name, rows, k):
    print(f"dequant {name} rows={rows} k={k}", flush=True)
    kind = KINDS[name]
    w = gaussian(200 + rows + k, (rows, k), 0.02)
    blocks = oracle.quantize(kind, w)
    exp = oracle.dequantize(kind, blocks, k)
    got = hip.dequantize(kind, blocks, k)
    assert np.array_equal(bits(got), bits(exp))


@pytest.mark.parametrize("name", ["q4_0", "q4_1", "q5_0", "q5_1", "q8_0", "q8_1", "q2_k", "q3_k", "q4_k", "q5_k", "q6_k"])
def test_dequantize_bit_exact_random_bytes(hip, oracle, name):
    """Every scale / nibble pattern, not only what a quantizer emits."""
    print(f"dequant random bytes {name}", flush=True)
    kind = KINDS[name]
    rng = np.random.default_rng(31)
    k = 16 * BLOCK_VALUES[kind]
    blocks = random_valid_blocks(rng, kind, 37, k)
    exp = oracle.dequantize(kind, blocks, k)
    got = hip.dequantize(kind, blocks, k)
    assert np.array_equal(bits(got), bits(exp))


def test_dequantize_q8_k_and_golden_blocks(hip, oracle, ref_goldens):
    x = gaussian(77, (2, 512))
    blocks = oracle.quantize(KIND_Q8_K, x)
    assert np.array_equal(bits(hip.dequantize(KIND_Q8_K, blocks, 512)), bits(oracle.dequantize(KIND_Q8_K, blocks, 512)))
    # the reference-held golden blocks: same tolerance as the reference's own test
    for name, tol in (("q4_0", 5e-4), ("q8_0", 5e-4), ("q4_k", 6e-4), ("q5_k", 6e-4), ("q6_k", 6e-4),
                      ("q4_1", 5e-4), ("q5_0", 5e-4), ("q5_1", 5e-4), ("q2_k", 6e-4), ("q3_k", 6e-4), ("q8_1", 5e-4)):
        exp = ref_goldens[f"g_llama_{name}_dequant"]
        got = hip.dequantize(KINDS[name], ref_goldens[f"g_llama_{name}"], exp.size)[0]
        assert np.max(np.abs(got - exp)) <= tol


@pytest.mark.parametrize("act_kind", [KIND_Q8_0, KIND_Q8_K])
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
# (300, 4000), (257, 4099) and (512, 4096): prompt-sized inputs, where a wavefront quantizes four blocks per launch slot
@pytest.mark.parametrize("rows,k", [(1, 2048), (5, 4096), (3, 300), (2, 70), (16, 14336), (300, 4000), (257, 4099),
                                    (512, 4096)])
def test_activation_quantizer_bit_exact(hip, oracle, act_kind, dtype, rows, k):
    print(f"act quant kind={act_kind} {np.dtype(dtype).name} rows={rows} k={k}", flush=True)
    x = gaussian(300 + rows * 7 + k, (rows, k)).astype(dtype)
    if rows > 1:
        x[1, : min(k, 256)] = 0  # an all-zero block
    x[0, 3] = -abs(x[0]).max() * 2  # the largest magnitude is negative
    if k > 40:
        x[0, 37] = -x[0, 3]  # same magnitude later in the block, opposite sign: first occurrence must win
    got = hip.quantize_activations(act_kind, x)
    exp = np.stack([oracle.pack(act_kind, x[r]) for r in range(rows)])
    assert got.shape == exp.shape
    assert np.array_equal(got, exp), f"{(got != exp).sum()} bytes differ"


def test_activation_quantizer_rounding_ties(hip, oracle):
    """Values that land exactly on .5 after scaling: Q8_0 rounds half away from zero, Q8_K half to even."""
    x = np.zeros((1, 256), dtype=np.float32)
    x[0, :32] = np.arange(32, dtype=np.float32) * 0.5
    x[0, 31] = 127.0  # scale = 1 -> values k/2 are exact ties
    x[0, 32:64] = -x[0, :32]
    x[0, 255] = -127.0
    for act_kind in (KIND_Q8_0, KIND_Q8_K):
        got = hip.quantize_activations(act_kind, x)
        exp = oracle.pack(act_kind, x[0])[None, :]
        assert np.array_equal(got, exp)


# ---------------------------------------------------------------- K-quant weight quantizers on the device
WEIGHT_QUANT_KINDS = {"q4_k": KIND_Q4_K, "q5_k": KIND_Q5_K, "q6_k": KIND_Q6_K}


@pytest.mark.parametrize("name", list(WEIGHT_QUANT_KINDS))
def test_weight_quantizer_reference_golden_and_reference_build(hip, name):
    """The reference's own golden blocks (its quantization test's 96-value pattern repeated to 256,
    test_backend_quantization.c:209-215) and the blocks its compiled quantizers wrote for Gaussian rows (fixture made
    by the reference build): the device writes the same bytes."""
    kind = WEIGHT_QUANT_KINDS[name]
    gold = np.load("tests/golden/reference_goldens.npz")
    src = gold["g_llama_test_input"]
    x = np.array([src[i % 96] for i in range(256)], dtype=np.float32)
    assert np.array_equal(hip.quantize_weights(kind, x)[0], gold[f"g_llama_{name}"])
    ref = np.load("tests/golden/ref_gaussian.npz")
    got = hip.quantize_weights(kind, ref[f"{name}_w"])
    assert np.array_equal(got, ref[f"{name}_blocks"]), f"{(got != ref[f'{name}_blocks']).sum()} bytes differ"


@pytest.mark.parametrize("name", list(WEIGHT_QUANT_KINDS))
def test_weight_quantizer_bit_exact(hip, oracle, name):
    """Byte equality with the CPU oracle: Gaussian weights at model scale, wide dynamic range, rows that are constant,
    all zero, all positive, all negative, tiny and huge, sub-blocks of zeros inside a live block, and a partial last
    block (the bytes beyond it are zeroed like the reference's)."""
    kind = WEIGHT_QUANT_KINDS[name]
    rng = np.random.default_rng(900 + kind)
    cases = [gaussian(901 + kind, (24, 1024), 0.02)]
    wide = gaussian(902 + kind, (8, 768)) * np.exp(rng.uniform(-12.0, 6.0, size=(8, 768))).astype(np.float32)
    cases.append(wide.astype(np.float32))
    special = np.zeros((10, 512), dtype=np.float32)
    special[0, :] = 0.37
    special[1, :] = 0.0
    special[2, :] = np.abs(gaussian(903, (512,)))
    special[3, :] = -np.abs(gaussian(904, (512,)))
    special[4, :] = gaussian(905, (512,)) * 1e-20
    special[5, :] = gaussian(906, (512,)) * 1e20
    special[6, :] = gaussian(907, (512,))
    special[6, 32:96] = 0.0            # zero sub-blocks inside a live block
    special[6, 256:272] = 0.0
    special[7, ::2] = 1.0              # two levels only
    special[8, 5] = 3.0                # one value, the rest zero
    special[9, :] = np.linspace(-1.0, 1.0, 512, dtype=np.float32)
    cases.append(special)
    cases.append(gaussian(908 + kind, (5, 300), 0.5))    # partial last block of 44 values
    cases.append(gaussian(909 + kind, (3, 70)))          # a single partial block
    for n, x in enumerate(cases):
        print(f"weight quantizer {name} case {n} shape {x.shape}", flush=True)
        got = hip.quantize_weights(kind, x)
        exp = oracle.quantize(kind, x)
        assert got.shape == exp.shape
        bad = np.argwhere(got != exp)
        assert bad.size == 0, f"{name} case {n}: {len(bad)} bytes differ, first at row {bad[0][0]} byte {bad[0][1]}"


def test_weight_quantizer_config_shapes(hip, oracle):
    """The decode configuration's own weights: N(0, 0.02) rows of 4096 and 14336 values through the device quantizer
    equal the oracle's blocks, and the quantized linear on them equals the one on the oracle's."""
    for name, k, rows in (("q4_k", 4096, 96), ("q6_k", 14336, 40)):
        kind = WEIGHT_QUANT_KINDS[name]
        w = gaussian(920 + k, (rows, k), 0.02)
        got = hip.quantize_weights(kind, w)
        assert np.array_equal(got, oracle.quantize(kind, w))
    with pytest.raises(Exception):
        hip.quantize_weights(KIND_Q4_0, gaussian(930, (2, 64)))
