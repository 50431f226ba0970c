"""GPU parity: prefill GEMM for fp16 activations and every weight format other than Q4_K (whose kernels have their own
tests) against the CPU oracle's direct fp16 route (cpu_vec_dot_*_f16, vec_dot_impl.h: the decode patterns of the
reference's fp16 dots, which for Q2_K / Q3_K / Q5_K / Q6_K differ from its dequantizers), and against the fp16 matvec of
the same library, which multiplies the same decoded weights on the vector units."""
import numpy as np
import pytest

from oracle.pyoracle import KINDS
from tests.util import gaussian, parity_metrics, random_valid_blocks

pytestmark = pytest.mark.gpu
NAMES = ["q4_0", "q4_1", "q5_0", "q5_1", "q8_0", "q8_1", "q2_k", "q3_k", "q5_k", "q6_k"]


@pytest.fixture(scope="module")
def hip():
    from marmot_amd import HipBackend

    b = HipBackend(0)
    yield b
    b.close()


@pytest.fixture(scope="module")
def matvec(monkeypatch_module):
    from marmot_amd import HipBackend

    monkeypatch_module.setenv("MARMOT_HIP_NO_GEMM", "1")
    b = HipBackend(0)
    monkeypatch_module.delenv("MARMOT_HIP_NO_GEMM")
    yield b
    b.close()


@pytest.fixture(scope="module")
def monkeypatch_module():
    mp = pytest.MonkeyPatch()
    yield mp
    mp.undo()


def check(hip, oracle, name, blocks, x, M, what, bias=None, out_dtype=np.float32):
    kind = KINDS[name]
    got = hip.linear(x, blocks, kind, M, bias=bias, out_dtype=out_dtype)
    assert hip.last_route() == f"gemm_{name}_f16_mfma", (what, hip.last_route())
    ref = oracle.matmul(kind, blocks, x, M, bias=bias, out_dtype=out_dtype)
    g32, r32 = got.astype(np.float32), ref.astype(np.float32)
    assert np.all(np.isfinite(g32)), what
    m_floor, m_sum, m_max = parity_metrics(g32, r32)
    print(f"{what}: floored-rel {m_floor:.3e} sum-rel {m_sum:.3e} max-norm {m_max:.3e}", flush=True)
    if out_dtype == np.float32:
        # fp32 accumulation on both sides: bound against the output scale, and per element in the reference test's own
        # form |d| <= abs + rel * |ref| with the absolute term scaled to the row's magnitude
        assert m_max <= 1e-5 and m_sum <= 1e-5, (what, m_floor, m_sum, m_max)
        scale = np.sqrt(np.mean(r32.astype(np.float64) ** 2, axis=1, keepdims=True))
        assert np.all(np.abs(g32 - r32) <= 2e-5 * scale + 5e-5 * np.abs(r32)), what
    else:
        assert m_max <= 2e-3, (what, m_max)
    return g32


@pytest.mark.parametrize("name", NAMES)
def test_gemm_every_format_matches_oracle(hip, oracle, name):
    """Ragged token and row counts around the 64 x 128 tile, K from one K-quant block to 28, K split across workgroups
    (few tiles) and unsplit (many), bias."""
    kind = KINDS[name]
    for n, (N, K, M) in enumerate([(9, 256, 33), (70, 512, 129), (64, 4096, 128), (130, 1024, 300), (200, 768, 515),
                                   (33, 7168, 64)]):
        blocks = oracle.quantize(kind, gaussian(700 + n, (M, K), 0.02))
        x = gaussian(710 + n, (N, K)).astype(np.float16)
        bias = gaussian(720 + n, (M,)) if n % 2 else None
        check(hip, oracle, name, blocks, x, M, f"{name} {N}x{K}x{M}", bias=bias)


@pytest.mark.parametrize("name", [n for n in NAMES if not n.endswith("_k")])
def test_gemm_32_value_formats_odd_stage_counts(hip, oracle, name):
    """A workgroup's two K groups take alternate stages of 128 values: one stage (the second group has none), three
    and five stages, 29 stages split across workgroups."""
    kind = KINDS[name]
    for n, (N, K, M) in enumerate([(5, 128, 40), (70, 384, 129), (33, 640, 300), (12, 3712, 64)]):
        blocks = oracle.quantize(kind, gaussian(750 + n, (M, K), 0.02))
        x = gaussian(760 + n, (N, K)).astype(np.float16)
        check(hip, oracle, name, blocks, x, M, f"{name} {N}x{K}x{M}")


@pytest.mark.parametrize("name", NAMES)
def test_gemm_every_format_random_blocks_matvec_and_fp16_output(hip, matvec, oracle, name):
    """Arbitrary block bytes (every code, scale and min pattern; scales of both signs) and activations far from unit
    scale against the oracle; the fp16 matvec of a device object created with MARMOT_HIP_NO_GEMM decodes the same
    weights and must agree; fp16 output with an fp16 bias; one, three and eight rows."""
    kind = KINDS[name]
    rng = np.random.default_rng(730)
    M, K, N = 160, 1536, 96
    blocks = random_valid_blocks(rng, kind, M, K)
    x = (gaussian(731, (N, K)) * 30.0).astype(np.float16)
    x[0, :] = 2000.0
    x[1, :] = 0.0
    g = check(hip, oracle, name, blocks, x, M, f"{name} random bytes")
    mv = matvec.linear(x, blocks, kind, M)
    assert "direct" in matvec.last_route()
    assert np.max(np.abs(g - mv)) <= 1e-5 * np.max(np.abs(mv))
    soft = oracle.quantize(kind, gaussian(732, (M, K), 0.02))
    x16 = gaussian(733, (N, K)).astype(np.float16)
    bias16 = gaussian(734, (M,)).astype(np.float16)
    check(hip, oracle, name, soft, x16, M, f"{name} f16 out", bias=bias16, out_dtype=np.float16)
    for n in (1, 3, 8):  # decode steps and small batches take the same kernel (one tile of 64 tokens, few of them real)
        few = check(hip, oracle, name, soft, x16[:n], M, f"{name} {n} tokens")
        mv = matvec.linear(x16[:n], soft, kind, M)
        assert "direct" in matvec.last_route()
        assert np.max(np.abs(few - mv)) <= 1e-5 * np.max(np.abs(mv))


def test_gemm_q6_k_layer_shape(hip, oracle):
    """The `down` projection of a Llama-3-8B layer (Q6_K 4096 x 14336) at 512 prompt tokens: a band of rows against the
    oracle, the first tokens against a float64 product of the decoded weights everywhere."""
    name, kind = "q6_k", KINDS["q6_k"]
    M, K, N = 4096, 14336, 512
    from tests.util import quantize_weights

    blocks = quantize_weights(oracle, kind, gaussian(740, (M, K), 0.02))
    x = gaussian(741, (N, K)).astype(np.float16)
    got = hip.linear(x, blocks, kind, M)
    assert hip.last_route() == "gemm_q6_k_f16_mfma"
    band = slice(2048, 2048 + 64)
    ref = oracle.matmul(kind, blocks[band], x, 64, threads=16)
    m_floor, m_sum, m_max = parity_metrics(got[:, band], ref)
    assert m_max <= 1e-5 and m_sum <= 1e-5, (m_floor, m_sum, m_max)
