"""GPU parity, part 4: prefill GEMM (Q4_K weights, fp16 activations, MFMA) against the CPU oracle's direct fp16
route, which is what the reference's CPU backend runs for fp16 activations by default
(matmul_quant_dispatch.c:449-470, vec_dot_impl.h:973-1023)."""
import numpy as np
import pytest

from oracle.pyoracle import KIND_Q4_K
from tests.util import gaussian, parity_metrics, quantize_weights, random_valid_blocks

pytestmark = pytest.mark.gpu
THREADS = 16


@pytest.fixture(scope="module")
def hip():
    from marmot_amd import HipBackend

    b = HipBackend(0)
    yield b
    b.close()


def exact_f64(oracle, blocks, x, M, K):
    """The same weights and activations in float64: what both implementations approximate."""
    deq = oracle.dequantize(KIND_Q4_K, blocks, K).astype(np.float64)
    return x.astype(np.float64) @ deq.T


def check_against_oracle(hip, oracle, blocks, x, M, K, what, bias=None, out_dtype=np.float32):
    got = hip.linear(x, blocks, KIND_Q4_K, M, bias=bias, out_dtype=out_dtype)
    assert "gemm" in hip.last_route(), hip.last_route()
    ref = oracle.matmul(KIND_Q4_K, blocks, x, M, bias=bias, out_dtype=out_dtype, threads=THREADS)
    got32, ref32 = got.astype(np.float32), ref.astype(np.float32)
    m_floor, m_sum, m_max = parity_metrics(got32, ref32)
    print(f"{what}: floored-rel {m_floor:.3e} sum-rel {m_sum:.3e} max-norm {m_max:.3e}", flush=True)
    assert np.all(np.isfinite(got32))
    if out_dtype == np.float32:
        # bound against the output scale: max|d| / max|r| and sum|d| / sum|r| (fp32 accumulate on both sides)
        assert m_max <= 1e-5 and m_sum <= 1e-5, (m_floor, m_sum, m_max)
        # and per element with the reference test's own form |d| <= abs + rel*|ref| (test_matmul_quantized.c:166-177),
        # the absolute term scaled to this output's magnitude
        scale = np.sqrt(np.mean(ref32.astype(np.float64) ** 2, axis=1, keepdims=True))  # per token row
        assert np.all(np.abs(got32 - ref32) <= 2e-5 * scale + 5e-5 * np.abs(ref32))
    else:
        assert m_max <= 2e-3
    return got32, ref32


@pytest.mark.parametrize("N", [1, 2, 5, 8, 9, 64, 128, 130, 512])
def test_gemm_small_shapes(hip, oracle, N):
    """Token counts from a decode step (one token: the fp16 route has no other kernel) to around the 128-token tile, M
    not a multiple of the 256-row tile, K-split and single pass."""
    M, K = 300, 1024
    blocks = oracle.quantize(KIND_Q4_K, gaussian(500, (M, K), 0.02))
    x = gaussian(501 + N, (N, K)).astype(np.float16)
    check_against_oracle(hip, oracle, blocks, x, M, K, f"gemm N={N} M={M} K={K}")


def test_gemm_random_block_bytes_and_large_activations(hip, oracle):
    """Every scale / min / nibble pattern, and activations far from unit scale (sub-block sums stay in fp16 range)."""
    rng = np.random.default_rng(510)
    M, K, N = 256, 2048, 96
    blocks = random_valid_blocks(rng, KIND_Q4_K, M, K)
    x = (gaussian(511, (N, K)) * 300.0).astype(np.float16)
    x[0, :] = 60000.0  # near the fp16 maximum
    x[1, :] = 0.0
    check_against_oracle(hip, oracle, blocks, x, M, K, "gemm random bytes")


def test_gemm_bias_and_f16_output(hip, oracle):
    M, K, N = 512, 1024, 40
    blocks = oracle.quantize(KIND_Q4_K, gaussian(520, (M, K), 0.02))
    x = gaussian(521, (N, K)).astype(np.float16)
    bias = gaussian(522, (M,))
    check_against_oracle(hip, oracle, blocks, x, M, K, "gemm bias f32", bias=bias)
    check_against_oracle(hip, oracle, blocks, x, M, K, "gemm f16 out", bias=bias, out_dtype=np.float16)


@pytest.mark.parametrize("N", [64, 128, 512, 2048])
def test_config3_prefill_gemm(hip, oracle, N):
    """Q4_K 4096 x 4096 (seed 30), fp16 activations N(0,1) (seed 31), fp32 out; sweep of token counts."""
    M = K = 4096
    blocks = quantize_weights(oracle, KIND_Q4_K, gaussian(30, (M, K), 0.02))
    x = gaussian(31, (N, K)).astype(np.float16)
    # the oracle's scalar direct route needs ~N*M*K/0.5e9 core-seconds: check a band of weight rows at the larger N
    rows = M if N <= 128 else 512
    r0 = 1024 if rows != M else 0
    got = hip.linear(x, blocks, KIND_Q4_K, M)
    assert "gemm" in hip.last_route()
    ref = oracle.matmul(KIND_Q4_K, blocks[r0:r0 + rows], x, rows, threads=THREADS)
    g = got[:, r0:r0 + rows]
    m_floor, m_sum, m_max = parity_metrics(g, ref)
    exact = exact_f64(oracle, blocks[r0:r0 + rows], x, rows, K)
    e_gpu = parity_metrics(g, exact)
    e_cpu = parity_metrics(ref, exact)
    print(f"C3 N={N}: hip vs cpu floored-rel {m_floor:.3e} sum-rel {m_sum:.3e} max-norm {m_max:.3e}; "
          f"vs float64: hip {e_gpu[0]:.3e}/{e_gpu[2]:.3e}, cpu {e_cpu[0]:.3e}/{e_cpu[2]:.3e}", flush=True)
    assert m_max <= 1e-5 and m_sum <= 1e-5
    # The floored metric max |y - r| / max(|r|, 1e-3 rms(r)) <= 1e-3 cannot be met AGAINST THE CPU at this shape: the
    # CPU route's own sequential fp32 sum over 4096 products is 2.5e-3 .. 3.3e-3 away from exact arithmetic on that
    # metric (outputs near zero), the HIP result 0.6e-3 .. 1.1e-3. What is asserted: the HIP result is closer to
    # exact arithmetic than the CPU is, on that very metric, and its distance from the CPU is what the two distances
    # from exact arithmetic explain.
    assert e_gpu[0] <= e_cpu[0] and e_gpu[0] <= 1.5e-3, (e_gpu, e_cpu)
    assert m_floor <= e_gpu[0] + e_cpu[0] + 1e-6, (m_floor, e_gpu, e_cpu)
    scale = np.sqrt(np.mean(ref.astype(np.float64) ** 2, axis=1, keepdims=True))
    assert np.all(np.abs(g - ref) <= 2e-5 * scale + 5e-5 * np.abs(ref))
    # the HIP result is at least as close to exact arithmetic as the CPU reference's sequential fp32 sum
    assert e_gpu[2] <= max(e_cpu[2] * 1.5, 1e-6)
    # rows outside the checked band: K-split and full tiles must agree with a float64 product everywhere
    full_exact = exact_f64(oracle, blocks, x[:8], M, K)
    assert parity_metrics(got[:8], full_exact)[2] <= 1e-5


def test_gemm_loader_tile_and_self_loading_tile_agree(oracle, monkeypatch):
    """The 64 x 128 tile exists twice: fed by loader wavefronts (default) and with wavefronts that load for
    themselves (MARMOT_HIP_NO_GEMM_LOADERS, read when a device object is created). Both compute the same exact-operand
    products and differ only in fp32 summation order: each must meet the oracle bound, and they must agree with one
    another to the same bound, on ragged token / row counts, one block of K, K split across workgroups, bias and
    fp16 output."""
    from marmot_amd import HipBackend

    loaders = HipBackend(0)
    monkeypatch.setenv("MARMOT_HIP_NO_GEMM_LOADERS", "1")
    plain = HipBackend(0)
    monkeypatch.delenv("MARMOT_HIP_NO_GEMM_LOADERS")
    try:
        cases = [(9, 256, 33), (70, 512, 129), (64, 4096, 128), (130, 1024, 300), (200, 768, 515), (512, 2048, 640)]
        for n, (N, K, M) in enumerate(cases):
            print(f"gemm tile pair N={N} K={K} M={M}", flush=True)
            blocks = oracle.quantize(KIND_Q4_K, gaussian(560 + n, (M, K), 0.02))
            x = gaussian(570 + n, (N, K)).astype(np.float16)
            bias = gaussian(580 + n, (M,)) if n % 2 else None
            a, ref = check_against_oracle(loaders, oracle, blocks, x, M, K, f"loader tile {N}x{K}x{M}", bias=bias)
            b, _ = check_against_oracle(plain, oracle, blocks, x, M, K, f"self-loading tile {N}x{K}x{M}", bias=bias)
            assert np.max(np.abs(a - b)) <= 1e-5 * np.max(np.abs(ref))
        N, K, M = 96, 1024, 260
        blocks = oracle.quantize(KIND_Q4_K, gaussian(590, (M, K), 0.02))
        x = gaussian(591, (N, K)).astype(np.float16)
        bias = gaussian(592, (M,)).astype(np.float16)
        a, _ = check_against_oracle(loaders, oracle, blocks, x, M, K, "loader tile f16 out", bias=bias, out_dtype=np.float16)
        b, _ = check_against_oracle(plain, oracle, blocks, x, M, K, "self-loading tile f16 out", bias=bias,
                                    out_dtype=np.float16)
        assert np.max(np.abs(a - b)) <= 2e-3 * np.max(np.abs(a))
    finally:
        loaders.close()
        plain.close()


def test_gemm_wide_tile(oracle, monkeypatch):
    """The 128 x 128 tile keeps its running sums in units of the current block's super-block scale (one rescale per
    block instead of a second accumulator set). Forced at every token count with MARMOT_HIP_GEMM_WIDE: ragged token /
    row counts, one block of K, K split across workgroups, every scale / min / nibble pattern with super-block scales
    of both signs down to fp16 denormals, blocks and whole rows whose scale is zero, bias and fp16 output; and the
    default device must take the tile by itself where one round of such tiles covers most of the chip."""
    from marmot_amd import HipBackend

    monkeypatch.setenv("MARMOT_HIP_GEMM_WIDE", "1")
    wide = HipBackend(0)
    monkeypatch.delenv("MARMOT_HIP_GEMM_WIDE")
    plain = HipBackend(0)
    try:
        cases = [(9, 256, 33), (130, 256, 128), (256, 512, 128), (300, 768, 515), (512, 1024, 300), (640, 2048, 640)]
        for n, (N, K, M) in enumerate(cases):
            print(f"wide tile N={N} K={K} M={M}", flush=True)
            blocks = oracle.quantize(KIND_Q4_K, gaussian(660 + n, (M, K), 0.02))
            x = gaussian(670 + n, (N, K)).astype(np.float16)
            bias = gaussian(680 + n, (M,)) if n % 2 else None
            a, ref = check_against_oracle(wide, oracle, blocks, x, M, K, f"wide tile {N}x{K}x{M}", bias=bias)
            assert wide.last_route() == "gemm_q4_k_f16_mfma_wide"
            b, _ = check_against_oracle(plain, oracle, blocks, x, M, K, f"default tile {N}x{K}x{M}", bias=bias)
            assert np.max(np.abs(a - b)) <= 1e-5 * np.max(np.abs(ref))
        rng = np.random.default_rng(690)
        M, K, N = 256, 2048, 200
        blocks = random_valid_blocks(rng, KIND_Q4_K, M, K)
        x = (gaussian(691, (N, K)) * 300.0).astype(np.float16)
        x[0, :] = 60000.0
        x[1, :] = 0.0
        check_against_oracle(wide, oracle, blocks, x, M, K, "wide tile random bytes")
        dead = blocks.copy().reshape(M, K // 256, 144)
        dead[::3, 1, 0:2] = 0   # a block in the middle of every third row
        dead[5, :, 0:2] = 0     # a whole row (its min terms remain)
        dead[7, 0, 0:2] = 0     # the first block of a row
        dead[9, -1, 0:2] = 0    # the last one
        dead[11, 2:5, 0:2] = 0  # a run
        dead = dead.reshape(blocks.shape)
        bias = gaussian(692, (M,)).astype(np.float16)
        check_against_oracle(wide, oracle, dead, x, M, K, "wide tile zero scales")
        soft = oracle.quantize(KIND_Q4_K, gaussian(694, (M, K), 0.02)).reshape(M, K // 256, 144).copy()
        soft[::4, 3, 0:2] = 0
        soft[6, :, 0:2] = 0
        x16 = gaussian(695, (N, K)).astype(np.float16)
        check_against_oracle(wide, oracle, soft.reshape(blocks.shape), x16, M, K, "wide tile f16 out", bias=bias,
                             out_dtype=np.float16)
        # the band the default route takes by itself: 6 x 32 tiles at 768 tokens x 4096 rows on 256 compute units
        M = K = 4096
        N = 768
        blocks = quantize_weights(oracle, KIND_Q4_K, gaussian(30, (M, K), 0.02))
        x = gaussian(693, (N, K)).astype(np.float16)
        got = plain.linear(x, blocks, KIND_Q4_K, M)
        units = plain.caps()["num_compute_units"]
        if 192 <= units and 8 * 192 >= 5 * units:
            assert plain.last_route() == "gemm_q4_k_f16_mfma_wide", plain.last_route()
        exact = exact_f64(oracle, blocks[1000:1256], x, 256, K)
        assert parity_metrics(got[:, 1000:1256], exact)[2] <= 2e-6
    finally:
        wide.close()
        plain.close()
