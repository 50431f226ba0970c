"""GPU parity, part 2: marmot_linear on the HIP backend against the CPU oracle (through the C ABI)."""
import numpy as np
import pytest

from oracle.pyoracle import BLOCK_VALUES, KIND_Q8_1, KIND_Q2_K, KIND_Q3_K, KIND_Q4_0, KIND_Q4_1, KIND_Q5_0, KIND_Q5_1, KIND_Q4_K, KIND_Q5_K, KIND_Q6_K, KIND_Q8_0
from tests.util import assert_matmul_parity, bits, gaussian, parity_metrics, quantize_weights, random_valid_blocks

pytestmark = pytest.mark.gpu

KINDS = {"q4_0": KIND_Q4_0, "q8_0": KIND_Q8_0, "q4_k": KIND_Q4_K, "q5_k": KIND_Q5_K, "q6_k": KIND_Q6_K,
         "q4_1": KIND_Q4_1, "q5_0": KIND_Q5_0, "q5_1": KIND_Q5_1, "q2_k": KIND_Q2_K, "q3_k": KIND_Q3_K,
         "q8_1": KIND_Q8_1}
THREADS = 16


@pytest.fixture(scope="module")
def hip():
    from marmot_amd import HipBackend

    b = HipBackend(0)
    yield b
    b.close()


@pytest.mark.parametrize("name", ["Q4_0", "Q4_1", "Q5_0", "Q5_1", "Q8_0", "Q8_1", "Q2_K", "Q3_K", "Q4_K", "Q5_K", "Q6_K"])
def test_reference_matmul_goldens_fp32(hip, ref_goldens, name):
    """The reference's own golden cases (tests/backend/golden_matmul_llama.h), its own tolerance."""
    kind, N, K, M = (int(v) for v in ref_goldens[f"matmul_{name}_dims"])
    w = ref_goldens[f"matmul_{name}_weight"]
    x = ref_goldens[f"matmul_{name}_input_f32"].reshape(N, K)
    exp = ref_goldens[f"matmul_{name}_expected_f32"].reshape(N, M)
    got = hip.linear(x, w, kind, M)
    assert np.all(np.abs(got - exp) <= 2e-5 + 5e-5 * np.abs(exp)), (got, exp)


@pytest.mark.parametrize("name", ["Q4_0", "Q4_1", "Q5_0", "Q5_1", "Q8_0", "Q8_1", "Q2_K", "Q3_K", "Q4_K", "Q5_K", "Q6_K"])
def test_reference_matmul_goldens_fp16(hip, ref_goldens, name):
    """fp16 activations: the reference's golden outputs, which for Q2_K, Q3_K, Q5_K and Q6_K are snapshots of its
    fp16 direct dots as written (their block indexing differs from the dequantizers; the direct route mirrors it)."""
    kind, N, K, M = (int(v) for v in ref_goldens[f"matmul_{name}_dims"])
    w = ref_goldens[f"matmul_{name}_weight"]
    x = ref_goldens[f"matmul_{name}_input_f16"].view(np.float16).reshape(N, K)
    exp = ref_goldens[f"matmul_{name}_expected_f16"].reshape(N, M)
    got = hip.linear(x, w, kind, M)
    assert np.all(np.abs(got - exp) <= 2e-5 + 5e-5 * np.abs(exp)), (got, exp)


def test_config1_q8_0_matvec_full_size(hip, oracle):
    """Q8_0, W 5632 x 2048 from N(0, 0.02) seed 0, x N(0,1) seed 1, batch 1."""
    M, K = 5632, 2048
    w = gaussian(0, (M, K), 0.02)
    blocks = quantize_weights(oracle, KIND_Q8_0, w)
    x = gaussian(1, (1, K))
    ref = oracle.matmul(KIND_Q8_0, blocks, x, M, threads=THREADS)
    got = hip.linear(x, blocks, KIND_Q8_0, M)
    print("route:", hip.last_route(), "metrics:", parity_metrics(got, ref), flush=True)
    assert_matmul_parity(got, ref, what="C1 Q8_0 5632x2048")
    # dequantized weights bit-exact
    assert np.array_equal(bits(hip.dequantize(KIND_Q8_0, blocks, K)), bits(oracle.dequantize(KIND_Q8_0, blocks, K)))


@pytest.mark.parametrize("name", ["q4_k", "q6_k"])
@pytest.mark.parametrize("M,K", [(14336, 4096), (4096, 14336)])
def test_config2_kquant_decode_full_size(hip, oracle, name, M, K):
    """Q4_K / Q6_K at Llama-3-8B FFN shapes, batch 1, 4 and 8, activations quantized to Q8_K on device."""
    kind = KINDS[name]
    i = ["q4_k", "q6_k"].index(name) * 2 + (0 if M == 14336 else 1)
    print(f"C2 {name} {M}x{K}: quantizing weights", flush=True)
    w = gaussian(10 + i, (M, K), 0.02)
    blocks = quantize_weights(oracle, kind, w)
    del w
    d_w = hip.to_device(blocks)
    # dequantized weights: bit-exact over every element of the matrix
    d_f = hip.alloc(M * K * 4)
    hip.dequantize_d(kind, d_w, M, K, d_f)
    deq = d_f.download(np.float32, (M, K))
    d_f.free()
    step = 1024
    for r0 in range(0, M, step):
        exp = oracle.dequantize(kind, blocks[r0:r0 + step], K)
        assert np.array_equal(bits(deq[r0:r0 + step]), bits(exp)), f"dequant differs in rows {r0}.."
    del deq
    for N in (1, 4, 8):
        print(f"C2 {name} {M}x{K} N={N}", flush=True)
        x = gaussian(20 + i, (N, K))
        ref = oracle.matmul(kind, blocks, x, M, threads=THREADS)
        d_x = hip.to_device(x)
        d_o = hip.alloc(N * M * 4)
        hip.linear_d(kind, d_w, d_x, 0, N, K, M, d_o, 0)
        got = d_o.download(np.float32, (N, M))
        d_x.free()
        d_o.free()
        m = assert_matmul_parity(got, ref, what=f"C2 {name} {M}x{K} N={N}")
        print("   route:", hip.last_route(), "metrics:", m, flush=True)
    d_w.free()


@pytest.mark.parametrize("name", ["q4_0", "q4_1", "q5_0", "q5_1", "q8_0", "q8_1", "q2_k", "q3_k", "q4_k", "q5_k", "q6_k"])
@pytest.mark.parametrize("N", [1, 2, 3, 5, 8, 11, 16, 19])
def test_linear_batches_and_ragged_rows(hip, oracle, name, N):
    """All column-tile widths (8/4/2/1) and M not a multiple of the rows-per-workgroup."""
    kind = KINDS[name]
    M, K = 203, 2048
    blocks = oracle.quantize(kind, gaussian(60, (M, K), 0.02))
    x = gaussian(61 + N, (N, K))
    ref = oracle.matmul(kind, blocks, x, M)
    got = hip.linear(x, blocks, kind, M)
    assert_matmul_parity(got, ref, what=f"{name} N={N}")


@pytest.mark.parametrize("name", ["q4_0", "q4_1", "q5_0", "q5_1", "q8_0", "q8_1", "q2_k", "q3_k", "q4_k", "q5_k", "q6_k"])
@pytest.mark.parametrize("K", [256, 512, 768, 1280, 8192, 11008, 28672])
def test_linear_k_sweep(hip, oracle, name, K):
    """Rows shorter than one wave-load, rows needing several wavefronts, and long rows."""
    kind = KINDS[name]
    M = 70
    blocks = oracle.quantize(kind, gaussian(70, (M, K), 0.02))
    for N in (1, 4):
        x = gaussian(71 + N, (N, K))
        ref = oracle.matmul(kind, blocks, x, M)
        got = hip.linear(x, blocks, kind, M)
        assert_matmul_parity(got, ref, what=f"{name} K={K} N={N}")


@pytest.mark.parametrize("name,K", [("q6_k", 3584), ("q6_k", 256 * 13), ("q8_0", 32 * 113), ("q2_k", 256 * 7),
                                    ("q3_k", 256 * 5), ("q4_0", 32 * 99)])
def test_linear_rows_off_16_byte_boundaries(hip, oracle, name, K):
    """Rows whose byte length is not a multiple of 16 (3584 = the hidden size of Qwen2-7B in Q6_K: 14 blocks of 210
    bytes) at decode sizes: the loader of the LDS ring copies every step from the 16-byte boundary below its first row,
    and the tensor's last bytes come two at a time when the tensor does not end on such a boundary. Row counts that end
    inside a step, on a step and on a workgroup."""
    kind = KINDS[name]
    for M in (3584, 1031, 64):
        blocks = oracle.quantize(kind, gaussian(75, (M, K), 0.02))
        for N in (1, 2, 4):
            x = gaussian(76 + N, (N, K))
            got = hip.linear(x, blocks, kind, M)
            assert_matmul_parity(got, oracle.matmul(kind, blocks, x, M, threads=8), what=f"{name} {M}x{K} N={N}")


@pytest.mark.parametrize("name", ["q4_0", "q4_1", "q5_0", "q5_1", "q8_0", "q8_1", "q2_k", "q3_k", "q4_k", "q5_k", "q6_k"])
def test_linear_ragged_k(hip, oracle, name):
    """K not a multiple of the block: weight and activation tails are zero-padded blocks."""
    kind = KINDS[name]
    bv = BLOCK_VALUES[kind]
    K = 3 * bv + bv // 2 + 3
    M = 9
    blocks = oracle.quantize(kind, gaussian(80, (M, K), 0.02))
    x = gaussian(81, (3, K))
    ref = oracle.matmul(kind, blocks, x, M)
    got = hip.linear(x, blocks, kind, M)
    assert_matmul_parity(got, ref, what=f"{name} ragged K={K}")


@pytest.mark.parametrize("name", ["q4_0", "q4_1", "q5_0", "q5_1", "q8_0", "q8_1", "q2_k", "q3_k", "q4_k", "q5_k", "q6_k"])
def test_linear_random_block_bytes(hip, oracle, name):
    """Weights that are arbitrary block bytes (all 6-bit scale / min patterns, negative Q6_K scales)."""
    kind = KINDS[name]
    rng = np.random.default_rng(90)
    M, K = 33, 2048
    blocks = random_valid_blocks(rng, kind, M, K)
    x = gaussian(91, (4, K))
    ref = oracle.matmul(kind, blocks, x, M)
    got = hip.linear(x, blocks, kind, M)
    assert_matmul_parity(got, ref, what=f"{name} random bytes")


@pytest.mark.parametrize("name", ["q8_0", "q2_k", "q3_k", "q4_k", "q5_k", "q6_k"])
def test_linear_bias_epilogue(hip, oracle, name):
    kind = KINDS[name]
    M, K, N = 50, 1024, 3
    blocks = oracle.quantize(kind, gaussian(100, (M, K), 0.02))
    x = gaussian(101, (N, K))
    bias = gaussian(102, (M,))
    ref = oracle.matmul(kind, blocks, x, M, bias=bias)
    got = hip.linear(x, blocks, kind, M, bias=bias)
    d = np.abs(got - ref)
    assert np.max(d) <= 1e-5 * max(1.0, np.abs(ref).max())


@pytest.mark.parametrize("name", ["q4_0", "q4_1", "q5_0", "q5_1", "q8_0", "q8_1", "q2_k", "q3_k", "q4_k", "q5_k", "q6_k"])
def test_linear_fp16_direct_small_batch(hip, oracle, name):
    """fp16 activations take the direct route (no activation quantization) like the CPU reference."""
    kind = KINDS[name]
    M, K = 64, 1024
    blocks = oracle.quantize(kind, gaussian(110, (M, K), 0.02))
    for N in (1, 3, 7):
        x = gaussian(111 + N, (N, K)).astype(np.float16)
        ref = oracle.matmul(kind, blocks, x, M)
        got = hip.linear(x, blocks, kind, M)
        assert "direct" in hip.last_route() or "gemm" in hip.last_route()
        assert_matmul_parity(got, ref, what=f"{name} fp16 N={N}")
        got16 = hip.linear(x, blocks, kind, M, out_dtype=np.float16)
        ref16 = oracle.matmul(kind, blocks, x, M, out_dtype=np.float16)
        assert np.max(np.abs(got16.astype(np.float32) - ref16.astype(np.float32))) <= \
            2e-3 * np.abs(ref16.astype(np.float32)).max()
        # forced packing of fp16 activations equals the fp32 packed path on the widened values
        forced = hip.linear(x, blocks, kind, M, force_pack=True)
        assert_matmul_parity(forced, oracle.matmul(kind, blocks, x, M, force_pack=True), what=f"{name} forced")


def test_linear_dual_output_equals_two_singles(hip, oracle):
    """cpu_matmul_quantized_dual_output semantics (test_matmul_quantized.c:202-298)."""
    M, K, N = 96, 2048, 5
    a = oracle.quantize(KIND_Q4_K, gaussian(120, (M, K), 0.02))
    b = oracle.quantize(KIND_Q4_K, gaussian(121, (M, K), 0.02))
    x = gaussian(122, (N, K))
    oa, ob = hip.linear_dual(x, a, b, KIND_Q4_K, M)
    assert np.array_equal(bits(oa), bits(hip.linear(x, a, KIND_Q4_K, M)))
    assert np.array_equal(bits(ob), bits(hip.linear(x, b, KIND_Q4_K, M)))


def test_linear_error_behaviour(hip, oracle):
    from marmot_amd import MarmotHipError

    M, K = 8, 256
    blocks = oracle.quantize(KIND_Q4_K, gaussian(130, (M, K), 0.02))
    x = gaussian(131, (1, K))
    with pytest.raises(MarmotHipError) as e:  # fp32 input cannot produce fp16 output (helpers/matmul.c:104-112)
        hip.linear(x, blocks, KIND_Q4_K, M, out_dtype=np.float16)
    assert e.value.code == -6
    with pytest.raises(MarmotHipError) as e:  # unsupported quant kind -> NOT_IMPLEMENTED (fallback signal)
        hip.linear_d(12, hip.to_device(blocks), hip.to_device(x), 0, 1, K, M, hip.alloc(64), 0)  # Q8_K weights
    assert e.value.code == -8
    # N = 0 is a no-op
    hip.linear_d(KIND_Q4_K, hip.to_device(blocks), hip.to_device(x), 0, 0, K, M, hip.alloc(64), 0)
    hip.synchronize()


@pytest.mark.parametrize("name", ["q4_0", "q4_1", "q5_0", "q5_1", "q8_0", "q8_1", "q2_k", "q3_k", "q4_k", "q5_k", "q6_k"])
def test_loader_consumer_matvec_equals_register_streaming_matvec(oracle, name, monkeypatch):
    """The loader/consumer matvec (weights through an LDS ring) keeps the lane mapping and the reduction order of the
    register-streaming kernel: the two must agree bit for bit, on whole and ragged row groups, one and two K slices
    per lane, fused and packed activations. Route switches are read when a device object is created, so each variant
    gets a device object of its own (both without the row-owning kernels, which sum in another order)."""
    from marmot_amd import HipBackend

    kind = KINDS[name]
    monkeypatch.setenv("MARMOT_HIP_NO_ROW_KERNELS", "1")
    ring = HipBackend(0)
    monkeypatch.setenv("MARMOT_HIP_NO_LDS_RING", "1")
    streaming = HipBackend(0)
    monkeypatch.delenv("MARMOT_HIP_NO_LDS_RING")
    monkeypatch.delenv("MARMOT_HIP_NO_ROW_KERNELS")
    try:
        for M, K, N in ((256, 2048, 1), (203, 4096, 1), (77, 8192, 1), (64, 14336, 1), (40, 28672, 1), (203, 4096, 2)):
            blocks = oracle.quantize(kind, gaussian(500 + K, (M, K), 0.02))
            x = gaussian(501 + K + N, (N, K))
            with_ring = ring.linear(x, blocks, kind, M)
            without = streaming.linear(x, blocks, kind, M)
            assert "rows" not in ring.last_route() and "rows" not in streaming.last_route()
            assert np.array_equal(bits(with_ring), bits(without)), f"{name} {M}x{K} N={N}"
            assert_matmul_parity(with_ring, oracle.matmul(kind, blocks, x, M), what=f"{name} {M}x{K} N={N}")
    finally:
        ring.close()
        streaming.close()



def _special_activations(K: int) -> np.ndarray:
    """One activation row that drives the Q8_K packer through its exact path and its corner cases, block by block:
    +max and -max of equal magnitude in every order and lane position (first occurrence decides the sign of every
    code), an all-zero block, a block of tiny values, a block with one huge value, ordinary blocks in between."""
    x = gaussian(7001, (1, K))
    nb = K // 256
    for b in range(nb):
        blk = x[0, b * 256:(b + 1) * 256]
        mode = b % 8
        if mode == 1:  # tie: +m first, then -m, positions spread over the 16-value groups of different lanes
            m = np.float32(np.abs(blk).max() * 1.5)
            p, q = (17 * b) % 256, (17 * b + 101) % 256
            lo, hi = min(p, q), max(p, q)
            blk[lo], blk[hi] = m, -m
        elif mode == 2:  # tie: -m first
            m = np.float32(np.abs(blk).max() * 1.25)
            p, q = (29 * b + 3) % 256, (29 * b + 64) % 256
            lo, hi = min(p, q), max(p, q)
            blk[lo], blk[hi] = -m, m
        elif mode == 3:
            blk[:] = 0.0
        elif mode == 4:
            blk *= np.float32(1e-36)  # below the packer's fast-path range
        elif mode == 5:
            blk[(13 * b) % 256] = np.float32(-3.0e4)
        elif mode == 6:  # tie inside one lane's 16 values, in its rotated groups
            m = np.float32(np.abs(blk).max() * 2.0)
            base = 16 * ((5 * b) % 16)
            blk[base + 13], blk[base + 2] = m, -m
    return x


@pytest.mark.parametrize("M,K", [(4096, 14336), (4100, 14336), (14336, 4096), (14337, 4096), (4096, 11008),
                                 (8192, 8192), (28672, 2048)])
def test_resident_share_decode_kernel(oracle, M, K, monkeypatch):
    """The resident-share Q4_K decode kernel (one activation row, weights of 16 MB and more, rows of up to 64 blocks):
    whole and ragged last workgroups, one and two K segments per row, odd block counts, the Q8_K packer's exact path
    (ties, zero and tiny blocks); against the oracle and against the ring form of the row kernel, which it replaces
    for these shapes and whose lane mapping and summation order it keeps (bit-equal results)."""
    from marmot_amd import HipBackend

    kind = KIND_Q4_K
    resident = HipBackend(0)
    monkeypatch.setenv("MARMOT_HIP_NO_RESIDENT_ROWS", "1")
    ring = HipBackend(0)
    monkeypatch.delenv("MARMOT_HIP_NO_RESIDENT_ROWS")
    try:
        rng = np.random.Generator(np.random.PCG64(M + K))
        blocks = random_valid_blocks(rng, kind, M, K)
        bias = gaussian(M, (M,))
        for x, with_bias in ((gaussian(K, (1, K)), False), (_special_activations(K), True)):
            got = resident.linear(x, blocks, kind, M, bias=bias if with_bias else None)
            assert resident.last_route() == "matvec_rows2_q4_k_q8_k_fused", resident.last_route()
            other = ring.linear(x, blocks, kind, M, bias=bias if with_bias else None)
            assert ring.last_route() != "matvec_rows2_q4_k_q8_k_fused"
            ref = oracle.matmul(kind, blocks, x, M, threads=THREADS)
            if with_bias:
                ref = ref + bias[None, :]
            assert_matmul_parity(got, ref, what=f"resident share {M}x{K} bias={with_bias}")
            assert_matmul_parity(other, ref, what=f"ring {M}x{K} bias={with_bias}")
            assert np.array_equal(bits(got), bits(other)), f"{M}x{K}: resident-share and ring kernels differ"
    finally:
        resident.close()
        ring.close()


@pytest.mark.parametrize("name", ["q4_k", "q6_k"])
def test_logits_projection_at_vocabulary_size(hip, oracle, name):
    """The logits projection of a Llama-3 model: 128256 rows of 4096 (295 MB of Q4_K, 431 MB of Q6_K: beyond the sizes at
    which the row-owning kernels hand over to the streaming ones), one and four activation rows, on arbitrary valid
    block bytes (no quantizer run)."""
    kind = KINDS[name]
    M, K = 128256, 4096
    rng = np.random.Generator(np.random.PCG64(128256 + kind))
    blocks = random_valid_blocks(rng, kind, M, K)
    d_w = hip.to_device(blocks)
    try:
        for N in (1, 4):
            print(f"logits {name} {M}x{K} N={N}", flush=True)
            x = gaussian(9000 + N, (N, K))
            d_x = hip.to_device(x)
            d_o = hip.alloc(N * M * 4)
            hip.linear_d(kind, d_w, d_x, 0, N, K, M, d_o, 0)
            got = d_o.download(np.float32, (N, M))
            d_x.free()
            d_o.free()
            ref = oracle.matmul(kind, blocks, x, M, threads=THREADS)
            m = assert_matmul_parity(got, ref, what=f"logits {name} N={N}")
            print("   route:", hip.last_route(), "metrics:", m, flush=True)
    finally:
        d_w.free()
