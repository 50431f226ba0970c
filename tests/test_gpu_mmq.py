"""GPU parity, part 2b: the small-batch matmul on the int8 matrix cores (Q4_K from 3 activation rows, Q6_K from 5)
against the CPU oracle, through the C ABI: every pass shape (up to 8 / up to 16 rows per pass, several passes), ragged
row groups, K split over wavefronts and over workgroups (partials + ordered reduction), bias and fp16 epilogues, the
dual-output call, the prepacked-activation entry point and graph replay."""
import numpy as np
import pytest

from marmot_amd import capi
from oracle.pyoracle import KIND_Q4_K, KIND_Q5_K, KIND_Q6_K
from tests.util import assert_matmul_parity, bits, gaussian, random_valid_blocks

pytestmark = pytest.mark.gpu

KINDS = {"q4_k": KIND_Q4_K, "q5_k": KIND_Q5_K, "q6_k": KIND_Q6_K}
MIN_ROWS = {"q4_k": 3, "q6_k": 5}


@pytest.fixture(scope="module")
def hip():
    from marmot_amd import HipBackend

    b = HipBackend(0)
    yield b
    b.close()


@pytest.mark.parametrize("name", ["q4_k", "q6_k"])
def test_route_threshold(hip, oracle, name):
    """Below the threshold the fused matvec runs, from it on the MFMA kernel; both agree with the oracle."""
    kind = KINDS[name]
    M, K = 64, 1024
    blocks = oracle.quantize(kind, gaussian(300, (M, K), 0.02))
    for N in range(1, 8):
        x = gaussian(301 + N, (N, K))
        got = hip.linear(x, blocks, kind, M)
        route = hip.last_route()
        assert ("mmq_" in route) == (N >= MIN_ROWS[name]), (N, route)
        assert_matmul_parity(got, oracle.matmul(kind, blocks, x, M), what=f"{name} N={N} {route}")


@pytest.mark.parametrize("name", ["q4_k", "q6_k"])
def test_single_block_is_bit_exact(hip, oracle, name):
    """K = 256: one block per row, so no fp32 reassociation is left and the exact integer block dots must give the
    oracle's bits (same expression: (a.d * w.d) * isum - (a.d * w.dmin) * msum)."""
    kind = KINDS[name]
    M, K = 77, 256
    rng = np.random.default_rng(310)
    blocks = random_valid_blocks(rng, kind, M, K)
    # (Q6_K: 16 rows per pass; from 17 rows on the tiled kernel runs, which adds the two halves of a block separately)
    for N in ((5, 8, 16, 21) if name == "q4_k" else (5, 8, 16)):
        x = gaussian(311 + N, (N, K))
        got = hip.linear(x, blocks, kind, M)
        assert "mmq_" in hip.last_route() and "tile" not in hip.last_route()
        ref = oracle.matmul(kind, blocks, x, M)
        assert np.array_equal(bits(got), bits(ref)), f"{name} N={N}"


@pytest.mark.parametrize("name", ["q4_k", "q6_k"])
@pytest.mark.parametrize("N", [5, 8, 9, 16, 17, 33, 40])
def test_pass_shapes_and_ragged_row_groups(hip, oracle, name, N):
    """Passes of up to 16 rows (the last one partial), 4- and 8-register accumulators, M not a multiple of 32."""
    kind = KINDS[name]
    M, K = 32 * 9 + 13, 2048
    blocks = oracle.quantize(kind, gaussian(320, (M, K), 0.02))
    x = gaussian(321 + N, (N, K))
    got = hip.linear(x, blocks, kind, M)
    assert "mmq_" in hip.last_route()
    assert_matmul_parity(got, oracle.matmul(kind, blocks, x, M), what=f"{name} N={N}")


@pytest.mark.parametrize("name", ["q4_k", "q6_k"])
@pytest.mark.parametrize("M,K", [(40, 256 * 3), (64, 14336), (200, 256 * 23), (1024, 256 * 9)])
def test_k_split_over_wavefronts_and_workgroups(hip, oracle, name, M, K):
    """Few row groups and long rows: K is split over workgroups (fp32 partials, reduced in split order); block counts
    that do not divide evenly leave some wavefronts with fewer (or no) blocks."""
    kind = KINDS[name]
    blocks = oracle.quantize(kind, gaussian(330, (M, K), 0.02))
    for N in (6, 13):
        x = gaussian(331 + N, (N, K))
        got = hip.linear(x, blocks, kind, M)
        assert "mmq_" in hip.last_route()
        assert_matmul_parity(got, oracle.matmul(kind, blocks, x, M), what=f"{name} {M}x{K} N={N}")


@pytest.mark.parametrize("K", [1280, 3584, 11008])
def test_q6k_rows_off_16_byte_boundaries(hip, oracle, K):
    """Q6_K rows of 5, 14 and 43 blocks (210-byte blocks: such rows start at any even address) through the loader /
    consumer kernel, which rounds its 16-byte loads down per row; row counts that end inside a group of 32, tensors
    that do not end on a 16-byte boundary (the last chunk then comes two bytes at a time), K split over wavefronts and
    workgroups."""
    kind = KIND_Q6_K
    for M in (70, 1031, 4096):
        blocks = oracle.quantize(kind, gaussian(345, (M, K), 0.02))
        for N in (5, 8, 16):
            x = gaussian(346 + N, (N, K))
            got = hip.linear(x, blocks, kind, M)
            assert hip.last_route() == "mmq_q6_k_q8_k_mfma"
            assert_matmul_parity(got, oracle.matmul(kind, blocks, x, M, threads=8), what=f"Q6_K {M}x{K} N={N}")


@pytest.mark.parametrize("name", ["q4_k", "q6_k"])
@pytest.mark.parametrize("M,K", [(96, 1024), (64, 14336)])
def test_bias_and_fp16_epilogues(hip, oracle, name, M, K):
    """Bias on the direct store and after the split-K reduction; fp16 activations forced through the packed path with
    fp16 output: the dot is rounded to fp16 first, then the bias is added to the stored value."""
    kind = KINDS[name]
    N = 7
    blocks = oracle.quantize(kind, gaussian(340, (M, K), 0.02))
    x = gaussian(341, (N, K))
    bias = gaussian(342, (M,))
    ref = oracle.matmul(kind, blocks, x, M, bias=bias)
    got = hip.linear(x, blocks, kind, M, bias=bias)
    assert "mmq_" in hip.last_route()
    assert np.max(np.abs(got - ref)) <= 1e-3 * np.abs(ref).max()
    x16 = x.astype(np.float16)
    bias16 = bias.astype(np.float16)
    ref16 = oracle.matmul(kind, blocks, x16, M, bias=bias16, out_dtype=np.float16, force_pack=True)
    got16 = hip.linear(x16, blocks, kind, M, bias=bias16, out_dtype=np.float16, force_pack=True)
    assert "mmq_" in hip.last_route()
    assert np.max(np.abs(got16.astype(np.float32) - ref16.astype(np.float32))) <= \
        2e-3 * np.abs(ref16.astype(np.float32)).max()


@pytest.mark.parametrize("name", ["q4_k", "q6_k"])
@pytest.mark.parametrize("M,K", [(96, 2048), (64, 14336)])
def test_dual_output_equals_two_singles(hip, oracle, name, M, K):
    kind = KINDS[name]
    N = 9
    a = oracle.quantize(kind, gaussian(350, (M, K), 0.02))
    b = oracle.quantize(kind, gaussian(351, (M, K), 0.02))
    x = gaussian(352, (N, K))
    oa, ob = hip.linear_dual(x, a, b, kind, M)
    assert "mmq_" in hip.last_route()
    assert np.array_equal(bits(oa), bits(hip.linear(x, a, kind, M)))
    assert np.array_equal(bits(ob), bits(hip.linear(x, b, kind, M)))
    assert_matmul_parity(oa, oracle.matmul(kind, a, x, M), what=f"{name} dual a")


@pytest.mark.parametrize("name", ["q4_k", "q6_k"])
def test_prepacked_activations_and_graph_replay(hip, oracle, name):
    """Activations packed once (Q8_K rows) and reused; the captured matmul replays to the same bits each time, with
    other work and synchronizations between the replays."""
    kind = KINDS[name]
    M, K, N = 320, 14336, 8
    blocks = oracle.quantize(kind, gaussian(360, (M, K), 0.02))
    x = gaussian(361, (N, K))
    ref = oracle.matmul(kind, blocks, x, M)
    d_w = hip.to_device(blocks)
    d_x = hip.to_device(x)
    d_p = hip.alloc(hip.packed_activation_bytes(kind, N, K))
    d_out = hip.alloc(N * M * 4)
    hip.pack_activations_d(kind, d_x, capi.DT_F32, N, K, d_p)
    hip.linear_prepacked_d(kind, d_w, d_p, N, K, M, d_out)
    assert "mmq_" in hip.last_route()
    eager = d_out.download(np.float32, (N, M))
    assert_matmul_parity(eager, ref, what=f"{name} prepacked")
    fused = hip.linear(x, blocks, kind, M)
    if "mmq_rows" in hip.last_route():
        # fp32 activations take the row-owning kernel, which adds the blocks of a row in another order
        assert_matmul_parity(fused, ref, what=f"{name} fused")
        assert_matmul_parity(fused, eager, what=f"{name} fused against prepacked")
    else:
        assert np.array_equal(bits(eager), bits(fused))

    g = hip.graph_capture(lambda: hip.linear_d(kind, d_w, d_x, capi.DT_F32, N, K, M, d_out, capi.DT_F32))
    try:
        for rep in range(3):
            d_out.upload(np.full(N * M * 4, 0xFF, dtype=np.uint8))
            hip.graph_launch(g)
            hip.synchronize()
            got = d_out.download(np.float32, (N, M))
            assert np.array_equal(bits(got), bits(fused)), f"{name} replay {rep}"
            other = hip.linear(gaussian(370 + rep, (3, 256)), blocks[:, : blocks.shape[1] // (K // 256)].copy(), kind, M)
            assert other.shape == (3, M)
    finally:
        hip.graph_destroy(g)
        for b in (d_w, d_x, d_p, d_out):
            b.free()


@pytest.mark.parametrize("name", ["q4_k", "q5_k", "q6_k"])
@pytest.mark.parametrize("N", [17, 23, 31, 32, 33, 48, 64, 100])
def test_passes_of_32_rows(hip, oracle, name, N):
    """From 17 activation rows on, Q4_K / Q5_K (and Q6_K with 16-byte aligned rows: K = 2048 here; K = 7168 keeps the
    16-row passes) take 32 rows per pass (all 32 rows of the matrix-core product): full and
    partial passes, ragged row groups, K split within the workgroup and across workgroups, bias, float16 epilogue."""
    kind = KINDS[name]
    for M, K in ((203, 2048), (64, 7168)):
        blocks = oracle.quantize(kind, gaussian(380, (M, K), 0.02))
        x = gaussian(381 + N, (N, K))
        bias = gaussian(382, (M,))
        got = hip.linear(x, blocks, kind, M, bias=bias)
        assert "mmq_" in hip.last_route()
        assert_matmul_parity(got, oracle.matmul(kind, blocks, x, M, bias=bias), what=f"{name} {M}x{K} N={N}")
    x16 = x.astype(np.float16)
    ref16 = oracle.matmul(kind, blocks, x16, M, out_dtype=np.float16, force_pack=True)
    got16 = hip.linear(x16, blocks, kind, M, out_dtype=np.float16, force_pack=True)
    assert np.max(np.abs(got16.astype(np.float32) - ref16.astype(np.float32))) <= \
        2e-3 * np.abs(ref16.astype(np.float32)).max()


def test_row_owning_and_streaming_small_batch_kernels(hip, oracle, monkeypatch):
    """Q4_K with up to 16 rows has two small-batch kernels: the row-owning one (fp32 rows quantized inside the kernel, or
    packed rows copied into LDS by its loaders) and the streaming one with a workgroup per 32 weight rows, which a
    device object created with MARMOT_HIP_NO_ROW_KERNELS keeps using. Both against the oracle, and bit-exact on single
    blocks; the row-owning kernel with one and several row groups per workgroup, K split over 1..12 consumers, ragged
    rows and blocks, and a ring that is reused."""
    from marmot_amd import HipBackend

    monkeypatch.setenv("MARMOT_HIP_NO_ROW_KERNELS", "1")
    streaming = HipBackend(0)
    monkeypatch.delenv("MARMOT_HIP_NO_ROW_KERNELS")
    kind = KIND_Q4_K
    try:
        rng = np.random.default_rng(380)
        blocks = random_valid_blocks(rng, kind, 300, 256)
        for N in (3, 8, 16):
            x = gaussian(381 + N, (N, 256))
            ref = oracle.matmul(kind, blocks, x, 300)
            for dev, route in ((hip, "mmq_rows_q4_k_q8_k"), (streaming, "mmq_q4_k_q8_k_mfma")):
                got = dev.linear(x, blocks, kind, 300)
                assert dev.last_route().startswith(route), dev.last_route()
                assert np.array_equal(bits(got), bits(ref)), f"single block N={N} {route}"
        # (M, K, N): 5000 rows = 2 row groups of 10 per workgroup; 1500 x 2560: 6 rows per workgroup, 10 blocks in
        # tasks of 3 (the last one short); 700 x 14336 packed (N * K too large to quantize in the kernel);
        # 40000 x 1024: 10 row groups per workgroup, one consumer each, ring reused
        for M, K, N in ((5000, 1024, 3), (1500, 2560, 7), (4096, 4096, 16), (700, 14336, 5), (40000, 1024, 4),
                        (1000, 4096, 12)):
            w = oracle.quantize(kind, gaussian(390 + M, (M, K), 0.02))
            x = gaussian(391 + M + N, (N, K))
            ref = oracle.matmul(kind, w, x, M, threads=16)
            got = hip.linear(x, w, kind, M)
            assert "mmq_rows" in hip.last_route(), (M, K, N, hip.last_route())
            assert_matmul_parity(got, ref, what=f"row-owning {M}x{K} N={N} {hip.last_route()}")
            old = streaming.linear(x, w, kind, M)
            assert streaming.last_route() == "mmq_q4_k_q8_k_mfma"
            assert_matmul_parity(old, ref, what=f"streaming {M}x{K} N={N}")
    finally:
        streaming.close()


# ---------------------------------------------------------------- tiled int8 GEMM (Q4_K, 33 activation rows and more)
@pytest.mark.parametrize("N,M,K", [(33, 96, 512), (40, 4096, 1024), (48, 128, 256), (64, 100, 512), (100, 203, 2048), (130, 300, 1024), (64, 128, 4096),
                                   (192, 64, 7168), (512, 512, 4096)])
@pytest.mark.parametrize("name", ["q4_k", "q5_k"])
def test_tiled_int8_gemm_matches_oracle(hip, oracle, name, N, M, K):
    """Prefill with fp32 activations: 128 rows x 64 tokens per workgroup on the int8 matrix cores. Full and ragged
    tiles in both directions, one to 28 blocks per row, K split across workgroups when the tiles do not fill the chip
    (partials + ordered reduction), bias."""
    kind = KINDS[name]
    blocks = oracle.quantize(kind, gaussian(400 + N, (M, K), 0.02))
    x = gaussian(401 + N, (N, K))
    bias = gaussian(402, (M,))
    got = hip.linear(x, blocks, kind, M, bias=bias)
    assert hip.last_route() == f"mmq_{name}_q8_k_mfma_tile"
    assert_matmul_parity(got, oracle.matmul(kind, blocks, x, M, bias=bias), what=f"{name} tile {M}x{K} N={N}")


@pytest.mark.parametrize("name", ["q4_k", "q5_k"])
def test_tiled_int8_gemm_random_blocks_and_the_pass_kernel(hip, oracle, monkeypatch, name):
    """Arbitrary block bytes (every nibble, scale and min pattern) against the oracle; a device object created with
    MARMOT_HIP_NO_GEMM_I8 keeps the 32-row passes of the streaming kernel, and both kernels agree within the bound."""
    from marmot_amd import HipBackend

    kind = KINDS[name]
    N, M, K = 96, 160, 1536
    blocks = random_valid_blocks(np.random.default_rng(410), kind, M, K)
    x = gaussian(411, (N, K))
    ref = oracle.matmul(kind, blocks, x, M)
    tiled = hip.linear(x, blocks, kind, M)
    assert hip.last_route() == f"mmq_{name}_q8_k_mfma_tile"
    assert_matmul_parity(tiled, ref, what="tile, random blocks")
    monkeypatch.setenv("MARMOT_HIP_NO_GEMM_I8", "1")
    passes = HipBackend(0)
    monkeypatch.delenv("MARMOT_HIP_NO_GEMM_I8")
    try:
        got = passes.linear(x, blocks, kind, M)
        assert passes.last_route() == f"mmq_{name}_q8_k_mfma"
        assert_matmul_parity(got, ref, what="passes, random blocks")
        assert_matmul_parity(tiled, got, what="tile against passes")
    finally:
        passes.close()


@pytest.mark.parametrize("name", ["q4_k", "q5_k"])
def test_tiled_int8_gemm_integers_are_exact(hip, name):
    """Packed activations and weight blocks whose scales are powers of two: every fp32 operation of the kernel except
    the one addition per block is then exact, so the output must equal, bit for bit, the block sums
    a.d * (w.d * isum - w.dmin * msum) formed in exact integer arithmetic and added in block order."""
    kind = KINDS[name]
    q5 = name == "q5_k"
    bb, qs_off = (176, 48) if q5 else (144, 16)
    N, M, K = 70, 200, 512
    nb = K // 256
    rng = np.random.default_rng(420)
    blocks = random_valid_blocks(rng, kind, M, K).reshape(M, nb, bb).copy()
    d_exp = rng.integers(-12, -6, size=(M, nb))
    m_exp = rng.integers(-12, -6, size=(M, nb))
    blocks[:, :, 0:2] = np.ldexp(1.0, d_exp).astype(np.float16).view(np.uint8).reshape(M, nb, 2)
    blocks[:, :, 2:4] = np.ldexp(1.0, m_exp).astype(np.float16).view(np.uint8).reshape(M, nb, 2)
    q = rng.integers(-127, 128, size=(N, K)).astype(np.int8)
    a_exp = rng.integers(-8, -2, size=(N, nb))
    lay = hip.packed_activation_layout(kind, N, K)
    image = np.zeros(lay.total_bytes, np.uint8)
    vals = np.zeros((N, lay.values_per_row), np.int8)
    vals[:, :K] = q
    image[lay.values_offset:lay.values_offset + vals.size] = vals.view(np.uint8).reshape(-1)
    ad = np.ldexp(1.0, a_exp).astype(np.float32)
    image[lay.scales_offset:lay.scales_offset + ad.nbytes] = ad.view(np.uint8).reshape(-1)
    sums = q.reshape(N, K // 16, 16).astype(np.int16).sum(axis=2, dtype=np.int16)
    image[lay.sums_offset:lay.sums_offset + sums.nbytes] = sums.view(np.uint8).reshape(-1)
    # integer block sums from the block bytes (get_scale_min_k4, kquant_common.h:29-37; nibble order q4k_gguf.c)
    sc = np.zeros((M, nb, 8), np.int64)
    mn = np.zeros((M, nb, 8), np.int64)
    s12 = blocks[:, :, 4:16].astype(np.int64)
    for jj in range(8):
        if jj < 4:
            sc[:, :, jj] = s12[:, :, jj] & 63
            mn[:, :, jj] = s12[:, :, jj + 4] & 63
        else:
            sc[:, :, jj] = (s12[:, :, jj + 4] & 15) | ((s12[:, :, jj - 4] >> 6) << 4)
            mn[:, :, jj] = (s12[:, :, jj + 4] >> 4) | ((s12[:, :, jj] >> 6) << 4)
    qs = blocks[:, :, qs_off:qs_off + 128].reshape(M, nb, 4, 32).astype(np.int64)
    wq = np.zeros((M, nb, 8, 32), np.int64)
    wq[:, :, 0::2, :] = qs & 15
    wq[:, :, 1::2, :] = qs >> 4
    if q5:  # bit sb of qh[l] is the fifth bit of value l of sub-block sb (q5k_gguf.c:162-198)
        qh = blocks[:, :, 16:48].astype(np.int64)
        for sb_ in range(8):
            wq[:, :, sb_, :] += ((qh >> sb_) & 1) << 4
    a = q.reshape(N, nb, 8, 32).astype(np.int64)
    want = np.zeros((N, M), np.float32)
    for b in range(nb):
        dots = np.einsum("nsk,msk->nms", a[:, b], wq[:, b])                      # [N, M, 8]
        isum = (dots * sc[None, :, b, :]).sum(axis=2)
        msum = (a[:, b].sum(axis=2)[:, None, :] * mn[None, :, b, :]).sum(axis=2)
        assert np.abs(isum).max() < 2 ** 24 and np.abs(msum).max() < 2 ** 24
        v = (np.ldexp(1.0, d_exp[None, :, b]) * isum - np.ldexp(1.0, m_exp[None, :, b]) * msum).astype(np.float32)
        want = (want + (np.ldexp(1.0, a_exp[:, b, None]).astype(np.float32) * v)).astype(np.float32)
    d_w, d_p, d_out = hip.to_device(blocks.reshape(M, nb * bb)), hip.to_device(image), hip.alloc(N * M * 4)
    hip.linear_prepacked_d(kind, d_w, d_p, N, K, M, d_out)
    assert hip.last_route() == f"mmq_{name}_q8_k_mfma_tile"
    got = d_out.download(np.float32, (N, M))
    for b_ in (d_w, d_p, d_out):
        b_.free()
    assert np.array_equal(bits(got), bits(want))


@pytest.mark.parametrize("N,M,K", [(33, 96, 2048), (64, 128, 2048), (100, 203, 4096), (130, 300, 6144), (64, 128, 14336),
                                   (512, 512, 4096)])
def test_tiled_int8_gemm_q6k_matches_oracle(hip, oracle, N, M, K):
    """The Q6_K form of the tile kernel (rows of a multiple of 8 blocks): blocks at every offset inside a 16-byte chunk,
    ragged tiles, K split across workgroups, bias. Rows of another length keep the 32-row passes."""
    kind = KIND_Q6_K
    blocks = oracle.quantize(kind, gaussian(430 + N, (M, K), 0.02))
    x = gaussian(431 + N, (N, K))
    bias = gaussian(432, (M,))
    got = hip.linear(x, blocks, kind, M, bias=bias)
    assert hip.last_route() == "mmq_q6_k_q8_k_mfma_tile"
    assert_matmul_parity(got, oracle.matmul(kind, blocks, x, M, bias=bias), what=f"Q6_K tile {M}x{K} N={N}")
    if K == 2048:
        # rows that are not a multiple of 8 blocks start at any even address (rows of 5, 14 and 43 blocks: the last two
        # are the hidden size of Qwen2-7B and the FFN size of Llama-2-7B): the tile rounds down per row
        for K2 in (1024 + 256, 3584, 11008):
            b2 = oracle.quantize(kind, gaussian(433, (M, K2), 0.02))
            x2 = gaussian(434, (N, K2))
            got2 = hip.linear(x2, b2, kind, M)
            assert hip.last_route() == "mmq_q6_k_q8_k_mfma_tile"
            assert_matmul_parity(got2, oracle.matmul(kind, b2, x2, M), what=f"Q6_K tile, unaligned rows K={K2}")


def test_tiled_int8_gemm_q6k_random_blocks_and_exact_integers(hip, oracle):
    """Arbitrary Q6_K block bytes against the oracle; then packed activations and blocks whose scales are powers of two:
    the output must equal, bit for bit, a.d * w.d * (sum_g sc_g * ((u_g - 32) . a_g)) formed in exact integer
    arithmetic per half block and added the way the kernel adds (each half of a workgroup's blocks in block order, the
    two halves, then the workgroups along K)."""
    kind = KIND_Q6_K
    rng = np.random.default_rng(440)
    for N, M, K in ((70, 200, 2048), (70, 200, 1792), (100, 131, 3328)):  # rows of 8, 7 and 13 blocks
        blocks = random_valid_blocks(rng, kind, M, K)
        x = gaussian(441, (N, K))
        got = hip.linear(x, blocks, kind, M)
        assert hip.last_route() == "mmq_q6_k_q8_k_mfma_tile"
        assert_matmul_parity(got, oracle.matmul(kind, blocks, x, M), what=f"Q6_K tile, random blocks K={K}")
    N, M, K = 70, 200, 1792  # the exact-integer part on rows of 7 blocks: every row starts at another offset mod 16
    nb = K // 256
    blocks = random_valid_blocks(rng, kind, M, K)

    blocks = blocks.reshape(M, nb, 210).copy()
    d_exp = rng.integers(-14, -8, size=(M, nb))
    blocks[:, :, 208:210] = np.ldexp(1.0, d_exp).astype(np.float16).view(np.uint8).reshape(M, nb, 2)
    blocks[:, :, 192:208] = rng.integers(-31, 32, size=(M, nb, 16)).astype(np.int8).view(np.uint8)  # keeps sums < 2^24
    q = rng.integers(-127, 128, size=(N, K)).astype(np.int8)
    a_exp = rng.integers(-8, -2, size=(N, nb))
    lay = hip.packed_activation_layout(kind, N, K)
    image = np.zeros(lay.total_bytes, np.uint8)
    vals = np.zeros((N, lay.values_per_row), np.int8)
    vals[:, :K] = q
    image[lay.values_offset:lay.values_offset + vals.size] = vals.view(np.uint8).reshape(-1)
    ad = np.ldexp(1.0, a_exp).astype(np.float32)
    image[lay.scales_offset:lay.scales_offset + ad.nbytes] = ad.view(np.uint8).reshape(-1)
    sums = q.reshape(N, K // 16, 16).astype(np.int16).sum(axis=2, dtype=np.int16)
    image[lay.sums_offset:lay.sums_offset + sums.nbytes] = sums.view(np.uint8).reshape(-1)
    # the 6-bit values of a block (q6k_gguf.c:63-99): value 128 h + 32 q + l = (ql[64 h + 32 (q & 1) + l] nibble q >> 1)
    # | ((qh[32 h + l] >> 2 q) & 3) << 4, minus 32; group 16 values
    ql = blocks[:, :, 0:128].astype(np.int64).reshape(M, nb, 2, 2, 32)    # [h][q & 1][l]
    qh = blocks[:, :, 128:192].astype(np.int64).reshape(M, nb, 2, 32)     # [h][l]
    u = np.zeros((M, nb, 2, 4, 32), np.int64)
    for qq in range(4):
        nib = (ql[:, :, :, qq & 1, :] >> 4) if (qq >> 1) else (ql[:, :, :, qq & 1, :] & 15)
        u[:, :, :, qq, :] = nib | (((qh >> (2 * qq)) & 3) << 4)
    w = (u - 32).reshape(M, nb, 2, 8, 16)                                  # [half][group of the half][16]
    sc = blocks[:, :, 192:208].view(np.int8).astype(np.int64).reshape(M, nb, 2, 8)
    a = q.astype(np.int64).reshape(N, nb, 2, 8, 16)
    # four tiles on a chip of `cus` compute units: K is split over workgroups (at least two blocks each), every
    # workgroup adds its two halves, and the reduction adds the workgroups' partial sums in order, starting from zero
    cus = hip.caps()["num_compute_units"]
    tiles = -(-N // 64) * -(-M // 128)
    splits = min(cus // tiles, nb // 2) if tiles * 2 <= cus else 1
    per_split = -(-nb // max(splits, 1))
    want = np.zeros((N, M), np.float32)
    for b_lo in range(0, nb, per_split):
        halves = [np.zeros((N, M), np.float32), np.zeros((N, M), np.float32)]
        for b in range(b_lo, min(nb, b_lo + per_split)):
            scale = (np.ldexp(1.0, a_exp[:, b, None]).astype(np.float32) *
                     np.ldexp(1.0, d_exp[None, :, b]).astype(np.float32))
            for h in range(2):
                dots = np.einsum("ngk,mgk->nmg", a[:, b, h], w[:, b, h])      # [N, M, 8]
                isum = (dots * sc[None, :, b, h, :]).sum(axis=2)
                assert np.abs(isum).max() < 2 ** 24
                halves[h] = (halves[h] + scale * isum.astype(np.float32)).astype(np.float32)
        part = (halves[0] + halves[1]).astype(np.float32)
        want = part if per_split >= nb else (want + part).astype(np.float32)
    d_w, d_p, d_out = hip.to_device(blocks.reshape(M, nb * 210)), hip.to_device(image), hip.alloc(N * M * 4)
    hip.linear_prepacked_d(kind, d_w, d_p, N, K, M, d_out)
    assert hip.last_route() == "mmq_q6_k_q8_k_mfma_tile"
    got = d_out.download(np.float32, (N, M))
    for b_ in (d_w, d_p, d_out):
        b_.free()
    assert np.array_equal(bits(got), bits(want))


# ---------------------------------------------------------------- tiled int8 GEMM for the 32-value formats (Q8_0, Q4_0)
Q80_KINDS = {"q8_0": 5, "q4_0": 1, "q4_1": 2, "q5_0": 3, "q5_1": 4}


@pytest.mark.parametrize("N,M,K", [(9, 70, 256), (20, 300, 512), (32, 128, 1024), (33, 96, 512), (40, 4096, 1024),
                                   (48, 128, 256), (64, 100, 512),
                                   (100, 203, 2048), (130, 300, 1024), (64, 128, 4096), (192, 64, 7168),
                                   (512, 512, 4096)])
@pytest.mark.parametrize("name", ["q8_0", "q4_0", "q4_1", "q5_0", "q5_1"])
def test_tiled_int8_gemm_32_value_formats_match_oracle(hip, oracle, name, N, M, K):
    """Prefill with fp32 activations for Q8_0 / Q4_0 / Q4_1 / Q5_0 / Q5_1 weights (activations packed to Q8_0): one
    int8 matrix instruction per 32-value block and 32 x 32 outputs, the two block scales applied per output and block
    as in cpu_vec_dot_q8_0_q8_0 (vec_dot_impl.h:452-479), the minimum of Q4_1 / Q5_1 times the token's scaled code sum
    added per block (:186-217, :288-349). Full and ragged tiles, one to 28 rounds of 256 values, K split across
    workgroups when the tiles do not fill the chip, bias."""
    kind = Q80_KINDS[name]
    blocks = oracle.quantize(kind, gaussian(430 + N, (M, K), 0.02))
    x = gaussian(431 + N, (N, K))
    bias = gaussian(432, (M,))
    got = hip.linear(x, blocks, kind, M, bias=bias)
    assert hip.last_route() == f"gemm_{name}_q8_0_mfma_tile"
    assert_matmul_parity(got, oracle.matmul(kind, blocks, x, M, bias=bias), what=f"{name} tile {M}x{K} N={N}")


@pytest.mark.parametrize("name", ["q8_0", "q4_0", "q4_1", "q5_0", "q5_1"])
def test_tiled_int8_gemm_32_value_formats_random_blocks_routes_and_epilogues(hip, oracle, monkeypatch, name):
    """Arbitrary block bytes (every code, scales of both signs down to fp16 denormals) against the oracle and against
    the packed matvec that a device object created with MARMOT_HIP_NO_GEMM_I8 keeps; shapes the tile does not cover
    (K not a multiple of 256, fewer than nine rows) stay on the matvec; fp16 output with an fp16 bias; the dual call
    equals two single calls bit for bit."""
    from marmot_amd import HipBackend

    kind = Q80_KINDS[name]
    N, M, K = 96, 160, 1536
    blocks = random_valid_blocks(np.random.default_rng(440), kind, M, K)
    x = gaussian(441, (N, K))
    ref = oracle.matmul(kind, blocks, x, M)
    tiled = hip.linear(x, blocks, kind, M)
    assert hip.last_route() == f"gemm_{name}_q8_0_mfma_tile"
    assert_matmul_parity(tiled, ref, what="tile, random blocks")
    monkeypatch.setenv("MARMOT_HIP_NO_GEMM_I8", "1")
    plain = HipBackend(0)
    monkeypatch.delenv("MARMOT_HIP_NO_GEMM_I8")
    try:
        got = plain.linear(x, blocks, kind, M)
        assert plain.last_route() == f"matvec_{name}_q8_0"
        assert_matmul_parity(got, ref, what="matvec, random blocks")
        assert_matmul_parity(tiled, got, what="tile against matvec")
    finally:
        plain.close()
    for n2, k2 in ((8, 1536), (96, 1536 + 32)):
        b2 = oracle.quantize(kind, gaussian(442, (M, k2), 0.02))
        x2 = gaussian(443, (n2, k2))
        got = hip.linear(x2, b2, kind, M)
        assert hip.last_route() == f"matvec_{name}_q8_0", (n2, k2, hip.last_route())
        assert_matmul_parity(got, oracle.matmul(kind, b2, x2, M), what=f"{name} N={n2} K={k2}")
    soft = oracle.quantize(kind, gaussian(444, (M, K), 0.02))
    bias16 = gaussian(445, (M,)).astype(np.float16)
    x16 = x.astype(np.float16)  # fp16 activations forced through the packed path, fp16 output
    got16 = hip.linear(x16, soft, kind, M, bias=bias16, out_dtype=np.float16, force_pack=True)
    assert hip.last_route() == f"gemm_{name}_q8_0_mfma_tile"
    ref16 = oracle.matmul(kind, soft, x16, M, bias=bias16, out_dtype=np.float16, force_pack=True)
    assert np.max(np.abs(got16.astype(np.float32) - ref16.astype(np.float32))) <= 2e-3 * np.max(np.abs(ref16.astype(np.float32)))
    other = oracle.quantize(kind, gaussian(446, (M, K), 0.02))
    a, b = hip.linear_dual(x, soft, other, kind, M)
    assert hip.last_route() == f"gemm_{name}_q8_0_mfma_tile"
    assert np.array_equal(bits(a), bits(hip.linear(x, soft, kind, M)))
    assert np.array_equal(bits(b), bits(hip.linear(x, other, kind, M)))
    # activations packed once by the caller, K split across workgroups (one tile: four splits), with a bias: the same
    # bits as the call that packs for itself
    from marmot_amd import DT_F32
    n3, m3, k3 = 40, 128, 2048
    w3 = oracle.quantize(kind, gaussian(447, (m3, k3), 0.02))
    x3 = gaussian(448, (n3, k3))
    b3 = gaussian(449, (m3,))
    d_w, d_x, d_b = hip.to_device(w3), hip.to_device(x3), hip.to_device(b3)
    d_p, d_out = hip.alloc(hip.packed_activation_bytes(kind, n3, k3)), hip.alloc(n3 * m3 * 4)
    hip.pack_activations_d(kind, d_x, DT_F32, n3, k3, d_p)
    hip.linear_prepacked_d(kind, d_w, d_p, n3, k3, m3, d_out, d_bias=d_b)
    assert hip.last_route() == f"gemm_{name}_q8_0_mfma_tile"
    pre = d_out.download(np.float32, (n3, m3))
    for b_ in (d_w, d_x, d_b, d_p, d_out):
        b_.free()
    assert np.array_equal(bits(pre), bits(hip.linear(x3, w3, kind, m3, bias=b3)))
    assert_matmul_parity(pre, oracle.matmul(kind, w3, x3, m3, bias=b3), what=f"{name} prepacked, K split")


Q23K_KINDS = {"q2_k": 7, "q3_k": 8}


@pytest.mark.parametrize("N,M,K", [(9, 70, 256), (20, 300, 512), (32, 128, 1024), (33, 96, 512), (40, 4096, 1024),
                                   (64, 100, 512), (100, 203, 2048),
                                   (130, 300, 1024), (64, 128, 4096), (192, 64, 7168), (512, 512, 4096)])
@pytest.mark.parametrize("name", ["q2_k", "q3_k"])
def test_tiled_int8_gemm_q2k_q3k_match_oracle(hip, oracle, name, N, M, K):
    """Prefill with fp32 activations for Q2_K / Q3_K weights (activations packed to Q8_K): group scales multiplied into
    the int8 operands, two chains of matrix instructions per block (Q2_K: scaled values and group minima; Q3_K: the
    value split into a signed high part and a low bit), cpu_vec_dot_q2_k_q8_k / cpu_vec_dot_q3_k_q8_k
    (vec_dot_impl.h:560-687). Full and ragged tiles, one to 28 blocks, K split across workgroups, bias."""
    kind = Q23K_KINDS[name]
    blocks = oracle.quantize(kind, gaussian(460 + N, (M, K), 0.02))
    x = gaussian(461 + N, (N, K))
    bias = gaussian(462, (M,))
    got = hip.linear(x, blocks, kind, M, bias=bias)
    assert hip.last_route() == f"gemm_{name}_q8_k_mfma_tile"
    assert_matmul_parity(got, oracle.matmul(kind, blocks, x, M, bias=bias), what=f"{name} tile {M}x{K} N={N}")


@pytest.mark.parametrize("name", ["q2_k", "q3_k"])
def test_tiled_int8_gemm_q2k_q3k_random_blocks_and_routes(hip, oracle, monkeypatch, name):
    """Arbitrary block bytes (every two-bit value, mask bit, group scale and minimum, Q3_K's scale -32 with value -4
    included: their product, +128, does not fit a signed byte) against the oracle and against the packed matvec of a
    device object created with MARMOT_HIP_NO_GEMM_I8; fewer than five rows stay on the matvec; the dual call equals two
    single calls bit for bit."""
    from marmot_amd import HipBackend

    kind = Q23K_KINDS[name]
    N, M, K = 96, 160, 1536
    blocks = random_valid_blocks(np.random.default_rng(470), kind, M, K)
    x = gaussian(471, (N, K))
    ref = oracle.matmul(kind, blocks, x, M)
    tiled = hip.linear(x, blocks, kind, M)
    assert hip.last_route() == f"gemm_{name}_q8_k_mfma_tile"
    assert_matmul_parity(tiled, ref, what="tile, random blocks")
    monkeypatch.setenv("MARMOT_HIP_NO_GEMM_I8", "1")
    plain = HipBackend(0)
    monkeypatch.delenv("MARMOT_HIP_NO_GEMM_I8")
    try:
        got = plain.linear(x, blocks, kind, M)
        assert plain.last_route() == f"matvec_{name}_q8_k"
        assert_matmul_parity(got, ref, what="matvec, random blocks")
        assert_matmul_parity(tiled, got, what="tile against matvec")
    finally:
        plain.close()
    for n_small, route in ((4, f"matvec_{name}_q8_k_fused"), (5, f"gemm_{name}_q8_k_mfma_tile"),
                           (8, f"gemm_{name}_q8_k_mfma_tile")):
        xs = gaussian(472 + n_small, (n_small, K))
        got = hip.linear(xs, blocks, kind, M)
        assert hip.last_route() == route, (n_small, hip.last_route())
        assert_matmul_parity(got, oracle.matmul(kind, blocks, xs, M), what=f"{name} N={n_small}")
    other = random_valid_blocks(np.random.default_rng(473), kind, M, K)
    a, b = hip.linear_dual(x, blocks, other, kind, M)
    assert hip.last_route() == f"gemm_{name}_q8_k_mfma_tile"
    assert np.array_equal(bits(a), bits(tiled))
    assert np.array_equal(bits(b), bits(hip.linear(x, other, kind, M)))


@pytest.mark.parametrize("name", ["q8_0", "q4_0", "q5_0"])
def test_tiled_int8_gemm_32_value_formats_integers_are_exact(hip, name):
    """Packed activations and weight blocks whose scales are powers of two: the integer dot, its conversion and the
    product of the two scales are then exact, and what is left is one rounding per block in the multiply-add that
    accumulates it. The output must equal, bit for bit, that chain formed from exact integer dots: blocks 0..3 and
    4..7 of the one round of 256 values are accumulated separately, each in block order, and the two sums are added."""
    kind = Q80_KINDS[name]
    q8 = name == "q8_0"
    bb = {"q8_0": 34, "q4_0": 18, "q5_0": 22}[name]
    N, M, K = 70, 200, 256
    nb = K // 32
    rng = np.random.default_rng(450)
    blocks = random_valid_blocks(rng, kind, M, K).reshape(M, nb, bb).copy()
    d_exp = rng.integers(-12, -6, size=(M, nb))
    blocks[:, :, 0:2] = np.ldexp(1.0, d_exp).astype(np.float16).view(np.uint8).reshape(M, nb, 2)
    q = rng.integers(-127, 128, size=(N, K)).astype(np.int8)
    a_exp = rng.integers(-8, -2, size=(N, nb))
    lay = hip.packed_activation_layout(kind, N, K)
    image = np.zeros(lay.total_bytes, np.uint8)
    vals = np.zeros((N, lay.values_per_row), np.int8)
    vals[:, :K] = q
    image[lay.values_offset:lay.values_offset + vals.size] = vals.view(np.uint8).reshape(-1)
    ad = np.ldexp(1.0, a_exp).astype(np.float32)
    image[lay.scales_offset:lay.scales_offset + ad.nbytes] = ad.view(np.uint8).reshape(-1)
    if q8:
        wq = blocks[:, :, 2:].view(np.int8).astype(np.int64)                       # [M, nb, 32]
    elif name == "q4_0":  # byte i: value i in the low nibble, value 16 + i in the high nibble, both minus 8
        qs = blocks[:, :, 2:].astype(np.int64)
        wq = np.concatenate([(qs & 15) - 8, (qs >> 4) - 8], axis=2)
    else:  # Q5_0: bit i of the 32-bit word at byte 2 is value i's fifth bit; the values minus 16
        qs = blocks[:, :, 6:].astype(np.int64)
        qh = blocks[:, :, 2:6].copy().view(np.uint32).astype(np.int64)          # [M, nb, 1]
        fifth = (qh >> np.arange(32)) & 1                                          # [M, nb, 32]
        wq = np.concatenate([qs & 15, qs >> 4], axis=2) + 16 * fifth - 16
    a = q.reshape(N, nb, 32).astype(np.int64)
    dots = np.einsum("nbk,mbk->nmb", a, wq)                                        # [N, M, nb]
    scale = np.ldexp(1.0, a_exp[:, None, :] + d_exp[None, :, :])
    terms = dots * scale                                                           # exact in float64
    halves = []
    for first in (0, 4):
        acc = np.zeros((N, M), np.float32)
        for b in range(first, first + 4):  # fp32 fused multiply-add: one rounding of the exact sum
            acc = (acc.astype(np.float64) + terms[:, :, b]).astype(np.float32)
        halves.append(acc)
    want = halves[0] + halves[1]
    d_w, d_p, d_out = hip.to_device(blocks.reshape(M, nb * bb)), hip.to_device(image), hip.alloc(N * M * 4)
    hip.linear_prepacked_d(kind, d_w, d_p, N, K, M, d_out)
    assert hip.last_route() == f"gemm_{name}_q8_0_mfma_tile"
    got = d_out.download(np.float32, (N, M))
    for b_ in (d_w, d_p, d_out):
        b_.free()
    assert np.array_equal(bits(got), bits(want))
