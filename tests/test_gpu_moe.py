"""GPU parity, part 3: top-k, router softmax and the grouped MoE expert FFN against the CPU oracle."""
import numpy as np
import pytest

from oracle.pyoracle import KIND_Q2_K, KIND_Q3_K, KIND_Q4_1, KIND_Q4_K, KIND_Q5_0, KIND_Q5_1, KIND_Q5_K, KIND_Q6_K, KIND_Q8_0
from tests.test_oracle_moe import make_experts
from oracle.pyoracle import KIND_Q8_K
from tests.util import assert_matmul_parity, assert_moe_parity, gaussian, parity_metrics, quantize_weights

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def hip():
    from marmot_amd import HipBackend

    b = HipBackend(0)
    yield b
    b.close()


def test_topk_reference_tie_case(hip):
    x = np.array([[1, 4, 4, 2, -1], [0, -3, 5, 5, 1]], dtype=np.float32)
    vals, idx = hip.topk(x, 3)
    assert np.array_equal(vals, np.array([[4, 4, 2], [5, 5, 1]], dtype=np.float32))
    assert np.array_equal(idx, np.array([[1, 2, 3], [2, 3, 4]], dtype=np.int32))


def test_topk_special_values(hip, oracle):
    """Infinities, NaNs, -FLT_MAX (never selected: the list starts at -FLT_MAX and only strictly larger values go
    in), k == cols, rows with fewer than k selectable values, a ragged column count."""
    fmax = np.finfo(np.float32).max
    x = np.array([[np.inf, 1, np.inf, -np.inf, np.nan, 1, -fmax, 0, 2, np.nan, -1],
                  [np.nan, np.nan, -np.inf, -fmax, -np.inf, np.nan, -fmax, 7, np.nan, 7, -np.inf],
                  [-np.inf] * 11,
                  [0, -0.0, 0, -0.0, 5, 5, 5, -3, -3, 1e-45, -1e-45]], dtype=np.float32)
    for k in (1, 4, 11):
        v, i = hip.topk(x, k)
        ov, oi = oracle.topk(x, k)
        assert np.array_equal(i, oi), (k, i, oi)
        assert np.array_equal(v.view(np.uint32), ov.view(np.uint32)), (k, v, ov)
    assert i[2].tolist() == [-1] * 11 and np.all(v[2] == -fmax)
    rng = np.random.default_rng(11)
    x = rng.integers(-3, 4, size=(9, 333)).astype(np.float32)
    v, i = hip.topk(x, 40)
    ov, oi = oracle.topk(x, 40)
    assert np.array_equal(i, oi) and np.array_equal(v, ov)


def test_topk_and_softmax_match_oracle(hip, oracle):
    rng = np.random.default_rng(7)
    x = rng.integers(-4, 5, size=(130, 128)).astype(np.float32)
    v, i = hip.topk(x, 8)
    ov, oi = oracle.topk(x, 8)
    assert np.array_equal(i, oi) and np.array_equal(v, ov)
    logits = gaussian(8, (64, 128))
    v, i = hip.topk(logits, 8)
    ov, oi = oracle.topk(logits, 8)
    assert np.array_equal(i, oi) and np.array_equal(v.view(np.uint32), ov.view(np.uint32))
    sm = hip.softmax_rows(v)
    assert np.allclose(sm, oracle.softmax_rows(ov), rtol=1e-6, atol=0)


@pytest.mark.parametrize("kind_gu,kind_dn", [(KIND_Q4_K, KIND_Q4_K), (KIND_Q4_K, KIND_Q6_K), (KIND_Q8_0, KIND_Q8_0),
                                             (KIND_Q5_K, KIND_Q5_K), (KIND_Q5_K, KIND_Q6_K),
                                             (KIND_Q5_0, KIND_Q5_1), (KIND_Q4_1, KIND_Q8_0),
                                             (KIND_Q2_K, KIND_Q3_K), (KIND_Q3_K, KIND_Q6_K)])
@pytest.mark.parametrize("T", [1, 3, 4, 5, 17, 64])
def test_moe_small(hip, oracle, kind_gu, kind_dn, T):
    """Decode-order path (T <= 4) and grouped path, several routes per expert (more than one work item)."""
    print(f"moe small kinds={kind_gu}/{kind_dn} T={T}", flush=True)
    E, F, H, k = 6, 256, 512, 3
    gate, up, down = make_experts(oracle, 400, E, F, H, kind_gu, kind_dn)
    hidden = gaussian(410 + T, (T, H))
    vals, ids = oracle.topk(gaussian(411 + T, (T, E)), k)
    w = oracle.softmax_rows(vals)
    ref = oracle.moe_experts(hidden, gate, up, down, ids, w, F, E, kind_gu, kind_dn, threads=8)
    got = hip.moe_experts(hidden, gate, up, down, ids, w, F, E, kind_gu, kind_dn)
    assert_moe_parity(got, ref, what=f"moe T={T}")


@pytest.mark.parametrize("T", [200, 1400])
def test_moe_many_routes(hip, oracle, T):
    """Route sort over several chunks of routes (one per wavefront), below and above the number of routes whose ids
    fit in LDS (4096); every expert gets many work items."""
    print(f"moe many routes T={T}", flush=True)
    E, F, H, k = 7, 256, 256, 3
    kind = KIND_Q4_K
    gate, up, down = make_experts(oracle, 430, E, F, H, kind, kind)
    hidden = gaussian(431 + T, (T, H))
    vals, ids = oracle.topk(gaussian(432 + T, (T, E)), k)
    w = oracle.softmax_rows(vals)
    ref = oracle.moe_experts(hidden, gate, up, down, ids, w, F, E, kind, kind, threads=8)
    got = hip.moe_experts(hidden, gate, up, down, ids, w, F, E, kind, kind)
    assert_moe_parity(got, ref, what=f"moe many routes T={T}")


def test_moe_q6k_experts_with_aligned_rows(hip, oracle):
    """Q6_K experts whose rows hold a multiple of 8 blocks (K = 2048): the grouped matmuls take the loader/consumer
    kernel with its 16-byte aligned row copies, both the dual gate/up launch and the down launch."""
    E, F, H, k, T = 4, 2048, 2048, 2, 9
    kind = KIND_Q6_K
    gate, up, down = make_experts(oracle, 440, E, F, H, kind, kind)
    hidden = gaussian(441, (T, H))
    vals, ids = oracle.topk(gaussian(442, (T, E)), k)
    w = oracle.softmax_rows(vals)
    ref = oracle.moe_experts(hidden, gate, up, down, ids, w, F, E, kind, kind, threads=8)
    got = hip.moe_experts(hidden, gate, up, down, ids, w, F, E, kind, kind)
    assert_moe_parity(got, ref, what="moe Q6_K aligned rows")


def test_moe_policies_duplicates_unrouted_and_errors(hip, oracle):
    from marmot_amd import MarmotHipError

    E, F, H, k = 5, 256, 256, 2
    kind = KIND_Q4_K
    gate, up, down = make_experts(oracle, 420, E, F, H, kind, kind)
    T = 7
    hidden = gaussian(421, (T, H))
    ids = np.array([[0, 1], [1, 1], [4, 2], [2, 4], [0, 0], [3, 1], [1, 3]], dtype=np.int32)
    w = np.abs(gaussian(422, (T, k))) + 0.1
    for policy, scale in ((0, 1.0), (1, 2.5), (2, 1.0), (2, 0.5)):
        ref = oracle.moe_experts(hidden, gate, up, down, ids, w, F, E, kind, kind, weights_scale=scale, policy=policy)
        got = hip.moe_experts(hidden, gate, up, down, ids, w, F, E, kind, kind, weights_scale=scale, policy=policy)
        assert_moe_parity(got, ref, what=f"moe policy={policy}")
    bad = ids.copy()
    bad[3, 1] = E
    with pytest.raises(MarmotHipError) as e:
        hip.moe_experts(hidden, gate, up, down, bad, w, F, E, kind, kind)
    assert e.value.code == -1
    with pytest.raises(MarmotHipError) as e:
        hip.moe_experts(hidden, gate, up, down, ids, w, F, E, kind, kind, ffn_type=1)  # GELU FFN: not implemented
    assert e.value.code == -8


Q8K_BLOCK_BYTES = 292  # marmot_q8_k_block_t: float d, int8 qs[256], int16 bsums[16]


def split_packed_image(lay, rows: int, image: np.ndarray):
    """(values int8 [rows, values_per_row], scales fp32 [rows, blocks], sums int16 [rows, blocks * sums_per_block])"""
    kp, nb, spb = lay.values_per_row, lay.blocks_per_row, lay.sums_per_block
    q = image[lay.values_offset:lay.values_offset + rows * kp].view(np.int8).reshape(rows, kp)
    d = image[lay.scales_offset:lay.scales_offset + rows * nb * 4].view(np.float32).reshape(rows, nb)
    sums = image[lay.sums_offset:lay.sums_offset + rows * nb * spb * 2].view(np.int16).reshape(rows, nb * spb)
    return q, d, sums


def packed_image_from_q8k_blocks(lay, blocks: np.ndarray) -> np.ndarray:
    """blocks: uint8 [rows, blocks_per_row * 292] of marmot_q8_k_block_t -> the library's packed image."""
    rows = blocks.shape[0]
    b = blocks.reshape(rows, lay.blocks_per_row, Q8K_BLOCK_BYTES)
    image = np.zeros(lay.total_bytes, dtype=np.uint8)
    q, d, sums = split_packed_image(lay, rows, image)
    d[:] = np.ascontiguousarray(b[:, :, 0:4]).view(np.float32).reshape(rows, -1)
    q[:] = np.ascontiguousarray(b[:, :, 4:260]).view(np.int8).reshape(rows, -1)
    sums[:] = np.ascontiguousarray(b[:, :, 260:292]).view(np.int16).reshape(rows, -1)
    return image


def check_moe_stages(hip, oracle, hidden, gate, up, down, ids, w, F, E, kind, ref, what, tol=1e-3):
    """Every stage of the expert FFN against the oracle's, each at max relative error (denominator floored at
    1e-3 * rms) <= tol: the gate / up projections; the SwiGLU product re-quantized to Q8_K (int8 values may differ
    by one step where the fp32 product sits on a rounding boundary, never by more); and the down projection +
    weighted combine when it is fed the ORACLE's re-quantized activations, which takes the int8 flips out of the
    comparison. Returns the metrics of each stage."""
    T, H = hidden.shape
    k = ids.shape[1]
    routes = T * k
    st = hip.moe_experts_probe(hidden, gate, up, down, ids, w, F, E, kind, kind)
    pos = st["route_pos"]
    assert np.array_equal(np.sort(pos.ravel()), np.arange(routes)), f"{what}: sorted positions are not a permutation"
    assert np.array_equal(st["sorted_tokens"][pos], np.repeat(np.arange(T, dtype=np.uint32)[:, None], k, 1))
    expert_of_pos = np.zeros(routes, dtype=np.int64)
    expert_of_pos[pos.ravel()] = ids.ravel()
    # one run per expert (ascending ids in the grouped order, first-use order in the decode order)
    runs = 1 + int(np.count_nonzero(np.diff(expert_of_pos)))
    assert runs == len(np.unique(expert_of_pos)), f"{what}: routes are not grouped by expert"
    gu_row_bytes = gate.size // (E * F)
    ref_gate = np.zeros((routes, F), dtype=np.float32)
    ref_up = np.zeros((routes, F), dtype=np.float32)
    for e in np.unique(expert_of_pos):
        sel = np.nonzero(expert_of_pos == e)[0]
        x = hidden[st["sorted_tokens"][sel]]
        sl = slice(e * F * gu_row_bytes, (e + 1) * F * gu_row_bytes)
        ref_gate[sel] = oracle.matmul(kind, gate.reshape(-1)[sl], x, F, threads=16)
        ref_up[sel] = oracle.matmul(kind, up.reshape(-1)[sl], x, F, threads=16)
    m_gate = assert_matmul_parity(st["gate_out"], ref_gate, tol, what=f"{what}: gate projection")
    m_up = assert_matmul_parity(st["up_out"], ref_up, tol, what=f"{what}: up projection")

    lay = hip.packed_activation_layout(kind, routes, F)
    assert lay.act_kind == KIND_Q8_K and lay.total_bytes == st["fused_packed"].size
    ref_fused = oracle.moe_glu(ref_gate, ref_up)
    ref_blocks = np.stack([oracle.pack(KIND_Q8_K, row) for row in ref_fused])
    ref_image = packed_image_from_q8k_blocks(lay, ref_blocks)
    q, d, sums = split_packed_image(lay, routes, st["fused_packed"])
    rq, rd, rsums = split_packed_image(lay, routes, ref_image)
    step = np.abs(q.astype(np.int32) - rq.astype(np.int32))
    assert step.max() <= 1, f"{what}: a re-quantized int8 value differs from the oracle's by {step.max()} steps"
    flips = int(np.count_nonzero(step))
    d_rel = float(np.max(np.abs(d.astype(np.float64) - rd) / np.maximum(np.abs(rd), 1e-30)))
    # the block scale is max / -128 of fp32 products whose silu comes from different exp routines: a few ulps
    assert d_rel <= 2.0 ** -20, f"{what}: Q8_K block scale differs by {d_rel:.3e}"
    assert np.abs(sums.astype(np.int32) - rsums.astype(np.int32)).max() <= 16
    # the sums must belong to the values that were stored
    assert np.array_equal(q.astype(np.int32).reshape(routes, -1, 16).sum(axis=2).astype(np.int16), sums)

    fed = hip.moe_experts_probe(hidden, gate, up, down, ids, w, F, E, kind, kind, fused_override=ref_image)
    m_down = assert_matmul_parity(fed["out"], ref, tol, what=f"{what}: down projection + combine on the oracle's "
                                                              f"re-quantized activations")
    return {"gate": m_gate, "up": m_up, "int8_flips": flips, "int8_total": int(q.size), "scale_rel": d_rel,
            "down_combine": m_down}


def test_moe_stages_small(hip, oracle):
    """The stage-wise comparison on a small layer, grouped and decode-order routing."""
    E, F, H, k = 6, 512, 512, 3
    kind = KIND_Q4_K
    gate, up, down = make_experts(oracle, 430, E, F, H, kind, kind)
    for T in (2, 33):
        hidden = gaussian(431 + T, (T, H))
        vals, ids = oracle.topk(gaussian(432 + T, (T, E)), k)
        w = oracle.softmax_rows(vals)
        ref = oracle.moe_experts(hidden, gate, up, down, ids, w, F, E, kind, kind, threads=8)
        m = check_moe_stages(hip, oracle, hidden, gate, up, down, ids, w, F, E, kind, ref, f"stages T={T}")
        print(f"stages T={T}:", m, flush=True)


def test_config5_qwen3_moe_layer(hip, oracle):
    """128 experts, top-8, hidden 2048, expert FFN 768, Q4_K, 64 tokens; router = top-8 of N(0,1) logits + softmax."""
    E, F, H, k, T = 128, 768, 2048, 8, 64
    kind = KIND_Q4_K
    print("C5: quantizing 3 x 128 expert matrices", flush=True)
    gate = quantize_weights(oracle, kind, gaussian(50, (E * F, H), 0.02))
    up = quantize_weights(oracle, kind, gaussian(51, (E * F, H), 0.02))
    down = quantize_weights(oracle, kind, gaussian(52, (E * H, F), 0.02))
    hidden = gaussian(53, (T, H))
    logits = gaussian(54, (T, E))
    vals, ids = hip.topk(logits, k)
    ov, oi = oracle.topk(logits, k)
    assert np.array_equal(ids, oi)
    w = hip.softmax_rows(vals)
    print("C5: oracle", flush=True)
    ref = oracle.moe_experts(hidden, gate, up, down, oi, oracle.softmax_rows(ov), F, E, kind, kind, threads=16)
    print("C5: hip", flush=True)
    got = hip.moe_experts(hidden, gate, up, down, ids, w, F, E, kind, kind)
    m = assert_moe_parity(got, ref, what="C5 MoE layer")
    print("C5 metrics:", m, "active experts:", len(np.unique(ids)), flush=True)
    print("C5: stage-wise", flush=True)
    stages = check_moe_stages(hip, oracle, hidden, gate, up, down, ids, w, F, E, kind, ref, "C5")
    print("C5 stages:", stages, flush=True)
    # End to end at the matmul bound as well. (An int8 value that flipped by one step would move one of the F terms
    # of an output by 1/127 of its scale; this layer has none, so the per-output bound holds for the whole layer.)
    assert m[0] <= 1e-3, f"C5 end to end: floored max relative error {m[0]:.3e} > 1e-3 with " \
                         f"{stages['int8_flips']} of {stages['int8_total']} re-quantized values one step apart"
    print(f"C5 end to end: floored max relative error {m[0]:.3e}, sum-relative {m[1]:.3e}, max-norm {m[2]:.3e}; "
          f"{stages['int8_flips']} of {stages['int8_total']} re-quantized values differ by one step", flush=True)
    # dequantized expert weights bit-exact (one expert of each matrix is enough: same kernel as the dense check)
    for blocks, rows, kk in ((gate, F, H), (down, H, F)):
        sl = blocks[:rows]
        assert np.array_equal(hip.dequantize(kind, sl, kk).view(np.uint32), oracle.dequantize(kind, sl, kk).view(np.uint32))
