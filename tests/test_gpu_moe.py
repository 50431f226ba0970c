"""GPU parity, part 3: top-k, router softmax and the grouped MoE expert FFN against the CPU oracle."""
import numpy as np
import pytest

from oracle.pyoracle import KIND_Q2_K, KIND_Q3_K, KIND_Q4_1, KIND_Q4_K, KIND_Q5_0, KIND_Q5_1, KIND_Q5_K, KIND_Q6_K, KIND_Q8_0
from tests.test_oracle_moe import make_experts
from tests.util import assert_moe_parity, gaussian, parity_metrics, quantize_weights

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
    # dequantized expert weights bit-exact (one expert of each matrix is enough: same kernel as the dense check)
    for blocks, rows, kk in ((gate, F, H), (down, H, F)):
        sl = blocks[:rows]
        assert np.array_equal(hip.dequantize(kind, sl, kk).view(np.uint32), oracle.dequantize(kind, sl, kk).view(np.uint32))
