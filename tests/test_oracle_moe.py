"""Pins the oracle's top-k and MoE driver: the reference's own tie case, brute force against per-token dense
math on the dequantized experts, and invariants (unrouted tokens, duplicate routes, policy handling)."""
import numpy as np
import pytest

from oracle.pyoracle import KIND_Q4_K, KIND_Q6_K, KIND_Q8_0, KIND_Q8_K
from tests.util import gaussian


def silu(x):
    return x / (1.0 + np.exp(-x))


def dense_moe_reference(oracle, hidden, gate_b, up_b, down_b, ids, w, F, E, kind_gu, kind_dn, weights_scale=1.0,
                        policy=1):
    """Float64 math with the activation quantization the packed path applies (same Q8 blocks as the oracle's packer),
    accumulated per token in an arbitrary order: what the MoE op means, independent of its grouping logic."""
    from oracle.pyoracle import BLOCK_VALUES, row_bytes

    T, H = hidden.shape
    gw = oracle.dequantize(kind_gu, gate_b.reshape(E * F, -1), H).astype(np.float64).reshape(E, F, H)
    uw = oracle.dequantize(kind_gu, up_b.reshape(E * F, -1), H).astype(np.float64).reshape(E, F, H)
    dw = oracle.dequantize(kind_dn, down_b.reshape(E * H, -1), F).astype(np.float64).reshape(E, H, F)

    def q8(x, kind):
        ak = KIND_Q8_K if BLOCK_VALUES[kind] == 256 else KIND_Q8_0
        return oracle.dequantize(ak, oracle.pack(ak, x.astype(np.float32))[None, :], x.size)[0].astype(np.float64)

    out = np.zeros((T, H))
    for t in range(T):
        xq = q8(hidden[t], kind_gu)
        ws = w[t].astype(np.float64)
        norm = weights_scale
        if policy == 2:
            s = float(np.sum(w[t], dtype=np.float32))
            norm = weights_scale / s if s > np.finfo(np.float32).tiny else 0.0
        for s_, e in enumerate(ids[t]):
            g = gw[e] @ xq
            u = uw[e] @ xq
            fused = (silu(g) * u)
            fq = q8(fused, kind_dn)
            out[t] += ws[s_] * norm * (dw[e] @ fq)
    return out


def make_experts(oracle, seed, E, F, H, kind_gu, kind_dn):
    gate = oracle.quantize(kind_gu, gaussian(seed, (E * F, H), 0.05))
    up = oracle.quantize(kind_gu, gaussian(seed + 1, (E * F, H), 0.05))
    down = oracle.quantize(kind_dn, gaussian(seed + 2, (E * H, F), 0.05))
    return gate, up, down


def test_topk_reference_tie_case(oracle):
    # tests/backend/test_backend_moe.c:126-173
    x = np.array([[1, 4, 4, 2, -1], [0, -3, 5, 5, 1]], dtype=np.float32)
    vals, idx = oracle.topk(x, 3)
    assert np.array_equal(vals, np.array([[4, 4, 2], [5, 5, 1]], dtype=np.float32))
    assert np.array_equal(idx, np.array([[1, 2, 3], [2, 3, 4]], dtype=np.int32))


def test_topk_matches_stable_argsort(oracle):
    rng = np.random.default_rng(5)
    x = rng.integers(-4, 5, size=(50, 33)).astype(np.float32)  # many ties
    vals, idx = oracle.topk(x, 7)
    order = np.argsort(-x, axis=1, kind="stable")[:, :7]
    assert np.array_equal(idx, order.astype(np.int32))
    assert np.array_equal(vals, np.take_along_axis(x, order, axis=1))


def test_softmax_rows(oracle):
    x = gaussian(6, (9, 8))
    got = oracle.softmax_rows(x)
    e = np.exp(x.astype(np.float64) - x.max(axis=1, keepdims=True))
    assert np.allclose(got, e / e.sum(axis=1, keepdims=True), rtol=2e-6, atol=0)
    assert np.allclose(got.sum(axis=1), 1.0, atol=1e-6)


@pytest.mark.parametrize("kind_gu,kind_dn", [(KIND_Q4_K, KIND_Q4_K), (KIND_Q4_K, KIND_Q6_K), (KIND_Q8_0, KIND_Q8_0)])
@pytest.mark.parametrize("T", [2, 9])  # decode path (<= 4 tokens) and grouped path
def test_moe_matches_dense_math(oracle, kind_gu, kind_dn, T):
    E, F, H, k = 6, 256, 512, 3
    gate, up, down = make_experts(oracle, 300, E, F, H, kind_gu, kind_dn)
    hidden = gaussian(310 + T, (T, H))
    logits = gaussian(311 + T, (T, E))
    vals, ids = oracle.topk(logits, k)
    w = oracle.softmax_rows(vals)
    got = oracle.moe_experts(hidden, gate, up, down, ids, w, F, E, kind_gu, kind_dn)
    ref = dense_moe_reference(oracle, hidden, gate, up, down, ids, w, F, E, kind_gu, kind_dn)
    assert np.max(np.abs(got - ref)) <= 2e-5 * np.abs(ref).max()


def test_moe_policies_duplicates_and_unrouted(oracle):
    E, F, H, k = 5, 256, 256, 2
    kind = KIND_Q4_K
    gate, up, down = make_experts(oracle, 320, E, F, H, kind, kind)
    T = 7
    hidden = gaussian(321, (T, H))
    ids = np.array([[0, 1], [1, 1], [4, 2], [2, 4], [0, 0], [3, 1], [1, 3]], dtype=np.int32)  # duplicate routes
    w = np.abs(gaussian(322, (T, k))) + 0.1
    for policy, scale in ((0, 1.0), (1, 2.5), (2, 1.0), (2, 0.5)):
        got = oracle.moe_experts(hidden, gate, up, down, ids, w, F, E, kind, kind, weights_scale=scale, policy=policy)
        ref = dense_moe_reference(oracle, hidden, gate, up, down, ids, w, F, E, kind, kind, weights_scale=scale,
                                  policy=policy)
        assert np.max(np.abs(got - ref)) <= 2e-5 * np.abs(ref).max()
    # grouped and decode paths agree up to the order in which a token's routes are added
    small = oracle.moe_experts(hidden[:3], gate, up, down, ids[:3], w[:3], F, E, kind, kind)
    forced = oracle.moe_experts(hidden[:3], gate, up, down, ids[:3], w[:3], F, E, kind, kind, force_grouped=True)
    assert np.max(np.abs(small - forced)) <= 1e-6 * np.abs(small).max()
    # threads change nothing
    a = oracle.moe_experts(np.tile(hidden, (6, 1)), gate, up, down, np.tile(ids, (6, 1)), np.tile(w, (6, 1)), F, E,
                           kind, kind, threads=1)
    b = oracle.moe_experts(np.tile(hidden, (6, 1)), gate, up, down, np.tile(ids, (6, 1)), np.tile(w, (6, 1)), F, E,
                           kind, kind, threads=4)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    # out-of-range expert id is an error (moe_ops.c:915-919)
    bad = ids.copy()
    bad[3, 1] = E
    with pytest.raises(RuntimeError):
        oracle.moe_experts(hidden, gate, up, down, bad, w, F, E, kind, kind)
