"""CPU: the oracle's restatement of marmot_paged_attention (src/backends/cpu/ops/paged_attention/paged_attention_ref.c),
pinned by (1) the closed-form case of the reference's own test (tests/backend/test_backend_paged_attention.c:162-288:
two tokens, identity keys and values, expected softmax weights and cache contents), (2) dense softmax attention in
float64 over each token's history read back through the block table -- what paged attention reduces to -- on caches
with history, shuffled physical blocks, grouped query heads, prompt chunks and decode tokens in one call, and (3) the
cache write as pure data movement (same storage type: the same bits; otherwise one conversion through float32)."""
import numpy as np
import pytest

from tests.attention_cases import NO_BLOCK, TOLERANCE, cache_after_write, dense_reference, make_case, to_f32

MO_INVALID, MO_DTYPE, MO_DIMS = -1, -6, -7


def run(oracle, case, **kw):
    kv_k, kv_v = case["kv_k"].copy(), case["kv_v"].copy()
    st, out = oracle.paged_attention(case["token_meta"], case["q"], case["k_new"], case["v_new"], kv_k, kv_v,
                                     case["block_table"], case["layer_idx"], case["scale"],
                                     act_bf16=case["act"] == "bf16", kv_bf16=case["kv"] == "bf16", **kw)
    return st, out, kv_k, kv_v


def test_reference_closed_form_case(oracle):
    """Two tokens of one sequence, one head of two values, block size 4, scale 1: q = k = v = identity rows."""
    eye = np.array([[[1.0, 0.0]], [[0.0, 1.0]]], dtype=np.float32)
    meta = np.array([[0, 0, 0, 2], [0, 1, 1, 1]], dtype=np.uint32)
    kv_k = np.zeros((1, 1, 1, 4, 2), np.float32)
    kv_v = np.zeros_like(kv_k)
    table = np.zeros((1, 1), np.uint32)
    st, out = oracle.paged_attention(meta, eye, eye.copy(), eye.copy(), kv_k, kv_v, table, 0, 1.0)
    assert st == 0
    e = np.exp(np.float32(1.0))
    assert abs(out[0, 0, 0] - 1.0) < 1e-4 and abs(out[0, 0, 1]) < 1e-4
    assert abs(out[1, 0, 0] - 1.0 / (1.0 + e)) < 1e-4 and abs(out[1, 0, 1] - e / (1.0 + e)) < 1e-4
    for cache in (kv_k, kv_v):
        assert np.array_equal(cache[0, 0, 0, :2], np.eye(2, dtype=np.float32)) and not cache[0, 0, 0, 2:].any()


@pytest.mark.parametrize("act,kv", [("f32", "f32"), ("f16", "f16"), ("f32", "f16"), ("f16", "f32"), ("bf16", "bf16"),
                                    ("f32", "bf16"), ("bf16", "f16")])
def test_matches_dense_attention_in_float64(oracle, act, kv):
    case = make_case(11, [(37, 1), (0, 19), (130, 5), (64, 1)], num_q_heads=8, num_kv_heads=2, head_dim=64, block_size=16,
                     act=act, kv=kv)
    st, out, kv_k, kv_v = run(oracle, case)
    assert st == 0
    want_k, want_v = cache_after_write(case)
    assert np.array_equal(kv_k.view(np.uint8), want_k.view(np.uint8))
    assert np.array_equal(kv_v.view(np.uint8), want_v.view(np.uint8))
    ref = dense_reference(case, want_k, want_v)
    err = np.max(np.abs(to_f32(out, act).astype(np.float64) - ref))
    assert err <= TOLERANCE[act] * np.abs(to_f32(want_v, kv)).max(), err


def test_long_history_spans_several_score_blocks(oracle):
    """head_dim 128: the reference scores 64 positions per block; 700 positions are eleven blocks with a running
    maximum that changes (keys scaled up so that late positions dominate)."""
    case = make_case(12, [(699, 1), (300, 2)], num_q_heads=4, num_kv_heads=4, head_dim=128, block_size=32)
    case["kv_k"][...] *= np.linspace(0.2, 3.0, case["kv_k"].shape[0], dtype=np.float32)[:, None, None, None, None]
    st, out, kv_k, kv_v = run(oracle, case)
    assert st == 0
    ref = dense_reference(case, kv_k, kv_v)
    assert np.max(np.abs(out - ref)) <= TOLERANCE["f32"] * np.abs(kv_v).max()


def test_missing_blocks_strided_views_and_token_count(oracle):
    case = make_case(13, [(40, 3), (5, 1)], num_q_heads=4, num_kv_heads=2, head_dim=32, block_size=8)
    seq = case["token_meta"][0, 0]
    case["block_table"][seq, 1] = NO_BLOCK  # a hole: positions 8..15 of that sequence are skipped
    st, out, kv_k, kv_v = run(oracle, case)
    assert st == 0
    ref = dense_reference(case, kv_k, kv_v)
    assert np.max(np.abs(out - ref)) <= TOLERANCE["f32"] * np.abs(kv_v).max()
    # a sequence whose table row is empty attends over nothing: zeros
    empty = dict(case, block_table=np.full_like(case["block_table"], NO_BLOCK))
    st, out0, _, _ = run(oracle, empty)
    assert st == 0 and not out0.any()
    # q / k_new / v_new as strided views (a fused projection's output), and fewer tokens than rows
    T = case["q"].shape[0]
    fused = np.zeros((T, 4 + 2 + 2, 32), np.float32)
    fused[:, :4], fused[:, 4:6], fused[:, 6:] = case["q"], case["k_new"], case["v_new"]
    view = dict(case, q=fused[:, :4], k_new=fused[:, 4:6], v_new=fused[:, 6:])
    st, out_v, kv_k2, kv_v2 = run(oracle, view)
    assert st == 0 and np.array_equal(out_v, out) and np.array_equal(kv_k2, kv_k)
    st, out_p, _, _ = run(oracle, case, token_count=2)
    assert st == 0 and not out_p[2:].any() and out_p[:2].any()


def test_argument_errors(oracle):
    case = make_case(14, [(3, 2)], num_q_heads=2, num_kv_heads=2, head_dim=8, block_size=4)
    assert run(oracle, dict(case, layer_idx=2))[0] == MO_DIMS
    bad = dict(case, token_meta=case["token_meta"].copy())
    bad["token_meta"][0, 0] = case["block_table"].shape[0]
    assert run(oracle, bad)[0] == MO_DIMS  # seq_slot out of range (paged_attention_ref.c:815-818)
    bad["token_meta"][0, 0] = 0
    bad["token_meta"][0, 2] = case["kv_k"].shape[0] * 4
    assert run(oracle, bad)[0] == MO_DIMS  # kv_slot block out of range (:819-822)
    odd = dict(case, kv_k=np.zeros((4, 2, 2, 6, 8), np.float32), kv_v=np.zeros((4, 2, 2, 6, 8), np.float32))
    assert run(oracle, odd)[0] == MO_INVALID  # block size not a power of two (:586-589)
    three = dict(case, q=np.zeros((2, 3, 8), np.float32))
    assert run(oracle, three)[0] == MO_INVALID  # 3 query heads over 2 kv heads (:590-595)
    assert run(oracle, case, token_count=0)[0] == 0


# ---------------------------------------------------------------- the FLOAT8_E4M3 cache
def test_fp8_e4m3_conversions(oracle):
    """The reference's e4m3 (src/utils/dtype_ref.c:118-212) against the format's definition: every code decodes to the
    value its fields say; encoding is the nearest code by table search with ties to the even mantissa, saturation at
    240 and the reference's clamp below the smallest normal; encode(decode(code)) is the code."""
    from tests.attention_cases import fp8_encode, fp8_values

    vals = fp8_values()
    dec = np.array([oracle.L.mo_fp8_e4m3_to_f32(c) for c in range(256)], dtype=np.float64)
    assert np.array_equal(np.isnan(dec), np.isnan(vals)) and np.array_equal(dec[~np.isnan(dec)], vals[~np.isnan(vals)])
    finite = [c for c in range(256) if not np.isnan(vals[c])]
    # encode(decode(code)) == code, except that -0.0 encodes as +0 (the sign is taken from `value < 0`)
    assert all(oracle.L.mo_f32_to_fp8_e4m3(float(vals[c])) == (0 if c == 0x80 else c) for c in finite)
    rng = np.random.default_rng(0)
    x = np.concatenate([rng.standard_normal(4000).astype(np.float32) * np.float32(s) for s in (0.001, 0.02, 1, 30, 300)])
    mids = ((vals[:0x77] + vals[1:0x78]) / 2).astype(np.float32)  # exact midpoints: ties
    x = np.concatenate([x, mids, -mids, np.array([0.0, -0.0, 240, 241, 1e9, -1e9, 2.0 ** -6, 2.0 ** -10], np.float32)])
    enc = np.array([oracle.L.mo_f32_to_fp8_e4m3(float(v)) for v in x], dtype=np.uint8)
    assert np.array_equal(enc, fp8_encode(x))
    assert oracle.L.mo_f32_to_fp8_e4m3(float("nan")) == 0x79 and oracle.L.mo_f32_to_fp8_e4m3(float("inf")) == 0x77


def _fp8_case(seed, seqs, **kw):
    """An empty fp8 cache (codes 0, scales 0) and a call that fills it."""
    case = make_case(seed, seqs, act="f32", kv="f32", **kw)
    shape = case["kv_k"].shape
    case["kv_k"], case["kv_v"] = np.zeros(shape, np.uint8), np.zeros(shape, np.uint8)
    case["k_scale"], case["v_scale"] = np.zeros(shape[:3], np.float32), np.zeros(shape[:3], np.float32)
    case["kv"] = "fp8"
    return case


def run_fp8(oracle, case):
    kv_k, kv_v, ks, vs = (case[n].copy() for n in ("kv_k", "kv_v", "k_scale", "v_scale"))
    st, out = oracle.paged_attention(case["token_meta"], case["q"], case["k_new"], case["v_new"], kv_k, kv_v,
                                     case["block_table"], case["layer_idx"], case["scale"], kv_k_scale=ks, kv_v_scale=vs)
    return st, out, kv_k, kv_v, ks, vs


def fp8_dense(case, kv_k, kv_v, ks, vs):
    """Dense float64 attention over the decoded cache (code value x block scale)."""
    from tests.attention_cases import fp8_values

    vals = fp8_values().astype(np.float32)
    dk = vals[kv_k] * ks[:, :, :, None, None]
    dv = vals[kv_v] * vs[:, :, :, None, None]
    return dense_reference(dict(case, kv="f32"), dk.astype(np.float32), dv.astype(np.float32)), dv


def test_fp8_cache_prefill_then_decode_with_growing_scales(oracle):
    """Call 1 fills blocks from empty (scales 0 -> max / 240); call 2 appends one louder token per sequence into
    partly filled blocks: the scale grows and the rows already there are re-encoded; a quieter token leaves scale and
    bytes alone. Cache bytes and scales against the independent numpy statement, attention against dense float64
    attention over the decoded cache."""
    from tests.attention_cases import fp8_cache_update

    case = _fp8_case(31, [(0, 21), (0, 9), (0, 40)], num_q_heads=4, num_kv_heads=2, head_dim=32, block_size=16, layers=2,
                     layer_idx=1)
    st, out, kv_k, kv_v, ks, vs = run_fp8(oracle, case)
    assert st == 0
    want_k, want_ks = fp8_cache_update(case, (case["kv_k"], case["k_new"]), case["k_scale"])
    want_v, want_vs = fp8_cache_update(case, (case["kv_v"], case["v_new"]), case["v_scale"])
    assert np.array_equal(kv_k, want_k) and np.array_equal(ks, want_ks)
    assert np.array_equal(kv_v, want_v) and np.array_equal(vs, want_vs)
    ref, dv = fp8_dense(case, kv_k, kv_v, ks, vs)
    assert np.max(np.abs(out - ref)) <= TOLERANCE["f32"] * np.abs(dv).max()
    # call 2: one token per sequence at the next position; sequence 0 louder (x4), sequence 1 quieter (x0.25)
    bs = case["block_size"]
    seqs = sorted(set(int(s) for s in case["token_meta"][:, 0]))
    nxt = {s: int(case["token_meta"][case["token_meta"][:, 0] == s, 1].max()) + 1 for s in seqs}
    meta = np.array([[s, nxt[s], int(case["block_table"][s, nxt[s] // bs]) * bs + nxt[s] % bs, 0] for s in seqs], np.uint32)
    rng = np.random.default_rng(32)
    gain = np.array([4.0, 0.25, 1.0], np.float32)[:, None, None]
    step = dict(case, token_meta=meta, q=rng.standard_normal((3, 4, 32), dtype=np.float32),
                k_new=rng.standard_normal((3, 2, 32), dtype=np.float32) * gain,
                v_new=rng.standard_normal((3, 2, 32), dtype=np.float32) * gain,
                kv_k=kv_k, kv_v=kv_v, k_scale=ks, v_scale=vs)
    st, out2, k2, v2, ks2, vs2 = run_fp8(oracle, step)
    assert st == 0
    want_k2, want_ks2 = fp8_cache_update(step, (kv_k, step["k_new"]), ks)
    want_v2, want_vs2 = fp8_cache_update(step, (kv_v, step["v_new"]), vs)
    assert np.array_equal(k2, want_k2) and np.array_equal(ks2, want_ks2)
    assert np.array_equal(v2, want_v2) and np.array_equal(vs2, want_vs2)
    b_loud, b_quiet = int(meta[0, 2]) // bs, int(meta[1, 2]) // bs
    assert (ks2[b_loud, 1] > ks[b_loud, 1]).all() and not np.array_equal(k2[b_loud, 1, :, :nxt[seqs[0]] % bs], kv_k[b_loud, 1, :, :nxt[seqs[0]] % bs])
    assert np.array_equal(ks2[b_quiet, 1], ks[b_quiet, 1])
    ref2, dv2 = fp8_dense(step, k2, v2, ks2, vs2)
    assert np.max(np.abs(out2 - ref2)) <= TOLERANCE["f32"] * np.abs(dv2).max()
    # the scale tensors are required with an fp8 cache (paged_attention_ref.c:695-698)
    st, _ = oracle.paged_attention(case["token_meta"], case["q"], case["k_new"], case["v_new"], case["kv_k"].copy(),
                                   case["kv_v"].copy(), case["block_table"], 1, case["scale"])
    assert st == MO_INVALID


def test_fp8_e4m3_reference_goldens(oracle, ref_goldens):
    """The e4m3 vectors of the reference's own conversion test (tests/backend/test_backend_conversions.c:78-97 over
    g_conv_fp8 and g_conv_fp8_half_bridge, tests/backend/golden_data.h:1859-1893): codes and round trips."""
    src = ref_goldens["g_conv_fp8_src"]
    assert [oracle.L.mo_f32_to_fp8_e4m3(float(v)) for v in src] == ref_goldens["g_conv_fp8_e4m3_bits"].tolist()
    back = np.array([oracle.L.mo_fp8_e4m3_to_f32(int(c)) for c in ref_goldens["g_conv_fp8_e4m3_bits"]], np.float32)
    assert np.array_equal(back, ref_goldens["g_conv_fp8_e4m3_roundtrip"])
    half = ref_goldens["g_conv_fp8_half_bridge_f16_bits"].view(np.float16).astype(np.float32)
    assert np.array_equal(half, ref_goldens["g_conv_fp8_half_bridge_src"])  # the f16 leg is exact for these values
    assert [oracle.L.mo_f32_to_fp8_e4m3(float(v)) for v in half] == ref_goldens["g_conv_fp8_half_bridge_fp8_bits"].tolist()
    back = np.array([oracle.L.mo_fp8_e4m3_to_f32(int(c)) for c in ref_goldens["g_conv_fp8_half_bridge_fp8_bits"]], np.float32)
    assert np.array_equal(back, ref_goldens["g_conv_fp8_half_bridge_roundtrip"])


def test_fp8_cache_update_hand_computed(oracle):
    """The per-block scale and re-encoding rule of the fp8 cache (paged_attention_ref.c:825-989) on cases whose bytes
    follow from the format by hand: first row of a block (scale = max / 240 bit for bit, largest element = 0x77), a
    louder row (scale doubles, the row already there is re-encoded), a row that is not louder (nothing already there
    changes)."""
    from tests.attention_cases import fp8_hand_case_arrays, fp8_hand_cases

    kv_k, kv_v = np.zeros((1, 1, 1, 4, 4), np.uint8), np.zeros((1, 1, 1, 4, 4), np.uint8)
    ks, vs = np.zeros((1, 1, 1), np.float32), np.zeros((1, 1, 1), np.float32)
    for pos, k_row, v_row, k_codes, k_scale, v_codes, v_scale in fp8_hand_cases():
        meta, q, k_new, v_new, table = fp8_hand_case_arrays(pos, k_row, v_row)
        st, _ = oracle.paged_attention(meta, q, k_new, v_new, kv_k, kv_v, table, 0, 0.5, kv_k_scale=ks, kv_v_scale=vs)
        assert st == 0
        assert kv_k[0, 0, 0].tolist() == k_codes, (pos, kv_k[0, 0, 0])
        assert kv_v[0, 0, 0].tolist() == v_codes, (pos, kv_v[0, 0, 0])
        assert ks.view(np.uint32)[0, 0, 0] == np.float32(k_scale).view(np.uint32), (pos, ks)
        assert vs.view(np.uint32)[0, 0, 0] == np.float32(v_scale).view(np.uint32), (pos, vs)


def test_fp8_cache_update_ignores_nan_codes_in_the_block_maximum(oracle):
    """Rows already in a block may hold NaN codes (exponent field 15): the reference's maximum over the block skips
    them (a comparison with NaN is false, paged_attention_ref.c:866-905), so the new scale comes from the finite
    codes and the new rows; a NaN code re-encodes to the NaN code."""
    from tests.attention_cases import fp8_cache_update

    case = _fp8_case(41, [(0, 6)], num_q_heads=2, num_kv_heads=2, head_dim=16, block_size=8, layers=1, layer_idx=0)
    st, _, kv_k, kv_v, ks, vs = run_fp8(oracle, case)
    assert st == 0
    seq = int(case["token_meta"][0, 0])
    b = int(case["block_table"][seq, 0])
    kv_k[b, 0, 0, 2, 3] = 0x7F   # NaN codes among the rows already there
    kv_k[b, 0, 1, 4, 0] = 0xFF
    kv_v[b, 0, 0, 1, 5] = 0x7A
    meta = np.array([[seq, 6, b * 8 + 6, 0]], np.uint32)
    rng = np.random.default_rng(42)
    step = dict(case, token_meta=meta, q=rng.standard_normal((1, 2, 16), dtype=np.float32),
                k_new=rng.standard_normal((1, 2, 16), dtype=np.float32) * np.float32(5.0),
                v_new=rng.standard_normal((1, 2, 16), dtype=np.float32) * np.float32(5.0),
                kv_k=kv_k, kv_v=kv_v, k_scale=ks, v_scale=vs)
    st, _, k2, v2, ks2, vs2 = run_fp8(oracle, step)
    assert st == 0
    want_k, want_ks = fp8_cache_update(step, (kv_k, step["k_new"]), ks)
    want_v, want_vs = fp8_cache_update(step, (kv_v, step["v_new"]), vs)
    assert np.isfinite(ks2).all() and np.isfinite(vs2).all() and (ks2[b, 0] > ks[b, 0]).all()
    assert np.array_equal(ks2, want_ks) and np.array_equal(vs2, want_vs)
    assert np.array_equal(k2, want_k) and np.array_equal(v2, want_v)
    assert k2[b, 0, 0, 2, 3] & 0x7F >= 0x78 and v2[b, 0, 0, 1, 5] & 0x7F >= 0x78  # still NaN codes
