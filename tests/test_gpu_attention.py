"""GPU parity: paged attention through the C ABI against the CPU oracle and against dense float64 attention: the cache
write is bit-exact (pure data movement and one dtype conversion), the attention output agrees within fp32 summation
noise (both sides accumulate in fp32, in different orders) plus one rounding of the output type."""
import numpy as np
import pytest

from marmot_amd import capi
from tests.attention_cases import NO_BLOCK, TOLERANCE, cache_after_write, dense_reference, make_case, to_f32

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def hip():
    from marmot_amd import HipBackend

    b = HipBackend(0)
    yield b
    b.close()


def run_hip(hip, case, **kw):
    kv_k, kv_v = case["kv_k"].copy(), case["kv_v"].copy()
    out = hip.paged_attention(case["token_meta"], case["q"], case["k_new"], case["v_new"], kv_k, kv_v,
                              case["block_table"], case["layer_idx"], case["scale"], act_bf16=case["act"] == "bf16",
                              kv_bf16=case["kv"] == "bf16", **kw)
    return out, kv_k, kv_v


def run_oracle(oracle, case, **kw):
    kv_k, kv_v = case["kv_k"].copy(), case["kv_v"].copy()
    st, out = oracle.paged_attention(case["token_meta"], case["q"], case["k_new"], case["v_new"], kv_k, kv_v,
                                     case["block_table"], case["layer_idx"], case["scale"],
                                     act_bf16=case["act"] == "bf16", kv_bf16=case["kv"] == "bf16", **kw)
    assert st == 0
    return out, kv_k, kv_v


def check(hip, oracle, case, what):
    got, kv_k, kv_v = run_hip(hip, case)
    # FLOAT16 caches with rows of 128 values in blocks of 16 positions or more take the kernel whose scores run on the
    # matrix cores (BFLOAT16 caches likewise); everything else the kernel that works on the vector units
    mfma = case["kv"] in ("f16", "bf16") and case["q"].shape[-1] == 128 and case["block_size"] >= 16
    assert hip.last_route() == ("paged_attention_mfma_scores" if mfma else "paged_attention"), what
    ref, ref_k, ref_v = run_oracle(oracle, case)
    assert np.array_equal(kv_k.view(np.uint8), ref_k.view(np.uint8)), f"{what}: key cache"
    assert np.array_equal(kv_v.view(np.uint8), ref_v.view(np.uint8)), f"{what}: value cache"
    act, kv = case["act"], case["kv"]
    vmax = np.nanmax(np.abs(to_f32(ref_v, kv)))  # (rows that no token reads may hold NaN)
    g32, r32 = to_f32(got, act).astype(np.float64), to_f32(ref, act).astype(np.float64)
    assert np.max(np.abs(g32 - r32)) <= TOLERANCE[act] * vmax, f"{what}: against the oracle"
    dense = dense_reference(case, ref_k, ref_v)
    assert np.max(np.abs(g32 - dense)) <= TOLERANCE[act] * vmax, f"{what}: against dense float64 attention"


def test_reference_closed_form_case(hip):
    """tests/backend/test_backend_paged_attention.c:162-288"""
    eye = np.array([[[1.0, 0.0]], [[0.0, 1.0]]], dtype=np.float32)
    meta = np.array([[0, 0, 0, 2], [0, 1, 1, 1]], dtype=np.uint32)
    kv_k = np.zeros((1, 1, 1, 4, 2), np.float32)
    kv_v = np.zeros_like(kv_k)
    out = hip.paged_attention(meta, eye, eye.copy(), eye.copy(), kv_k, kv_v, np.zeros((1, 1), np.uint32), 0, 1.0)
    e = np.exp(np.float32(1.0))
    assert abs(out[0, 0, 0] - 1.0) < 1e-4 and abs(out[0, 0, 1]) < 1e-4
    assert abs(out[1, 0, 0] - 1.0 / (1.0 + e)) < 1e-4 and abs(out[1, 0, 1] - e / (1.0 + e)) < 1e-4
    for cache in (kv_k, kv_v):
        assert np.array_equal(cache[0, 0, 0, :2], np.eye(2, dtype=np.float32)) and not cache[0, 0, 0, 2:].any()


@pytest.mark.parametrize("act,kv", [("f32", "f32"), ("f16", "f16"), ("f32", "f16"), ("f16", "f32"), ("bf16", "bf16"),
                                    ("f32", "bf16"), ("bf16", "f16")])
@pytest.mark.parametrize("head_dim", [64, 128, 256])
def test_dtypes_and_head_dims(hip, oracle, act, kv, head_dim):
    case = make_case(21 + head_dim, [(37, 1), (0, 19), (130, 5), (64, 1)], num_q_heads=8, num_kv_heads=2,
                     head_dim=head_dim, block_size=16, act=act, kv=kv)
    check(hip, oracle, case, f"{act}/{kv} head_dim={head_dim}")


@pytest.mark.parametrize("head_dim,block_size,hq,hkv", [(2, 4, 1, 1), (40, 8, 6, 3), (80, 1, 4, 4), (96, 32, 2, 1),
                                                        (200, 64, 3, 1), (128, 256, 4, 2)])
def test_ragged_head_dims_and_block_sizes(hip, oracle, head_dim, block_size, hq, hkv):
    """Head dimensions that are not 16 x 4 / 8 / 16 values take the element-wise loads; block sizes from 1 to 256."""
    case = make_case(40 + head_dim, [(70, 3), (9, 1), (0, 2)], num_q_heads=hq, num_kv_heads=hkv, head_dim=head_dim,
                     block_size=block_size, act="f32", kv="f16")
    check(hip, oracle, case, f"head_dim={head_dim} block={block_size}")


@pytest.mark.parametrize("kv", ["f16", "bf16"])
@pytest.mark.parametrize("hq,hkv,block_size", [(3, 3, 16), (6, 3, 32), (8, 2, 16), (16, 2, 64), (4, 1, 128)])
def test_matrix_core_scores_path(hip, oracle, hq, hkv, block_size, kv):
    """FLOAT16 caches with rows of 128 values: the scores run on the matrix cores (key rows as the row operand, the query
    split into two FLOAT16 parts). Histories that end on, before and behind a 16-position tile edge; one, two, four and
    eight query heads per key / value head; NaN in every cache row no token may read (rows behind a sequence's end and
    blocks outside the table); a hole in the table; queries of very large and very small magnitude."""
    hists = [0, 14, 15, 16, 31, 32, 33, 255, 256, 257, 700]
    case = make_case(900 + hq + block_size, [(h, 1) for h in hists] + [(40, 5)], num_q_heads=hq, num_kv_heads=hkv,
                     head_dim=128, block_size=block_size, act="f32", kv=kv)
    # rows that no token attends to: behind the last position of every sequence, and every unreferenced block
    bs, table = block_size, case["block_table"]
    nan = np.nan if kv == "f16" else np.uint16(0x7fc0)  # BFLOAT16 rows travel as bit patterns
    last = {}
    for seq, pos, _, _ in case["token_meta"]:
        last[int(seq)] = max(last.get(int(seq), -1), int(pos))
    used = np.zeros(case["kv_k"].shape[0], bool)
    for seq, end in last.items():
        for b in range(table.shape[1]):
            tb = int(table[seq, b])
            if tb == int(NO_BLOCK):
                continue
            used[tb] = True
            lo = max(0, end + 1 - b * bs)
            if lo < bs:
                case["kv_k"][tb, :, :, lo:, :] = nan
                case["kv_v"][tb, :, :, lo:, :] = nan
    case["kv_k"][~used] = nan
    case["kv_v"][~used] = nan
    check(hip, oracle, case, f"matrix-core scores {hq}/{hkv} block {block_size}")
    # a hole in the middle of the longest history
    longest = max(last, key=last.get)
    holed = dict(case, block_table=table.copy())
    holed["block_table"][longest, 1] = NO_BLOCK
    check(hip, oracle, holed, "matrix-core scores, hole")
    # magnitudes: scores of +-60 (one position takes all the weight) and of 1e-6 (uniform weights)
    for factor in (40.0, 1e-4):
        scaled = dict(case, q=(case["q"] * np.float32(factor)).astype(np.float32))
        check(hip, oracle, scaled, f"matrix-core scores, query x {factor}")


def test_long_context_decode_batch(hip, oracle):
    """16 sequences with 1000 to 3000 positions of history, one token each, grouped query heads, fp16 cache."""
    rng = np.random.default_rng(50)
    seqs = [(int(h), 1) for h in rng.integers(1000, 3000, 16)]
    case = make_case(51, seqs, num_q_heads=8, num_kv_heads=2, head_dim=128, block_size=16, act="f32", kv="f16",
                     layers=1, layer_idx=0)
    check(hip, oracle, case, "decode batch")


def test_prompt_of_many_tokens_takes_unsplit_histories(hip, oracle):
    """A prompt chunk of 640 tokens on top of 100 positions of history, next to a short second sequence: enough
    (token, heads) pairs that no history is split across workgroups (decode-sized calls above split it)."""
    case = make_case(60, [(100, 640), (3, 8)], num_q_heads=4, num_kv_heads=2, head_dim=64, block_size=32, act="f16",
                     kv="f16", layers=1, layer_idx=0)
    check(hip, oracle, case, "prompt chunk")


def test_holes_strided_views_token_count_and_errors(hip, oracle):
    case = make_case(13, [(40, 3), (5, 1)], num_q_heads=4, num_kv_heads=2, head_dim=32, block_size=8)
    seq = case["token_meta"][0, 0]
    case["block_table"][seq, 1] = NO_BLOCK
    check(hip, oracle, case, "hole in the block table")
    empty = dict(case, block_table=np.full_like(case["block_table"], NO_BLOCK))
    out0, _, _ = run_hip(hip, empty)
    assert not out0.any()
    # q / k_new / v_new as views of one buffer (what a fused projection leaves), fewer tokens than rows
    T = case["q"].shape[0]
    fused = np.zeros((T, 8, 32), np.float32)
    fused[:, :4], fused[:, 4:6], fused[:, 6:] = case["q"], case["k_new"], case["v_new"]
    view = dict(case, q=fused[:, :4], k_new=fused[:, 4:6], v_new=fused[:, 6:])
    plain, kv_k, _ = run_hip(hip, case)
    out_v, kv_k2, _ = run_hip(hip, view)
    assert np.array_equal(out_v, plain) and np.array_equal(kv_k2, kv_k)
    out_p, kv_p, _ = run_hip(hip, case, token_count=2)  # only the first two tokens are stored and served
    ref_p, ref_kp, _ = run_oracle(oracle, case, token_count=2)
    assert not out_p[2:].any() and np.array_equal(kv_p, ref_kp)
    assert np.max(np.abs(out_p - ref_p)) <= TOLERANCE["f32"] * np.abs(case["kv_v"]).max()
    # errors, in the reference's order and with its codes
    def code(c, **kw):
        with pytest.raises(capi.MarmotHipError) as e:
            run_hip(hip, c, **kw)
        return e.value.code
    assert code(dict(case, layer_idx=2)) == -7
    bad = dict(case, token_meta=case["token_meta"].copy())
    bad["token_meta"][1, 0] = case["block_table"].shape[0]
    assert code(bad) == -7
    bad["token_meta"][1, 0] = 0
    bad["token_meta"][1, 2] = case["kv_k"].shape[0] * 8
    assert code(bad) == -7
    # without the check such a token is skipped: nothing outside the buffers is touched, the other tokens are served
    out_s, _, _ = run_hip(hip, bad, validate=False)
    keep = [t for t in range(T) if t != 1]
    assert np.isfinite(out_s).all() and out_s[keep].any()
    odd = dict(case, kv_k=np.zeros((4, 2, 2, 6, 32), np.float32), kv_v=np.zeros((4, 2, 2, 6, 32), np.float32))
    assert code(odd) == -1
    assert code(dict(case, q=np.zeros((T, 3, 32), np.float32))) == -1
    big = make_case(14, [(3, 1)], num_q_heads=1, num_kv_heads=1, head_dim=320, block_size=4)
    assert code(big) == -8  # head dimensions beyond 256 are left to the caller's fallback


# ---------------------------------------------------------------- the FLOAT8_E4M3 cache
def _fp8_case(seed, seqs, act="f32", room=0, **kw):
    """An empty fp8 cache (codes 0, scales 0) and a call that fills it; `room` more positions per sequence have blocks
    in the table for later decode steps."""
    case = make_case(seed, [(h, n + room) for h, n in seqs], act=act, kv="f32", **kw)
    meta = case["token_meta"]
    last = {int(s): int(meta[meta[:, 0] == s, 1].max()) for s in set(meta[:, 0])}
    keep = np.array([int(pos) <= last[int(s)] - room for s, pos, _, _ in meta])
    case["token_meta"] = np.ascontiguousarray(meta[keep])
    for n in ("q", "k_new", "v_new"):
        case[n] = np.ascontiguousarray(case[n][keep])
    shape = case["kv_k"].shape
    case["kv_k"], case["kv_v"] = np.zeros(shape, np.uint8), np.zeros(shape, np.uint8)
    case["k_scale"], case["v_scale"] = np.zeros(shape[:3], np.float32), np.zeros(shape[:3], np.float32)
    return case


def _fp8_both(hip, oracle, case, what):
    """One call on both sides from the same cache state: cache bytes and scales bit-exact (the write path is integer
    and exactly rounded float work: maxima, one division, the e4m3 encoder), attention within fp32 summation noise of
    the oracle and of dense float64 attention over the decoded cache. Returns the state after the call."""
    from tests.attention_cases import fp8_values

    state = {n: case[n].copy() for n in ("kv_k", "kv_v", "k_scale", "v_scale")}
    got = hip.paged_attention(case["token_meta"], case["q"], case["k_new"], case["v_new"], state["kv_k"], state["kv_v"],
                              case["block_table"], case["layer_idx"], case["scale"], act_bf16=case["act"] == "bf16",
                              kv_k_scale=state["k_scale"], kv_v_scale=state["v_scale"])
    # rows of 128 codes in blocks of 16 positions or more: scores on the matrix cores (codes widened to FLOAT16 in
    # registers), everything else on the vector units
    mfma = case["q"].shape[-1] == 128 and case["block_size"] >= 16
    assert hip.last_route() == ("paged_attention_mfma_scores" if mfma else "paged_attention"), what
    ref_state = {n: case[n].copy() for n in ("kv_k", "kv_v", "k_scale", "v_scale")}
    st, ref = oracle.paged_attention(case["token_meta"], case["q"], case["k_new"], case["v_new"], ref_state["kv_k"],
                                     ref_state["kv_v"], case["block_table"], case["layer_idx"], case["scale"],
                                     act_bf16=case["act"] == "bf16", kv_k_scale=ref_state["k_scale"],
                                     kv_v_scale=ref_state["v_scale"])
    assert st == 0
    for n in ("k_scale", "v_scale", "kv_k", "kv_v"):
        assert np.array_equal(state[n].view(np.uint8), ref_state[n].view(np.uint8)), f"{what}: {n}"
    vals = fp8_values().astype(np.float32)
    dk = (vals[state["kv_k"]] * state["k_scale"][:, :, :, None, None]).astype(np.float32)
    dv = (vals[state["kv_v"]] * state["v_scale"][:, :, :, None, None]).astype(np.float32)
    act = case["act"]
    vmax = np.abs(dv).max()
    g32, r32 = to_f32(got, act).astype(np.float64), to_f32(ref, act).astype(np.float64)
    assert np.max(np.abs(g32 - r32)) <= TOLERANCE[act] * vmax, f"{what}: against the oracle"
    dense = dense_reference(dict(case, kv="f32"), dk, dv)
    assert np.max(np.abs(g32 - dense)) <= TOLERANCE[act] * vmax, f"{what}: against dense float64 attention"
    return state


def _next_step(case, state, seed, gains, act="f32"):
    """One more token per sequence at its next position, new rows scaled per sequence by `gains`."""
    from tests.attention_cases import to_storage

    bs = case["block_size"]
    meta0 = case["token_meta"]
    seqs = sorted(set(int(s) for s in meta0[:, 0]))
    nxt = {s: int(meta0[meta0[:, 0] == s, 1].max()) + 1 for s in seqs}
    meta = np.array([[s, nxt[s], int(case["block_table"][s, nxt[s] // bs]) * bs + nxt[s] % bs, 0] for s in seqs],
                    np.uint32)
    rng = np.random.default_rng(seed)
    hq, hkv, d = case["q"].shape[1], case["k_new"].shape[1], case["q"].shape[2]
    gain = np.asarray(gains, np.float32)[:len(seqs), None, None]
    return dict(case, token_meta=meta, q=to_storage(rng.standard_normal((len(seqs), hq, d), dtype=np.float32), act),
                k_new=to_storage(rng.standard_normal((len(seqs), hkv, d), dtype=np.float32) * gain, act),
                v_new=to_storage(rng.standard_normal((len(seqs), hkv, d), dtype=np.float32) * gain, act),
                kv_k=state["kv_k"], kv_v=state["kv_v"], k_scale=state["k_scale"], v_scale=state["v_scale"])


@pytest.mark.parametrize("act,head_dim,block_size,hq,hkv", [("f32", 32, 16, 4, 2), ("f16", 64, 16, 8, 2),
                                                            ("bf16", 128, 32, 8, 8), ("f32", 256, 16, 2, 1),
                                                            ("f16", 40, 8, 6, 3)])
def test_fp8_cache_prefill_then_decode(hip, oracle, act, head_dim, block_size, hq, hkv):
    """Call 1 fills blocks from empty (scales 0 -> max / 240); then three decode steps append to partly filled
    blocks: a louder token grows the block's scale and re-encodes the rows already there, a quieter one leaves scale
    and bytes alone; a step that opens a new block finds scale 0."""
    case = _fp8_case(300 + head_dim, [(0, 21), (0, 9), (0, 2 * block_size - 1)], act=act, room=3, num_q_heads=hq,
                     num_kv_heads=hkv, head_dim=head_dim, block_size=block_size, layers=2, layer_idx=1)
    state = _fp8_both(hip, oracle, case, "prefill")
    assert (state["k_scale"][:, 0] == 0).all(), "other layers' scales are not touched"
    for i, gains in enumerate(([4.0, 0.25, 1.0], [0.5, 8.0, 2.0], [1.0, 1.0, 16.0])):
        before = state
        case = _next_step(case, state, 400 + i, gains, act)
        state = _fp8_both(hip, oracle, case, f"decode step {i}")
        if i == 0:
            b_loud, b_quiet = (int(case["token_meta"][r, 2]) // block_size for r in (0, 1))
            assert (state["k_scale"][b_loud, 1] > before["k_scale"][b_loud, 1]).all()
            assert np.array_equal(state["k_scale"][b_quiet, 1], before["k_scale"][b_quiet, 1])


def test_fp8_cache_long_context_decode_batch(hip, oracle):
    """A decode batch over long fp8 histories takes the split-history kernels and the 16-byte cache loads."""
    case = _fp8_case(77, [(0, 700), (0, 333), (0, 1025), (0, 64)], room=1, num_q_heads=8, num_kv_heads=2, head_dim=128,
                     block_size=16, layers=1, layer_idx=0)
    state = _fp8_both(hip, oracle, case, "prompts")
    step = _next_step(case, state, 78, [1.0, 3.0, 0.5, 1.0])
    _fp8_both(hip, oracle, step, "decode over long histories")


def test_fp8_cache_decode_over_a_wide_block_table(hip, oracle):
    """Decode steps on an fp8 cache whose block table spans 2048 positions or more take the form of the kernel whose
    tile loop is pipelined (rows of the next tile and the table entry of the one after in flight); sequences with few
    tiles take its plain loop. A history of 2100 positions next to ones of 40 and 500, two decode steps, and a
    sequence whose last tile is partial."""
    case = _fp8_case(87, [(0, 2100), (0, 40), (0, 500)], room=2, num_q_heads=4, num_kv_heads=1, head_dim=128,
                     block_size=16, layers=1, layer_idx=0)
    assert case["block_table"].shape[1] * 16 >= 2048
    state = _fp8_both(hip, oracle, case, "prompts")
    step = _next_step(case, state, 88, [1.0, 2.0, 0.5])
    state = _fp8_both(hip, oracle, step, "decode, wide table")
    step = _next_step(step, state, 89, [4.0, 1.0, 1.0])
    _fp8_both(hip, oracle, step, "second decode step")


def test_fp8_cache_errors(hip):
    case = _fp8_case(5, [(0, 3)], num_q_heads=2, num_kv_heads=1, head_dim=16, block_size=4)
    args = (case["token_meta"], case["q"], case["k_new"], case["v_new"])
    with pytest.raises(capi.MarmotHipError) as e:  # paged_attention_ref.c:695-698
        hip.paged_attention(*args, case["kv_k"].copy(), case["kv_v"].copy(), case["block_table"], 1, case["scale"])
    assert e.value.code == -1 and "requires scale tensors" in str(e.value)
    f32 = make_case(5, [(0, 3)], num_q_heads=2, num_kv_heads=1, head_dim=16, block_size=4)
    with pytest.raises(capi.MarmotHipError) as e:
        hip.paged_attention(*args, f32["kv_k"].copy(), f32["kv_v"].copy(), f32["block_table"], 1, f32["scale"],
                            kv_k_scale=case["k_scale"].copy(), kv_v_scale=case["v_scale"].copy())
    assert e.value.code == -1


@pytest.mark.parametrize("head_dim", [64, 128, 256, 24])
def test_fp8_cache_given_codes(hip, oracle, head_dim):
    """Histories written as raw codes, one kind per sequence: only subnormal codes (magnitudes up to 7 x 2^-9, either
    sign, -0 included), every finite code, and all 256 codes (exponent field 15 decodes to NaN: that sequence checks
    the cache write next to NaN codes, bit for bit; its attention output is NaN on both sides: one NaN score makes a
    head's output NaN in the reference, and the device reports NaN for a head whose sum of weights is NaN).
    Each other sequence's output is judged against its own largest value."""
    from tests.attention_cases import fp8_values

    hist = 40
    case = _fp8_case(500 + head_dim, [(hist, 1)] * 3, room=0, num_q_heads=4, num_kv_heads=2, head_dim=head_dim,
                     block_size=16, layers=1, layer_idx=0)
    rng = np.random.default_rng(head_dim)
    shape = case["kv_k"].shape
    kinds = [lambda n: (rng.integers(0, 8, n) | (rng.integers(0, 2, n) << 7)),
             lambda n: (rng.integers(0, 0x78, n) | (rng.integers(0, 2, n) << 7)),
             lambda n: rng.integers(0, 256, n)]
    order = {int(s): i for i, s in enumerate(case["token_meta"][:, 0])}  # token row of each sequence slot
    for slot, row in order.items():
        blocks = case["block_table"][slot]
        for b in blocks[blocks != NO_BLOCK]:
            for cache in (case["kv_k"], case["kv_v"]):
                cache[b] = kinds[row % 3](shape[1:]).astype(np.uint8)
        if row % 3 == 0:  # quiet new rows beside the subnormal history
            case["k_new"][row] *= 1e-3
            case["v_new"][row] *= 1e-3
    case["k_scale"][...] = 1.0
    case["v_scale"][...] = 1.0
    state = {n: case[n].copy() for n in ("kv_k", "kv_v", "k_scale", "v_scale")}
    got = hip.paged_attention(case["token_meta"], case["q"], case["k_new"], case["v_new"], state["kv_k"], state["kv_v"],
                              case["block_table"], 0, case["scale"], kv_k_scale=state["k_scale"],
                              kv_v_scale=state["v_scale"])
    ref_state = {n: case[n].copy() for n in ("kv_k", "kv_v", "k_scale", "v_scale")}
    st, ref = oracle.paged_attention(case["token_meta"], case["q"], case["k_new"], case["v_new"], ref_state["kv_k"],
                                     ref_state["kv_v"], case["block_table"], 0, case["scale"],
                                     kv_k_scale=ref_state["k_scale"], kv_v_scale=ref_state["v_scale"])
    assert st == 0
    for n in ("k_scale", "v_scale", "kv_k", "kv_v"):
        assert np.array_equal(state[n].view(np.uint8), ref_state[n].view(np.uint8)), n
    vals = fp8_values()
    for slot, row in order.items():
        if row % 3 == 2:
            assert np.isnan(ref[row]).any()
            assert np.isnan(got[row]).all()  # every head of this sequence has NaN codes in its history
            continue
        blocks = case["block_table"][slot]
        blocks = blocks[blocks != NO_BLOCK]
        vmax = np.nanmax(np.abs(vals[state["kv_v"][blocks]] * state["v_scale"][blocks][:, :, :, None, None]))
        assert vmax > 0 and np.max(np.abs(got[row].astype(np.float64) - ref[row])) <= TOLERANCE["f32"] * vmax, row


def test_fp8_cache_update_hand_computed(hip):
    """The hand-computed fp8 cache scenario (tests/attention_cases.py::fp8_hand_cases: first row of a block, a louder
    row, a row that is not louder) through the HIP entry point: bytes and scale bits as computed by hand."""
    from tests.attention_cases import fp8_hand_case_arrays, fp8_hand_cases

    kv_k, kv_v = np.zeros((1, 1, 1, 4, 4), np.uint8), np.zeros((1, 1, 1, 4, 4), np.uint8)
    ks, vs = np.zeros((1, 1, 1), np.float32), np.zeros((1, 1, 1), np.float32)
    for pos, k_row, v_row, k_codes, k_scale, v_codes, v_scale in fp8_hand_cases():
        meta, q, k_new, v_new, table = fp8_hand_case_arrays(pos, k_row, v_row)
        hip.paged_attention(meta, q, k_new, v_new, kv_k, kv_v, table, 0, 0.5, kv_k_scale=ks, kv_v_scale=vs)
        assert kv_k[0, 0, 0].tolist() == k_codes, (pos, kv_k[0, 0, 0])
        assert kv_v[0, 0, 0].tolist() == v_codes, (pos, kv_v[0, 0, 0])
        assert ks.view(np.uint32)[0, 0, 0] == np.float32(k_scale).view(np.uint32), (pos, ks)
        assert vs.view(np.uint32)[0, 0, 0] == np.float32(v_scale).view(np.uint32), (pos, vs)


def test_fp8_cache_duplicate_slot_rescales_the_block_once(hip, oracle):
    """Two tokens of one call carry the same kv_slot (the block's first offset written): the block must be rescaled
    exactly once, like the reference does it; scales and the rows already there against the oracle. The duplicated
    row itself is written twice with the same scale (whichever token's values end up there is not defined)."""
    case = _fp8_case(901, [(0, 5)], room=1, num_q_heads=2, num_kv_heads=2, head_dim=32, block_size=8)
    state = _fp8_both(hip, oracle, case, "prefill")
    bs = case["block_size"]
    seq = int(case["token_meta"][0, 0])
    slot = int(case["block_table"][seq, 0]) * bs + 5
    meta = np.array([[seq, 5, slot, 0], [seq, 5, slot, 0]], np.uint32)
    rng = np.random.default_rng(902)
    row_k = rng.standard_normal((1, 2, 32), dtype=np.float32) * np.float32(8.0)  # louder than the block: it is rescaled
    row_v = rng.standard_normal((1, 2, 32), dtype=np.float32) * np.float32(8.0)
    step = dict(case, token_meta=meta, q=rng.standard_normal((2, 2, 32), dtype=np.float32),
                k_new=np.repeat(row_k, 2, axis=0), v_new=np.repeat(row_v, 2, axis=0), **state)
    _fp8_both(hip, oracle, step, "duplicate slot")


def test_fp8_cache_duplicate_slot_with_different_rows_keeps_the_later_one(hip, oracle):
    """Calls of up to 1024 tokens update the cache in one launch in which one workgroup writes all new rows of a block
    in token order: two tokens with one kv_slot and different rows leave the later token's row, as the reference's
    token loop does, and both rows count for the block's scale."""
    case = _fp8_case(911, [(0, 11)], room=1, num_q_heads=2, num_kv_heads=2, head_dim=32, block_size=8)
    state = _fp8_both(hip, oracle, case, "prefill")
    seq = int(case["token_meta"][0, 0])
    slot = int(case["block_table"][seq, 1]) * 8 + 3
    meta = np.array([[seq, 11, slot, 0]] * 3, np.uint32)
    rng = np.random.default_rng(912)
    gain = np.array([1.0, 9.0, 2.0], np.float32)[:, None, None]  # the loudest row is not the one that stays
    step = dict(case, token_meta=meta, q=rng.standard_normal((3, 2, 32), dtype=np.float32),
                k_new=rng.standard_normal((3, 2, 32), dtype=np.float32) * gain,
                v_new=rng.standard_normal((3, 2, 32), dtype=np.float32) * gain, **state)
    _fp8_both(hip, oracle, step, "duplicate slot, different rows")


def test_fp8_cache_update_in_four_launches(oracle, monkeypatch):
    """Calls of more than 1024 tokens (and every call under MARMOT_HIP_NO_FP8_UPDATE_FUSED, read when a device object
    is created) update the cache in four launches with scratch memory between them: the same bytes and scales."""
    from marmot_amd import HipBackend

    monkeypatch.setenv("MARMOT_HIP_NO_FP8_UPDATE_FUSED", "1")
    plain = HipBackend(0)
    monkeypatch.delenv("MARMOT_HIP_NO_FP8_UPDATE_FUSED")
    case = _fp8_case(921, [(0, 21), (0, 9), (0, 31)], room=3, num_q_heads=4, num_kv_heads=2, head_dim=64,
                     block_size=16)
    state = _fp8_both(plain, oracle, case, "prefill, four launches")
    for i, gains in enumerate([(1.0, 6.0, 0.2), (30.0, 1.0, 1.0), (0.0, 1.0, 50.0)]):
        case = _next_step(case, state, 930 + i, gains)
        state = _fp8_both(plain, oracle, case, f"decode step {i}, four launches")
