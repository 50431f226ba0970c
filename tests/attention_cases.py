"""Synthetic paged-attention workloads shared by the CPU and GPU tests: a paged KV cache with history, new tokens of
several sequences (prompt chunks and single decode tokens in one call, in any order), and the two independent
statements of the expected result: the cache after the write (pure data movement and dtype conversion) and dense
softmax attention in float64 over each token's history read back through the block table."""
import numpy as np

NO_BLOCK = 0xFFFFFFFF


def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """Round to nearest even on the float32 bits, as the reference's bfloat16 conversion does."""
    b = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    return ((b + 0x7FFF + ((b >> 16) & 1)) >> 16).astype(np.uint16)


def bf16_bits_to_f32(bits: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(bits, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def to_storage(x32: np.ndarray, name: str) -> np.ndarray:
    """float32 values in the storage type `name` ('f32', 'f16', 'bf16': bfloat16 bits in uint16)."""
    if name == "f32":
        return np.ascontiguousarray(x32, dtype=np.float32)
    if name == "f16":
        return x32.astype(np.float16)
    return f32_to_bf16_bits(x32)


def to_f32(a: np.ndarray, name: str) -> np.ndarray:
    return bf16_bits_to_f32(a).reshape(a.shape) if name == "bf16" else a.astype(np.float32)


def make_case(seed, seqs, num_q_heads, num_kv_heads, head_dim, block_size, act="f32", kv="f32", layers=2, layer_idx=1,
              spare_blocks=3, shuffle_tokens=True):
    """seqs: list of (history_len, new_tokens). Physical blocks are a random permutation; sequence slots are a random
    subset of the block table's rows; rows the call does not write hold finite garbage."""
    rng = np.random.default_rng(seed)
    max_seqs = len(seqs) + 2
    need = [-(-(h + n) // block_size) for h, n in seqs]
    max_blocks = max(need) + 1
    blocks = sum(need) + spare_blocks
    phys = rng.permutation(blocks)
    slots = rng.permutation(max_seqs)[:len(seqs)]
    table = np.full((max_seqs, max_blocks), NO_BLOCK, dtype=np.uint32)
    shape = (blocks, layers, num_kv_heads, block_size, head_dim)
    kv_k = to_storage(rng.standard_normal(shape, dtype=np.float32), kv)
    kv_v = to_storage(rng.standard_normal(shape, dtype=np.float32), kv)
    meta = []
    nxt = 0
    for s, (hist, new) in enumerate(seqs):
        for b in range(need[s]):
            table[slots[s], b] = phys[nxt]
            nxt += 1
        for p in range(hist, hist + new):
            meta.append((slots[s], p, int(table[slots[s], p // block_size]) * block_size + p % block_size, 0))
    meta = np.array(meta, dtype=np.uint32).reshape(-1, 4)
    if shuffle_tokens:
        meta = meta[rng.permutation(len(meta))]
    T = len(meta)
    q = to_storage(rng.standard_normal((T, num_q_heads, head_dim), dtype=np.float32), act)
    k_new = to_storage(rng.standard_normal((T, num_kv_heads, head_dim), dtype=np.float32), act)
    v_new = to_storage(rng.standard_normal((T, num_kv_heads, head_dim), dtype=np.float32), act)
    return {"token_meta": np.ascontiguousarray(meta), "q": q, "k_new": k_new, "v_new": v_new, "kv_k": kv_k, "kv_v": kv_v,
            "block_table": table, "layer_idx": layer_idx, "block_size": block_size, "act": act, "kv": kv,
            "scale": float(1.0 / np.sqrt(head_dim))}


def cache_after_write(case):
    """The caches once every token's new rows are stored at its kv_slot: same storage type = the same bits,
    otherwise through float32."""
    act, kv, bs, layer = case["act"], case["kv"], case["block_size"], case["layer_idx"]
    kv_k, kv_v = case["kv_k"].copy(), case["kv_v"].copy()
    for t, (_, _, slot, _) in enumerate(case["token_meta"]):
        b, off = int(slot) // bs, int(slot) % bs
        for dst, src in ((kv_k, case["k_new"]), (kv_v, case["v_new"])):
            dst[b, layer, :, off, :] = src[t] if act == kv else to_storage(to_f32(src[t], act), kv)
    return kv_k, kv_v


def dense_reference(case, kv_k, kv_v) -> np.ndarray:
    """softmax(scale * q . K) V in float64 over positions 0 .. pos of each token's sequence, read from the given
    caches through the block table (positions without a block are skipped)."""
    bs, layer = case["block_size"], case["layer_idx"]
    q = to_f32(case["q"], case["act"]).astype(np.float64)
    k64 = to_f32(kv_k, case["kv"]).astype(np.float64)
    v64 = to_f32(kv_v, case["kv"]).astype(np.float64)
    T, hq, d = q.shape
    group = hq // case["k_new"].shape[1]
    table = case["block_table"]
    out = np.zeros((T, hq, d))
    for t, (seq, pos, _, _) in enumerate(case["token_meta"]):
        rows = [(int(table[seq, p // bs]), p % bs) for p in range(int(pos) + 1)
                if p // bs < table.shape[1] and table[seq, p // bs] != NO_BLOCK]
        if not rows:
            continue
        bi = np.array([r[0] for r in rows])
        oi = np.array([r[1] for r in rows])
        for h in range(hq):
            K = k64[bi, layer, h // group, oi, :]
            V = v64[bi, layer, h // group, oi, :]
            s = (K @ q[t, h]) * case["scale"]
            w = np.exp(s - s.max())
            out[t, h] = (w / w.sum()) @ V
    return out


TOLERANCE = {"f32": 2e-5, "f16": 1.5e-3, "bf16": 1.2e-2}  # of the largest |v|: fp32 accumulation, one output rounding


# ---------------------------------------------------------------- the FLOAT8_E4M3 cache
def fp8_values() -> np.ndarray:
    """The 256 codes of the reference's e4m3 (1-4-3 bits, bias 7, exponent field 15 = NaN, largest finite 240),
    from the format's definition."""
    code = np.arange(256)
    field, mant = (code >> 3) & 15, code & 7
    mag = np.where(field == 0, mant / 8.0 * 2.0 ** -6, (1 + mant / 8.0) * 2.0 ** (field.astype(np.float64) - 7))
    val = np.where(code & 0x80, -mag, mag)
    return np.where(field == 15, np.nan, val)


def fp8_encode(x: np.ndarray) -> np.ndarray:
    """Nearest representable value, ties to the even mantissa, saturating at 240 -- found by searching the table of
    magnitudes (no exponent arithmetic), for float32 input; one quirk of the reference is kept (below)."""
    x = np.asarray(x, dtype=np.float32)
    table = fp8_values()[:0x78]  # non-negative finite codes 0 .. 0x77, ascending
    mag = np.abs(x).astype(np.float64)
    hi = np.clip(np.searchsorted(table, mag, side="left"), 0, 0x77)
    lo = np.clip(hi - 1, 0, 0x77)
    d_lo, d_hi = mag - table[lo], table[hi] - mag
    pick = np.where(d_lo < d_hi, lo, np.where(d_hi < d_lo, hi, np.where(lo % 2 == 0, lo, hi)))
    pick = np.where(mag >= 240.0, 0x77, pick)
    # the reference never rounds a magnitude below the smallest normal 2^-6 up into the normal range: it clamps the
    # subnormal mantissa to 7 (src/utils/dtype_ref.c:166-174)
    pick = np.where(mag < 2.0 ** -6, np.minimum(pick, 7), pick)
    pick = np.where(np.isnan(x), 0x79, pick)  # the reference's NaN code (no sign: `value < 0` is false for NaN)
    return (pick | np.where(x < 0, 0x80, 0)).astype(np.uint8)  # the sign of a negative value; -0.0 encodes as +0


def fp8_cache_update(case, kv, scales):
    """What one call does to an fp8 cache and its scales [blocks, layers, kv heads], for keys or values alike
    (`kv` = (cache, new rows as float32)): per touched block and head, scale = max(largest decoded magnitude among the
    rows below the first offset written, largest new magnitude) / 240 (1 when that is 0); rows already there are
    re-encoded when the scale changes; the new rows are encoded with it."""
    cache, new = kv
    cache, scales = cache.copy(), scales.copy()
    bs, layer = case["block_size"], case["layer_idx"]
    values = fp8_values().astype(np.float32)
    slots = case["token_meta"][:, 2].astype(np.int64)
    for b in np.unique(slots // bs):
        toks = np.nonzero(slots // bs == b)[0]
        existing = int((slots[toks] % bs).min())
        for h in range(cache.shape[2]):
            old = np.float32(scales[b, layer, h])
            big = np.float32(0.0)
            if existing > 0 and old > 0:
                mags = np.abs(values[cache[b, layer, h, :existing]] * old)
                big = np.float32(np.nanmax(mags)) if np.isfinite(mags).any() else np.float32(0.0)  # NaN codes never win
            big = max(big, np.abs(new[toks, h]).max())
            scale = np.float32(big) / np.float32(240.0) if big > 0 else np.float32(1.0)
            if existing > 0 and scale != old:
                dec = values[cache[b, layer, h, :existing]] * old if old > 0 else np.zeros((existing, cache.shape[4]), np.float32)
                cache[b, layer, h, :existing] = fp8_encode(dec.astype(np.float32) / scale)
            scales[b, layer, h] = scale
            for t in toks:
                cache[b, layer, h, slots[t] % bs] = fp8_encode(new[t, h].astype(np.float32) / scale)
    return cache, scales


def fp8_hand_cases():
    """Three consecutive calls on ONE block of four positions, one kv head of four values, whose cache bytes and scales
    follow from the format by hand (no restatement of the update rule is involved): every quotient value / scale lands
    on an e4m3 value with a wide margin to its neighbours, so the last bits of the float32 divisions do not matter.
      call 1, position 0 into the empty block: the block's scale becomes max|row| / 240 bit for bit and the row's
              largest element encodes to +-0x77 (240);
      call 2, position 1 twice as loud: the scale doubles and the row already there is re-encoded with it (its codes
              halve in value), the new row's largest element is +-0x77;
      call 3, position 2 quieter: the scale and every byte already there stay as they are.
    Returns a list of steps: (pos, k row, v row, expected k codes [4 positions x 4], expected k scale, v codes, v scale);
    positions not written yet keep the cache's initial zero bytes."""
    f = np.float32
    steps = []
    # e4m3 codes used: 240 = 0x77, 120 = 0x6f, 80 = 0x6a, 60 = 0x67, 40 = 0x62, 30 = 0x5f, 20 = 0x5a, 160 = 0x72, 0 = 0
    k1, v1 = [1.0, -3.0, 0.5, 0.0], [-2.0, 0.5, 0.25, 2.0]
    sk1, sv1 = f(3.0) / f(240.0), f(2.0) / f(240.0)
    kc1 = [[0x6A, 0xF7, 0x62, 0x00], [0] * 4, [0] * 4, [0] * 4]
    vc1 = [[0xF7, 0x67, 0x5F, 0x77], [0] * 4, [0] * 4, [0] * 4]
    steps.append((0, k1, v1, kc1, sk1, vc1, sv1))
    k2, v2 = [6.0, 0.0, 0.0, -1.5], [0.0, 1.0, -4.0, 0.0]
    sk2, sv2 = f(6.0) / f(240.0), f(4.0) / f(240.0)
    kc2 = [[0x62, 0xEF, 0x5A, 0x00], [0x77, 0x00, 0x00, 0xE7], [0] * 4, [0] * 4]
    vc2 = [[0xEF, 0x5F, 0x57, 0x6F], [0x00, 0x67, 0xF7, 0x00], [0] * 4, [0] * 4]
    steps.append((1, k2, v2, kc2, sk2, vc2, sv2))
    k3, v3 = [3.0, -0.75, 0.0, 0.0], [4.0, 0.0, -2.0, 0.0]  # v3 as loud as the block already is: same scale
    kc3 = [kc2[0], kc2[1], [0x6F, 0xDF, 0x00, 0x00], [0] * 4]
    vc3 = [vc2[0], vc2[1], [0x77, 0x00, 0xEF, 0x00], [0] * 4]
    steps.append((2, k3, v3, kc3, sk2, vc3, sv2))
    return steps


def fp8_hand_case_arrays(pos, k_row, v_row):
    """The arrays of one call of fp8_hand_cases (one sequence in slot 0, block 0, one q head)."""
    meta = np.array([[0, pos, pos, 0]], dtype=np.uint32)
    q = np.array([[[0.5, -0.25, 1.0, 0.125]]], dtype=np.float32)
    k_new = np.array([[k_row]], dtype=np.float32)
    v_new = np.array([[v_row]], dtype=np.float32)
    table = np.array([[0]], dtype=np.uint32)
    return meta, q, k_new, v_new, table
