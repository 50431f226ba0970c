"""Shared helpers of the test-suite: seeded inputs, threaded oracle quantization, parity metrics."""
from __future__ import annotations

import concurrent.futures as cf
import os

import numpy as np

from oracle.pyoracle import BLOCK_VALUES, KIND_Q8_0, KIND_Q8_K, row_bytes


def bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


def gaussian(seed: int, shape, scale: float = 1.0) -> np.ndarray:
    rng = np.random.Generator(np.random.PCG64(seed))
    x = rng.standard_normal(shape, dtype=np.float32)
    if scale != 1.0:
        x *= np.float32(scale)
    return x


def quantize_weights(oracle, kind: int, w: np.ndarray, workers: int | None = None) -> np.ndarray:
    """Oracle weight quantizer over row chunks in threads (ctypes releases the GIL)."""
    rows = w.shape[0]
    workers = workers or min(16, os.cpu_count() or 1)
    if rows < 4 * workers:
        return oracle.quantize(kind, w)
    bounds = np.linspace(0, rows, workers + 1).astype(int)
    with cf.ThreadPoolExecutor(workers) as ex:
        parts = list(ex.map(lambda i: oracle.quantize(kind, w[bounds[i]:bounds[i + 1]]), range(workers)))
    return np.concatenate(parts, axis=0)


def act_kind_for(kind: int) -> int:
    return KIND_Q8_K if BLOCK_VALUES[kind] == 256 else KIND_Q8_0


def parity_metrics(y: np.ndarray, r: np.ndarray):
    """(max relative error with the denominator floored at 1e-3 * rms(r),  sum|d| / sum|r|,  max|d| / max|r|)."""
    y = np.asarray(y, dtype=np.float64)
    r = np.asarray(r, dtype=np.float64)
    d = np.abs(y - r)
    rms = float(np.sqrt(np.mean(r * r))) if r.size else 0.0
    denom = np.maximum(np.abs(r), 1e-3 * rms + 1e-30)
    return float(np.max(d / denom)) if r.size else 0.0, float(d.sum() / (np.abs(r).sum() + 1e-30)), \
        float(d.max() / (np.abs(r).max() + 1e-30)) if r.size else 0.0


def assert_matmul_parity(y, r, tol=1e-3, what=""):
    m1, m2, m3 = parity_metrics(y, r)
    assert np.all(np.isfinite(np.asarray(y, dtype=np.float64))), f"{what}: non-finite output"
    assert m1 <= tol, f"{what}: max relative error {m1:.3e} > {tol} (sum-rel {m2:.3e}, max-norm {m3:.3e})"
    return m1, m2, m3


def assert_moe_parity(y, r, tol=1e-3, what=""):
    """MoE re-quantizes silu(gate)*up to Q8 before the down projection, so a last-ulp difference upstream (fp32
    summation order, expf) can move one int8 value by one step; that shifts individual outputs by ~1/127 of one of F
    terms. The bound is therefore taken against the output scale: max|d| / max|r| and sum|d| / sum|r| <= 1e-3
    (the reference's own MoE tests allow 3e-2..9e-2 against dense math, tests/backend/test_backend_moe.c:620-1081)."""
    m1, m2, m3 = parity_metrics(y, r)
    assert np.all(np.isfinite(np.asarray(y, dtype=np.float64))), f"{what}: non-finite output"
    assert m3 <= tol and m2 <= tol, f"{what}: max-norm error {m3:.3e}, sum-rel {m2:.3e} (floored-relative {m1:.3e})"
    return m1, m2, m3


def random_valid_blocks(rng, kind: int, rows: int, k: int) -> np.ndarray:
    """Arbitrary block bytes with finite, moderate fp16 scale fields (exercises every nibble / scale pattern)."""
    from oracle.pyoracle import BLOCK_BYTES

    nb = (k + BLOCK_VALUES[kind] - 1) // BLOCK_VALUES[kind]
    bb = BLOCK_BYTES[kind]
    raw = rng.integers(0, 256, size=(rows * nb, bb), dtype=np.uint8)
    offs = {1: [0], 2: [0, 2], 3: [0], 4: [0, 2], 5: [0], 6: [0, 2], 7: [80, 82], 8: [108], 9: [0, 2], 10: [0, 2], 11: [208]}[kind]
    for off in offs:
        h = raw[:, off:off + 2].copy().view(np.uint16)
        h &= 0xBBFF  # clear the top exponent bit: |value| < 2, no inf/nan
        raw[:, off:off + 2] = h.view(np.uint8)
    return raw.reshape(rows, nb * bb)
