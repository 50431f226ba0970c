"""CPU: the oracle's restatement of marmot_embedding_gather for block-quantized tables
(src/backends/cpu/ops/embedding/scalar/embedding_scalar.c:241-303, 381-447), pinned by the reference's own golden for
the Q4_0 table (tests/golden/embedding_q4_0_ragged.txt, transcribed to tests/golden/reference_embedding_q4_0.json: the
interleaved nibble order of the embedding path, which differs from the Q4_0 dequantizer's; Q4_1 tables take the same
order with the Q4_1 dequantizer's values) and, for the other kinds, by
the block dequantizers the quantization goldens pin (a gathered row is the dequantized row, bit for bit). The
reference also ships embedding_q5_0.txt / embedding_q5_1.txt, but its own test skips them unconditionally
(tests/backend/test_backend_embedding_golden.c:283-287, 298-302) and its Q5 dequantizers do not reproduce them: they pin
nothing and are not used here."""
import json
import os

import numpy as np
import pytest

from oracle.pyoracle import (KIND_Q8_1, KIND_Q2_K, KIND_Q3_K, KIND_Q4_0, KIND_Q4_1, KIND_Q4_K, KIND_Q5_0, KIND_Q5_1, KIND_Q5_K, KIND_Q6_K, KIND_Q8_0,
                             row_bytes)
from tests.util import bits, gaussian, random_valid_blocks

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_embedding_q4_0.json")


def load_golden():
    with open(GOLDEN) as f:
        g = json.load(f)
    table = np.frombuffer(bytes.fromhex(g["weights_hex"]), dtype=np.uint8)
    ids = np.array(g["ids"], dtype=np.int32)
    return g["vocab"], g["dim"], table, ids, np.array(g["expected"], dtype=np.float32).reshape(len(ids), g["dim"])


def test_reference_q4_0_embedding_golden(oracle):
    vocab, dim, table, ids, expected = load_golden()
    got = oracle.embedding_gather(KIND_Q4_0, table, vocab, dim, ids, bounds_check=True)
    # the reference's tolerance for this kind is 5e-4 (tests/backend/test_backend_embedding_golden.c:226-229)
    assert np.max(np.abs(got - expected)) <= 1e-6
    # and the order is NOT the block dequantizer's: that one disagrees with the golden
    plain = oracle.dequantize(KIND_Q4_0, table.reshape(vocab, -1), dim)[ids]
    assert np.max(np.abs(plain - expected)) > 1.0


def interleave_map(count: int = 32) -> np.ndarray:
    """Position in the dequantizer's order of value i of the embedding path's interleaved order: byte i / 2 holds
    dequantized value i / 2 in its low nibble and value 16 + i / 2 in its high nibble."""
    i = np.arange(count)
    return np.where(i & 1, 16 + (i >> 1), i >> 1)


def test_q4_1_tables_take_the_interleaved_order_of_the_q4_0_golden(oracle):
    """The reference decodes Q4_1 tables in the interleaved nibble order too (embedding_scalar.c:231-240) and holds no
    golden for it. Two facts it does hold pin the restatement: the order is the Q4_0 case's (its golden, checked
    here through the same index map on the golden's table), and the values are the Q4_1 dequantizer's (its goldens) --
    bit for bit, so a dropped minimum, a fused multiply-add or the dequantizer's order all fail."""
    sigma = interleave_map()
    # the index map itself, on the reference's golden for Q4_0
    vocab, dim, table, ids, expected = load_golden()
    nb = (dim + 31) // 32  # the golden's rows end inside a block: dequantize whole blocks, cut after the map
    full0 = oracle.dequantize(KIND_Q4_0, table.reshape(vocab, -1), nb * 32)[ids].reshape(len(ids), nb, 32)
    assert np.max(np.abs(full0[:, :, sigma].reshape(len(ids), -1)[:, :dim] - expected)) <= 1e-6
    # Q4_1: the same map applied to the dequantized rows
    rng = np.random.default_rng(5)
    vocab, dim = 29, 96
    table = random_valid_blocks(rng, KIND_Q4_1, vocab, dim)
    dense = oracle.dequantize(KIND_Q4_1, table, dim).reshape(vocab, dim // 32, 32)
    ids = rng.integers(0, vocab, (2, 7)).astype(np.int32)
    got = oracle.embedding_gather(KIND_Q4_1, table, vocab, dim, ids)
    want = dense[:, :, sigma].reshape(vocab, dim)[ids]
    assert got.shape == (2, 7, dim) and np.array_equal(bits(got), bits(want))
    assert not np.array_equal(bits(got), bits(dense.reshape(vocab, dim)[ids]))  # not the dequantizer's order
    # a ragged last block takes the first `count` values of the interleaved order
    table = random_valid_blocks(rng, KIND_Q4_1, 5, 64)
    dense = oracle.dequantize(KIND_Q4_1, table, 64).reshape(5, 2, 32)[:, :, sigma].reshape(5, 64)
    ragged = oracle.embedding_gather(KIND_Q4_1, table, 5, 50, np.arange(5, dtype=np.int64))
    assert np.array_equal(bits(ragged), bits(dense[:, :50]))
    half = oracle.embedding_gather(KIND_Q4_1, table, 5, 64, np.arange(5, dtype=np.int32), out_dtype=np.float16, scale=0.5)
    assert np.array_equal(half.view(np.uint16), (dense * np.float32(0.5)).astype(np.float16).view(np.uint16))


@pytest.mark.parametrize("kind", [KIND_Q8_0, KIND_Q4_K, KIND_Q5_K, KIND_Q6_K, KIND_Q5_0, KIND_Q5_1, KIND_Q2_K,
                                  KIND_Q3_K, KIND_Q8_1])
def test_gathered_rows_are_dequantized_rows(oracle, kind):
    rng = np.random.default_rng(800 + kind)
    vocab, dim = 37, 768 if kind in (KIND_Q2_K, KIND_Q3_K, KIND_Q4_K, KIND_Q5_K, KIND_Q6_K) else 96
    table = random_valid_blocks(rng, kind, vocab, dim)
    dense = oracle.dequantize(kind, table, dim)
    ids = rng.integers(0, vocab, (3, 5)).astype(np.int64)
    got = oracle.embedding_gather(kind, table, vocab, dim, ids)
    assert got.shape == (3, 5, dim) and np.array_equal(bits(got), bits(dense[ids]))
    # scale and float16 output: decoded * scale, one rounding
    half = oracle.embedding_gather(kind, table, vocab, dim, ids.astype(np.int32), out_dtype=np.float16, scale=0.5)
    want = (dense[ids] * np.float32(0.5)).astype(np.float16)
    assert np.array_equal(half.view(np.uint16), want.view(np.uint16))


def test_padding_and_out_of_range_tokens(oracle):
    kind, vocab, dim = KIND_Q4_K, 8, 256
    table = random_valid_blocks(np.random.default_rng(810), kind, vocab, dim)
    dense = oracle.dequantize(kind, table, dim)
    ids = np.array([3, 5, -1, 8, 0, 5], dtype=np.int32)
    got = oracle.embedding_gather(kind, table, vocab, dim, ids, padding_id=5)
    assert np.array_equal(bits(got[0]), bits(dense[3])) and np.array_equal(bits(got[4]), bits(dense[0]))
    for z in (1, 2, 3, 5):  # padding rows and out-of-range rows are zero
        assert not got[z].any()
    with pytest.raises(IndexError) as e:  # with the bounds check the first offender is reported
        oracle.embedding_gather(kind, table, vocab, dim, ids, padding_id=5, bounds_check=True)
    assert e.value.args[0] == 2
    # a negative padding id disables padding (embedding_scalar.c:411)
    got = oracle.embedding_gather(kind, table, vocab, dim, np.array([5], np.int32), padding_id=-1)
    assert np.array_equal(bits(got[0]), bits(dense[5]))
