"""GPU parity: quantized embedding gather against the CPU oracle, through the C ABI: bit-exact rows for every kind
(Q4_0 and Q4_1 tables in the embedding path's own nibble order: the reference's golden for Q4_0), token id dtypes, padding and
out-of-range tokens, the bounds check, scale and float16 output."""
import numpy as np
import pytest

from marmot_amd import capi
from oracle.pyoracle import KIND_Q8_1, KIND_Q2_K, KIND_Q3_K, KIND_Q4_0, KIND_Q4_1, KIND_Q4_K, KIND_Q5_0, KIND_Q5_1, KIND_Q5_K, KIND_Q6_K, KIND_Q8_0
from tests.test_oracle_embedding import load_golden
from tests.util import bits, random_valid_blocks

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def hip():
    from marmot_amd import HipBackend

    b = HipBackend(0)
    yield b
    b.close()


def test_reference_q4_0_embedding_golden(hip):
    vocab, dim, table, ids, expected = load_golden()
    got = hip.embedding_gather(KIND_Q4_0, table, vocab, dim, ids, bounds_check=True)
    assert np.max(np.abs(got - expected)) <= 1e-6


@pytest.mark.parametrize("kind", [KIND_Q4_0, KIND_Q4_1, KIND_Q5_0, KIND_Q5_1, KIND_Q8_0, KIND_Q8_1, KIND_Q2_K, KIND_Q3_K, KIND_Q4_K, KIND_Q5_K,
                                  KIND_Q6_K])
@pytest.mark.parametrize("ids_dtype", [np.int32, np.int64])
def test_gather_is_bit_exact(hip, oracle, kind, ids_dtype):
    rng = np.random.default_rng(820 + kind)
    vocab = 1000
    dim = 4096 if kind in (KIND_Q2_K, KIND_Q3_K, KIND_Q4_K, KIND_Q5_K, KIND_Q6_K) else 1120  # 1120 = 35 blocks of 32: several workgroups per row
    table = random_valid_blocks(rng, kind, vocab, dim)
    ids = rng.integers(0, vocab, (4, 9)).astype(ids_dtype)
    ids[1, 2], ids[3, 8] = 7, 7
    ref = oracle.embedding_gather(kind, table, vocab, dim, ids, padding_id=7)
    got = hip.embedding_gather(kind, table, vocab, dim, ids, padding_id=7)
    assert got.shape == (4, 9, dim) and np.array_equal(bits(got), bits(ref))
    ref16 = oracle.embedding_gather(kind, table, vocab, dim, ids, out_dtype=np.float16, scale=0.37)
    got16 = hip.embedding_gather(kind, table, vocab, dim, ids, out_dtype=np.float16, scale=0.37)
    assert np.array_equal(got16.view(np.uint16), ref16.view(np.uint16))
    ref_s = oracle.embedding_gather(kind, table, vocab, dim, ids, scale=3.0)
    assert np.array_equal(bits(hip.embedding_gather(kind, table, vocab, dim, ids, scale=3.0)), bits(ref_s))


def test_out_of_range_tokens_and_bounds_check(hip, oracle):
    kind, vocab, dim = KIND_Q6_K, 16, 512
    table = random_valid_blocks(np.random.default_rng(830), kind, vocab, dim)
    ids = np.array([3, 16, -2, 15, 2**40, 0], dtype=np.int64)
    ref = oracle.embedding_gather(kind, table, vocab, dim, ids)
    got = hip.embedding_gather(kind, table, vocab, dim, ids)
    assert np.array_equal(bits(got), bits(ref)) and not got[1].any() and not got[2].any() and not got[4].any()
    with pytest.raises(capi.MarmotHipError) as e:
        hip.embedding_gather(kind, table, vocab, dim, ids, bounds_check=True)
    assert e.value.code == -1 and "position 1" in e.value.detail
    # unsupported kinds and dtypes
    with pytest.raises(capi.MarmotHipError) as e:
        hip.embedding_gather(capi.KIND_Q8_K, table, vocab, dim, ids)
    assert e.value.code == -8
