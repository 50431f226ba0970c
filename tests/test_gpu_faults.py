"""Failure handling of the row-owning kernels: their wavefronts wait for one another through LDS words with a bounded
number of polls. With the limit forced to zero from the host every wavefront gives up at its first wait, the kernels
still run to their end, and the next synchronize reports MARMOT_HIP_ERROR_INVALID_OPERATION; a device object with the
default limit computes the same cases correctly afterwards."""
import numpy as np
import pytest

from oracle.pyoracle import KIND_Q4_K
from tests.util import assert_matmul_parity, gaussian, random_valid_blocks

pytestmark = pytest.mark.gpu

CASES = [  # (M, K, N, route): resident-share decode kernel, ring form of the row kernel, row-owning small-batch kernel
    (4096, 14336, 1, "matvec_rows2_q4_k_q8_k_fused"),
    (4096, 4096, 2, "matvec_rows_q4_k_q8_k_fused"),
    (4096, 4096, 8, "mmq_rows"),
]


@pytest.mark.parametrize("M,K,N,route", CASES)
def test_spin_limit_turns_a_stuck_workgroup_into_an_error(oracle, monkeypatch, M, K, N, route):
    from marmot_amd import HipBackend
    from marmot_amd.capi import MarmotHipError

    blocks = random_valid_blocks(np.random.Generator(np.random.PCG64(M + N)), KIND_Q4_K, M, K)
    x = gaussian(K + N, (N, K))
    monkeypatch.setenv("MARMOT_HIP_SPIN_LIMIT", "0")
    limited = HipBackend(0)
    monkeypatch.delenv("MARMOT_HIP_SPIN_LIMIT")
    try:
        d_w, d_x, d_o = limited.to_device(blocks), limited.to_device(x), limited.alloc(N * M * 4)
        limited.linear_d(KIND_Q4_K, d_w, d_x, 0, N, K, M, d_o, 0)
        assert route in limited.last_route(), limited.last_route()
        with pytest.raises(MarmotHipError) as e:
            limited.synchronize()
        assert e.value.code == -5 and "gave up waiting" in str(e.value)
        limited.synchronize()  # the mark is cleared once reported
    finally:
        limited.close()
    hip = HipBackend(0)
    try:
        got = hip.linear(x, blocks, KIND_Q4_K, M)
        assert route in hip.last_route()
        hip.synchronize()
        assert_matmul_parity(got, oracle.matmul(KIND_Q4_K, blocks, x, M, threads=16), what=f"{M}x{K} N={N}")
    finally:
        hip.close()
