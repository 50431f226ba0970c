"""The entry point that allocates nothing (marmot_hip_matmul_quantized_noalloc) against marmot_hip_matmul_quantized,
through the C ABI: same bits, on two calls in a row, the second with a smaller input (the static scratch array keeps the
first call's contents), for the routes that use scratch: the int8 small-batch kernel (quantized activations and K-split
partial sums) and the fp16 prefill GEMM (sub-block sums and partial sums). Oversized requests are refused."""
import numpy as np
import pytest

from marmot_amd import capi
from oracle.pyoracle import KIND_Q4_K, KIND_Q6_K
from tests.util import bits, gaussian

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def hip():
    from marmot_amd import HipBackend

    b = HipBackend(0)
    yield b
    b.close()


def run_pair(hip, oracle, kind, shapes, in_dtype):
    """shapes: [(N, K, M), ...] run in this order through the no-alloc entry point, each compared with the allocating one."""
    for idx, (N, K, M) in enumerate(shapes):
        blocks = oracle.quantize(kind, gaussian(900 + idx, (M, K), 0.02))
        x = gaussian(910 + idx, (N, K))
        if in_dtype == capi.DT_F16:
            x = x.astype(np.float16)
        d_w, d_x = hip.to_device(blocks), hip.to_device(x)
        d_ref, d_got = hip.alloc(N * M * 4), hip.alloc(N * M * 4)
        try:
            hip.linear_d(kind, d_w, d_x, in_dtype, N, K, M, d_ref, capi.DT_F32)
            route = hip.last_route()
            ref = d_ref.download(np.float32, (N, M))
            d_got.upload(np.full(N * M * 4, 0xFF, dtype=np.uint8))
            hip.linear_noalloc_d(kind, d_w, d_x, in_dtype, N, K, M, d_got, capi.DT_F32)
            assert hip.last_route() == route
            got = d_got.download(np.float32, (N, M))
            assert np.array_equal(bits(got), bits(ref)), f"call {idx} {(N, K, M)} route {route}"
        finally:
            for b in (d_w, d_x, d_ref, d_got):
                b.free()
        yield route


def test_small_batch_routes_two_calls_in_a_row(hip, oracle):
    # 16 activation rows with a K split over workgroups (few row groups), then a smaller call
    routes = list(run_pair(hip, oracle, KIND_Q4_K, [(16, 4096, 1024), (5, 1024, 320)], capi.DT_F32))
    assert all("mmq_" in r for r in routes), routes
    routes = list(run_pair(hip, oracle, KIND_Q6_K, [(12, 2048, 512), (6, 1024, 96)], capi.DT_F32))
    assert all("mmq_" in r for r in routes), routes


def test_prefill_gemm_two_calls_in_a_row(hip, oracle):
    routes = list(run_pair(hip, oracle, KIND_Q4_K, [(128, 2048, 1024), (64, 1024, 512)], capi.DT_F16))
    assert all("gemm_" in r for r in routes), routes


def test_packed_matvec_and_fused_routes(hip, oracle):
    # 8-row tiles of a 32-value format go through the packed scratch; one row is quantized inside the kernel (no scratch)
    from oracle.pyoracle import KIND_Q8_0

    list(run_pair(hip, oracle, KIND_Q8_0, [(8, 2048, 640), (1, 1024, 128)], capi.DT_F32))


def test_oversized_request_is_refused(hip, oracle):
    kind = KIND_Q4_K
    N, K, M = 1024, 8192, 64  # 1024 rows of 8192 int8 values alone exceed the 8 MiB array
    blocks = oracle.quantize(kind, gaussian(950, (M, K), 0.02))
    d_w, d_x = hip.to_device(blocks), hip.to_device(gaussian(951, (N, K)))
    d_out = hip.alloc(N * M * 4)
    try:
        with pytest.raises(capi.MarmotHipError) as err:
            hip.linear_noalloc_d(kind, d_w, d_x, capi.DT_F32, N, K, M, d_out, capi.DT_F32)
        assert err.value.code == -1 and "does not allocate" in err.value.detail
        # the allocating entry point takes the same call, and the device object still works afterwards
        hip.linear_d(kind, d_w, d_x, capi.DT_F32, N, K, M, d_out, capi.DT_F32)
        hip.linear_noalloc_d(kind, d_w, d_x, capi.DT_F32, 8, K, M, d_out, capi.DT_F32)
    finally:
        for b in (d_w, d_x, d_out):
            b.free()
