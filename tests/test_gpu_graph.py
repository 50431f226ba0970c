"""GPU tests of the batched-submission (HIP graph) part of the C ABI: the node limit of one captured graph, the node
count query, and that executable graphs stay valid when the library's workspace grows after they were captured."""
import numpy as np
import pytest

from marmot_amd import capi
from oracle.pyoracle import KIND_Q4_K
from tests.util import bits, gaussian

pytestmark = pytest.mark.gpu


@pytest.fixture()
def hip():
    from marmot_amd import HipBackend

    b = HipBackend(0)  # a device object of its own: the workspace starts empty
    yield b
    b.close()


def test_node_limit_and_count(hip):
    limit = hip.graph_max_nodes()
    assert limit == 1024
    buf = hip.alloc(4096)
    try:
        g = hip.graph_capture(lambda: [hip.lib.marmot_hip_memset(hip.dev, buf.ptr, i & 0xFF, 4096) for i in range(7)])
        assert hip.graph_last_capture_nodes() == 7
        hip.graph_launch(g)
        hip.synchronize()
        assert np.all(buf.download(np.uint8, (4096,)) == 6)
        hip.graph_destroy(g)

        with pytest.raises(capi.MarmotHipError) as err:
            hip.graph_capture(lambda: [hip.lib.marmot_hip_memset(hip.dev, buf.ptr, 1, 4096) for _ in range(limit + 1)])
        assert err.value.code == -5  # INVALID_OPERATION
        assert "limit is 1024" in err.value.detail
        assert hip.graph_last_capture_nodes() == limit + 1
        # the device object is usable afterwards: exactly the limit is accepted
        g = hip.graph_capture(lambda: [hip.lib.marmot_hip_memset(hip.dev, buf.ptr, 9, 4096) for _ in range(limit)])
        hip.graph_launch(g)
        hip.synchronize()
        assert np.all(buf.download(np.uint8, (4096,)) == 9)
        hip.graph_destroy(g)
    finally:
        buf.free()


def test_graph_survives_workspace_growth(hip, oracle):
    """A captured small-batch matmul reads packed activations and K-split partials in the workspace. A later eager call
    with a larger shape makes the workspace grow; the old one must stay allocated while the graph lives, and replays
    give the same bits as before."""
    kind = KIND_Q4_K
    M, K, N = 256, 1024, 8
    blocks = oracle.quantize(kind, gaussian(800, (M, K), 0.02))
    x = gaussian(801, (N, K))
    d_w, d_x = hip.to_device(blocks), hip.to_device(x)
    d_out = hip.alloc(N * M * 4)
    hip.linear_d(kind, d_w, d_x, capi.DT_F32, N, K, M, d_out, capi.DT_F32)  # sizes the workspace for this shape
    eager = d_out.download(np.float32, (N, M))
    g = hip.graph_capture(lambda: hip.linear_d(kind, d_w, d_x, capi.DT_F32, N, K, M, d_out, capi.DT_F32))
    try:
        # much larger activations: the workspace is outgrown several times over
        big_blocks = oracle.quantize(kind, gaussian(802, (64, 16384), 0.02))
        for n_big in (64, 512):
            big = hip.linear(gaussian(803, (n_big, 16384)), big_blocks, kind, 64)
            assert big.shape == (n_big, 64)
        for rep in range(3):
            d_out.upload(np.full(N * M * 4, 0xFF, dtype=np.uint8))
            hip.graph_launch(g)
            hip.synchronize()
            assert np.array_equal(bits(d_out.download(np.float32, (N, M))), bits(eager)), f"replay {rep}"
    finally:
        hip.graph_destroy(g)
        for b in (d_w, d_x, d_out):
            b.free()
