"""GPU tests of the branch sections of the C ABI (marmot_hip_branch_begin / _next / _join): independent calls on
different streams give the bits of the same calls made one after the other, outside and inside a captured graph, with
calls that use the library's workspace in every branch (each branch has its own), and the misuse cases are refused."""
import numpy as np
import pytest

from marmot_amd import capi
from oracle.pyoracle import KIND_Q4_K, KIND_Q6_K, KIND_Q8_0
from tests.util import bits, gaussian

pytestmark = pytest.mark.gpu


@pytest.fixture()
def hip():
    from marmot_amd import HipBackend

    b = HipBackend(0)  # a device object of its own: every branch's workspace starts empty
    yield b
    b.close()


class Linear:
    """One linear with device buffers: weight [M,K] of `kind`, fp32 input [N,K], fp32 output [N,M]."""

    def __init__(self, hip, oracle, seed, kind, M, K, N):
        self.hip, self.kind, self.M, self.K, self.N = hip, kind, M, K, N
        self.blocks = oracle.quantize(kind, gaussian(seed, (M, K), 0.02))
        self.x = gaussian(seed + 1, (N, K))
        self.d_w, self.d_x = hip.to_device(self.blocks), hip.to_device(self.x)
        self.d_out = hip.alloc(N * M * 4)

    def run(self):
        self.hip.linear_d(self.kind, self.d_w, self.d_x, capi.DT_F32, self.N, self.K, self.M, self.d_out, capi.DT_F32)

    def poison(self):
        self.d_out.upload(np.full(self.N * self.M * 4, 0xFF, dtype=np.uint8))

    def result(self):
        return self.d_out.download(np.float32, (self.N, self.M))

    def free(self):
        for b in (self.d_w, self.d_x, self.d_out):
            b.free()


# every one of these packs its fp32 rows into the workspace (and the 64-row ones keep K-split partial sums there):
# with one workspace for all branches the results would mix
SHAPES = [(KIND_Q4_K, 512, 4096, 16), (KIND_Q6_K, 256, 2048, 16), (KIND_Q8_0, 384, 2048, 12), (KIND_Q4_K, 256, 4096, 64)]


def make_linears(hip, oracle):
    return [Linear(hip, oracle, 4100 + 10 * i, *shape) for i, shape in enumerate(SHAPES)]


def test_branches_match_sequential_calls(hip, oracle):
    linears = make_linears(hip, oracle)
    try:
        expected = []
        for lin in linears:
            lin.run()
            hip.synchronize()
            expected.append(lin.result())
        for rep in range(5):
            for lin in linears:
                lin.poison()
            hip.branches(*[lin.run for lin in linears])
            # no synchronize in between: the download is enqueued behind the join
            for i, lin in enumerate(linears):
                assert np.array_equal(bits(lin.result()), bits(expected[i])), f"repeat {rep}, branch {i}"
    finally:
        for lin in linears:
            lin.free()


def test_work_after_the_join_waits_for_every_branch(hip, oracle):
    """Two branches write one activation tensor each; the linears enqueued after the join read them."""
    K1, M1, N = 2048, 1024, 16
    kind = KIND_Q4_K
    wa = oracle.quantize(kind, gaussian(4200, (M1, K1), 0.02))
    wb = oracle.quantize(kind, gaussian(4201, (M1, K1), 0.02))
    wc = oracle.quantize(kind, gaussian(4202, (256, M1), 0.02))
    x = gaussian(4203, (N, K1))
    d_wa, d_wb, d_wc, d_x = (hip.to_device(a) for a in (wa, wb, wc, x))
    d_ya, d_yb = hip.alloc(N * M1 * 4), hip.alloc(N * M1 * 4)
    d_za, d_zb = hip.alloc(N * 256 * 4), hip.alloc(N * 256 * 4)
    try:
        def first(d_w, d_y):
            return lambda: hip.linear_d(kind, d_w, d_x, capi.DT_F32, N, K1, M1, d_y, capi.DT_F32)

        def second(d_y, d_z):
            hip.linear_d(kind, d_wc, d_y, capi.DT_F32, N, M1, 256, d_z, capi.DT_F32)

        first(d_wa, d_ya)()
        first(d_wb, d_yb)()
        second(d_ya, d_za)
        second(d_yb, d_zb)
        want = (d_za.download(np.float32, (N, 256)), d_zb.download(np.float32, (N, 256)))
        for rep in range(5):
            for b, n in ((d_ya, N * M1 * 4), (d_yb, N * M1 * 4), (d_za, N * 256 * 4), (d_zb, N * 256 * 4)):
                b.upload(np.full(n, 0xFF, dtype=np.uint8))
            hip.branches(first(d_wa, d_ya), first(d_wb, d_yb))
            second(d_ya, d_za)
            second(d_yb, d_zb)
            got = (d_za.download(np.float32, (N, 256)), d_zb.download(np.float32, (N, 256)))
            assert np.array_equal(bits(got[0]), bits(want[0])) and np.array_equal(bits(got[1]), bits(want[1])), rep
    finally:
        for b in (d_wa, d_wb, d_wc, d_x, d_ya, d_yb, d_za, d_zb):
            b.free()


def test_branches_inside_a_captured_graph(hip, oracle):
    linears = make_linears(hip, oracle)
    try:
        expected = []
        for lin in linears:
            lin.run()
            hip.synchronize()
            expected.append(lin.result())
        # every branch's workspace must have its size before the capture (a capture cannot allocate)
        hip.branches(*[lin.run for lin in linears])
        hip.synchronize()

        def body():
            hip.branches(*[lin.run for lin in linears])
            linears[0].run()  # behind the join, once more on the main stream

        g = hip.graph_capture(body)
        assert hip.graph_last_capture_nodes() >= len(linears) + 1
        try:
            for rep in range(4):
                for lin in linears:
                    lin.poison()
                hip.graph_launch(g)
                hip.synchronize()
                for i, lin in enumerate(linears):
                    assert np.array_equal(bits(lin.result()), bits(expected[i])), f"replay {rep}, branch {i}"
                # eager work of the program between the replays
                linears[rep % len(linears)].run()
                hip.synchronize()
        finally:
            hip.graph_destroy(g)
    finally:
        for lin in linears:
            lin.free()


def test_a_capture_cannot_grow_a_branch_workspace(hip, oracle):
    """The first branch's workspace is the main one and has its size from an eager call; the second branch's is still
    empty, so recording a call that needs it is refused with the usual message, and the device object stays usable."""
    a = Linear(hip, oracle, 4300, KIND_Q6_K, 256, 2048, 16)
    b = Linear(hip, oracle, 4310, KIND_Q6_K, 256, 2048, 16)
    try:
        a.run()
        b.run()
        hip.synchronize()
        want = b.result()
        hip.branches(lambda: None, lambda: None)  # the first section of a device object makes the side streams
        with pytest.raises(capi.MarmotHipError) as err:
            hip.graph_capture(lambda: hip.branches(a.run, b.run))
        assert err.value.code == -5 and "workspace" in err.value.detail and "eagerly" in err.value.detail
        hip.branches(a.run, b.run)  # sizes the second branch's workspace
        g = hip.graph_capture(lambda: hip.branches(a.run, b.run))
        b.poison()
        hip.graph_launch(g)
        hip.synchronize()
        assert np.array_equal(bits(b.result()), bits(want))
        hip.graph_destroy(g)
    finally:
        a.free()
        b.free()


def last_error(lib) -> str:
    return lib.marmot_hip_last_error().decode()


def test_misuse_is_refused(hip):
    lib, dev = hip.lib, hip.dev
    import ctypes as C

    # a device object's first section makes its side streams: not inside a capture
    g = C.c_void_p()
    buf = hip.alloc(64)
    assert lib.marmot_hip_graph_begin_capture(dev) == 0
    assert lib.marmot_hip_memset(dev, C.c_void_p(buf.ptr), 0, 64) == 0
    assert lib.marmot_hip_branch_begin(dev) == -5
    assert "side streams" in last_error(lib)
    assert lib.marmot_hip_graph_end_capture(dev, C.byref(g)) == 0
    hip.graph_destroy(g)
    buf.free()
    assert lib.marmot_hip_branch_next(dev) == -5  # no section
    assert lib.marmot_hip_branch_join(dev) == -5
    assert lib.marmot_hip_branch_begin(dev) == 0
    assert lib.marmot_hip_branch_begin(dev) == -5  # sections do not nest
    assert lib.marmot_hip_graph_begin_capture(dev) == -5  # no capture from inside a section
    for _ in range(3):
        assert lib.marmot_hip_branch_next(dev) == 0
    assert lib.marmot_hip_branch_next(dev) == -1  # a fifth branch
    assert "at most 4" in last_error(lib)
    assert lib.marmot_hip_branch_join(dev) == 0
    assert lib.marmot_hip_branch_join(dev) == -5
    # a section opened inside a capture must be joined before the capture ends
    assert lib.marmot_hip_graph_begin_capture(dev) == 0
    assert lib.marmot_hip_branch_begin(dev) == 0
    assert lib.marmot_hip_branch_next(dev) == 0
    g = C.c_void_p()
    assert lib.marmot_hip_graph_end_capture(dev, C.byref(g)) == -5
    assert "branch_join" in last_error(lib)
    assert lib.marmot_hip_branch_join(dev) == 0
    assert lib.marmot_hip_graph_end_capture(dev, C.byref(g)) == 0
    hip.graph_destroy(g)
    hip.synchronize()


def test_noalloc_entry_point_only_in_the_first_branch(hip, oracle):
    a = Linear(hip, oracle, 4400, KIND_Q4_K, 256, 1024, 4)
    b = Linear(hip, oracle, 4410, KIND_Q4_K, 256, 1024, 4)
    try:
        a.run()
        b.run()
        hip.synchronize()
        want = a.result()

        def noalloc():
            hip.linear_noalloc_d(a.kind, a.d_w, a.d_x, capi.DT_F32, a.N, a.K, a.M, a.d_out, capi.DT_F32)

        a.poison()
        hip.branches(noalloc, b.run)  # first branch: allowed
        assert np.array_equal(bits(a.result()), bits(want))
        with pytest.raises(capi.MarmotHipError) as err:
            hip.branches(b.run, noalloc)
        assert err.value.code == -5 and "first branch" in err.value.detail
        hip.synchronize()
    finally:
        a.free()
        b.free()
