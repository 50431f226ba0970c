"""GPU: weights taken from a GGUF file through the library's reader: uploaded with marmot_hip_gguf_upload and used by
the raw-pointer matmul, and used in place (views into the file mapping) by the tensor-level backend, whose residency
table mirrors them once. Results against the CPU oracle on the weights that were written to the file."""
import numpy as np
import pytest

from marmot_amd import capi
from marmot_amd import tensor_abi as ta
from marmot_amd.gguf import GgufFile
from oracle.pyoracle import KINDS
from tests.gguf_writer import write_gguf
from tests.util import assert_matmul_parity, gaussian

pytestmark = pytest.mark.gpu

M, K = 96, 1024
NAMES = ["q4_k", "q5_k", "q6_k", "q8_0", "q3_k", "q5_0"]


@pytest.fixture(scope="module")
def model(tmp_path_factory, oracle):
    weights = {n: oracle.quantize(KINDS[n], gaussian(1000 + i, (M, K), 0.02)) for i, n in enumerate(NAMES)}
    tensors = [(f"blk.0.{n}.weight", n, (K, M), w) for n, w in weights.items()]
    tensors.append(("blk.0.bias", "f32", (M,), gaussian(1100, (M,))))
    path = write_gguf(str(tmp_path_factory.mktemp("gguf") / "model.gguf"), tensors, kv={"general.architecture": "test"})
    return path, weights


def test_uploaded_tensors_feed_the_matmul(model, oracle):
    from marmot_amd import HipBackend

    path, weights = model
    hip = HipBackend(0)
    try:
        with GgufFile(path) as g:
            x = gaussian(1200, (5, K))
            d_x = hip.to_device(x)
            d_o = hip.alloc(5 * M * 4)
            for n in NAMES:
                print(f"gguf upload {n}", flush=True)
                info = g.find(f"blk.0.{n}.weight")
                assert info.kind == KINDS[n] and info.shape == (M, K)
                d_w = g.upload(hip, info)
                hip.linear_d(info.kind, d_w, d_x, capi.DT_F32, 5, K, M, d_o, capi.DT_F32)
                got = d_o.download(np.float32, (5, M))
                assert_matmul_parity(got, oracle.matmul(info.kind, weights[n], x, M), what=f"gguf {n}")
                d_w.free()
            d_x.free()
            d_o.free()
    finally:
        hip.close()


def test_views_into_the_mapping_are_mirrored_once(model, oracle):
    path, weights = model
    with ta.HipContext() as ctx, GgufFile(path) as g:
        info = g.find("blk.0.q4_k.weight")
        bias_info = g.find("blk.0.bias")
        wt = ta.HostTensor.quantized(g.array(info), info.shape, info.kind)
        bt = ta.HostTensor.dense(g.array(bias_info))
        assert wt.t.data == info.address and bt.t.data == bias_info.address  # no copies: the file's pages
        x = gaussian(1300, (3, K))
        xt = ta.HostTensor.dense(x)
        yt = ta.HostTensor.empty((3, M), ta.DTYPE_F32)
        sel = ctx.query(ctx.matmul_signature(xt, wt, yt, bias=True))
        assert sel.supported
        before = ctx.residency().upload_bytes
        for run in range(2):
            prog = ta.Program()
            prog.matmul(sel.op_index, xt, wt, yt, bias=bt)
            assert ctx.execute(prog) == ta.SUCCESS, ctx.last_error()
            got = ctx.to_host(yt).copy()
            if run == 0:
                first = ctx.residency().upload_bytes - before
        assert first >= info.nbytes and ctx.residency().upload_bytes - before == first  # nothing uploaded twice
        ref = oracle.matmul(info.kind, weights["q4_k"], x, M, bias=g.array(bias_info).copy())
        assert_matmul_parity(got, ref, what="gguf view through the residency table")
        # what unloading the file does in the core: the backend forgets the host range before it is unmapped
        mirrors = ctx.residency().mirrors
        for t in (wt, bt, xt, yt):
            ctx.host_freed(t)
        assert ctx.residency().mirrors == mirrors - 4


def test_session_style_preload_then_linears_upload_nothing(model, oracle):
    """What an execution session does with a model's weights (marmot_tensor_to_device on every tensor before the
    first token, src/graph/execution_session.cpp:315-320): each announced view is mirrored and uploaded at once, the
    architecture comes from the file's metadata, and the linears that follow upload only their activations."""
    path, weights = model
    with ta.HipContext() as ctx, GgufFile(path) as g:
        assert g.get("general.architecture") == "test"
        tensors = {}
        base = ctx.residency()
        total = 0
        for n in NAMES:
            info = g.find(f"blk.0.{n}.weight")
            t = ta.HostTensor.quantized(g.array(info), info.shape, info.kind)
            ctx.host_changed(t)  # marmot_tensor_to_device: dst == src == the host pointer
            tensors[n] = (info, t)
            total += info.nbytes
        loaded = ctx.residency()
        assert loaded.mirrors == base.mirrors + len(NAMES) and loaded.uploads == base.uploads + len(NAMES)
        assert loaded.upload_bytes - base.upload_bytes == total
        x = gaussian(1400, (2, K))
        for n, (info, wt) in tensors.items():
            xt = ta.HostTensor.dense(x)
            yt = ta.HostTensor.empty((2, M), ta.DTYPE_F32)
            before = ctx.residency()
            prog = ta.Program()
            prog.matmul(ctx.query(ctx.matmul_signature(xt, wt, yt)).op_index, xt, wt, yt)
            assert ctx.execute(prog) == ta.SUCCESS, ctx.last_error()
            after = ctx.residency()
            assert after.upload_bytes - before.upload_bytes == x.nbytes, n   # the activations only
            assert_matmul_parity(ctx.to_host(yt), oracle.matmul(info.kind, weights[n], x, M), what=f"preloaded {n}")
            ctx.host_freed(xt)
            ctx.host_freed(yt)
        for _, t in tensors.values():
            ctx.host_freed(t)
