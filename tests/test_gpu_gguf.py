"""GPU: weights taken from a GGUF file through the library's reader: uploaded with marmot_hip_gguf_upload and used by
the raw-pointer matmul, and used in place (views into the file mapping) by the tensor-level backend, whose residency
table mirrors them once. Results against the CPU oracle on the weights that were written to the file."""
import ctypes as C

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


def test_synthetic_moe_file_of_the_reference_loader_test_on_the_device(oracle):
    """The file laid out like the reference's synthetic MoE model (tests/graph/test_gguf_loader.c:171-256; tensors at
    offsets that are 16 modulo 32): every tensor uploads to the bytes the file holds, and tensors used in place (views
    into the mapping at those offsets) go through the residency table into device operations: the final
    normalization's weight, the router projection's rows gathered by expert id, the softmax over the two experts."""
    import os

    from marmot_amd import HipBackend

    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "synthetic_qwen3moe.gguf")
    hip = HipBackend(0)
    try:
        with GgufFile(path) as g:
            for t, info in enumerate(g.tensors):
                print(f"synthetic gguf upload {info.name}", flush=True)
                d = g.upload(hip, info)
                n = info.nbytes // 4
                want = np.float32(t) + np.arange(n, dtype=np.float32) / np.float32(1024.0)
                assert np.array_equal(d.download(np.float32, (n,)), want), info.name
                d.free()
    finally:
        hip.close()
    with ta.HipContext() as ctx, GgufFile(path) as g:
        norm = g.find("blk.0.attn_k_norm.weight")   # 16 bytes, at an offset that is 16 modulo 32
        router = g.find("blk.0.ffn_gate_inp.weight")  # [experts = 2, hidden = 8]
        assert (norm.address - g.tensors[0].address) % 32 == 16
        wt = ta.HostTensor.strided(g.array(norm))
        x = gaussian(1300, (3, 4))
        xt, ot = ta.HostTensor.dense(x), ta.HostTensor.empty((3, 4), ta.DTYPE_F32)
        desc = ta.RmsNormDesc(xt.ptr, None, wt.ptr, ot.ptr, g.get("qwen3moe.attention.layer_norm_rms_epsilon"))
        assert ctx.lib.hip_rmsnorm_impl(ctx.device_ctx, C.byref(desc)) == ta.SUCCESS, ctx.last_error()
        ref = oracle.rms_norm(x, g.array(norm).copy(), eps=float(np.float32(1e-5)))
        assert np.allclose(ctx.to_host(ot), ref, rtol=1e-5, atol=1e-8)
        rt = ta.HostTensor.strided(g.array(router))
        ids = ta.HostTensor.dense(np.array([1, 0, 1], np.int32))
        rows = ta.HostTensor.empty((3, 8), ta.DTYPE_F32)
        probs = ta.HostTensor.empty((3, 8), ta.DTYPE_F32)
        prog = ta.Program()
        prog.gather_rows(ta.BC_OP_GATHER_ROWS, rt, ids, rows)
        prog.softmax(ta.BC_OP_SOFTMAX_F32, rows, probs, -1)
        assert ctx.execute(prog) == ta.SUCCESS, ctx.last_error()
        assert np.array_equal(ctx.to_host(rows), g.array(router)[[1, 0, 1]])
        assert np.allclose(ctx.to_host(probs), oracle.softmax(g.array(router)[[1, 0, 1]].copy()), rtol=3e-6)
        for t in (wt, xt, ot, rt, ids, rows, probs):
            ctx.host_range_freed(t)
