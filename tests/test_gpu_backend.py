"""GPU tests of the marmot_tensor_t-level backend: device vtable + residency table, impl functions, and bytecode
programs executed through the exported tables (config 4, the seven linears of one layer at 16 tokens, runs as one
program). Every result is compared with the CPU oracle on the same seeded inputs."""
import ctypes as C

import numpy as np
import pytest

from marmot_amd import tensor_abi as ta
from oracle.pyoracle import (KIND_Q8_1, KIND_Q2_K, KIND_Q3_K, KIND_Q4_0, KIND_Q4_1, KIND_Q4_K, KIND_Q5_0, KIND_Q5_1, KIND_Q5_K, KIND_Q6_K, KIND_Q8_0,
                             KIND_Q8_K, row_bytes)
from tests.test_oracle_moe import make_experts
from tests.util import assert_matmul_parity, assert_moe_parity, bits, gaussian, quantize_weights

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    with ta.HipContext() as c:
        yield c


def _linear(ctx, kind, wq, M, K, x, bias=None, out_dtype=ta.DTYPE_F32):
    xt = ta.HostTensor.dense(x)
    wt = ta.HostTensor.quantized(wq, (M, K), kind)
    yt = ta.HostTensor.empty((x.shape[0], M), out_dtype)
    bt = ta.HostTensor.dense(bias) if bias is not None else None
    ep = None
    if bt is not None:
        ep = ta.Epilogue()
        ep.bias = bt.ptr
    fn = getattr(ctx.lib, {KIND_Q4_0: "hip_matmul_quantized_q4_0", KIND_Q8_0: "hip_matmul_quantized_q8_0",
                           KIND_Q4_1: "hip_matmul_quantized_q4_1", KIND_Q5_0: "hip_matmul_quantized_q5_0",
                           KIND_Q5_1: "hip_matmul_quantized_q5_1", KIND_Q2_K: "hip_matmul_quantized_q2_k", KIND_Q8_1: "hip_matmul_quantized_q8_1",
                           KIND_Q3_K: "hip_matmul_quantized_q3_k",
                           KIND_Q4_K: "hip_matmul_quantized_q4_k", KIND_Q5_K: "hip_matmul_quantized_q5_k",
                           KIND_Q6_K: "hip_matmul_quantized_q6_k"}[kind])
    st = fn(ctx.device_ctx, xt.ptr, wt.ptr, C.byref(ep) if ep is not None else None, yt.ptr)
    if st == ta.SUCCESS:
        ctx.to_host(yt)
    # what tensor destruction does in the core: the backend forgets the host ranges (src/core/tensor/create.c)
    for t in (xt, wt, yt, bt):
        if t is not None:
            ctx.host_freed(t)
    return st, xt, wt, yt


@pytest.mark.parametrize("kind", [KIND_Q4_0, KIND_Q4_1, KIND_Q5_0, KIND_Q5_1, KIND_Q8_0, KIND_Q8_1, KIND_Q2_K, KIND_Q3_K,
                                  KIND_Q4_K, KIND_Q5_K, KIND_Q6_K])
def test_impl_matmul_matches_oracle(ctx, oracle, kind):
    print(f"backend impl matmul kind={kind}", flush=True)
    M, K, N = 96, 512, 5
    wq = oracle.quantize(kind, gaussian(700 + kind, (M, K), 0.02))
    x = gaussian(710 + kind, (N, K))
    bias = gaussian(720 + kind, (M,))
    st, xt, wt, yt = _linear(ctx, kind, wq, M, K, x, bias=bias)
    assert st == ta.SUCCESS, ctx.last_error()
    # outputs are flagged device-resident until the core asks for them (_linear already did)
    assert yt.t.memory_location == ta.MEMORY_DEVICE and not yt.t.needs_sync
    assert_matmul_parity(yt.array, oracle.matmul(kind, wq, x, M, bias=bias), what=f"impl kind={kind}")


@pytest.mark.parametrize("kind", [KIND_Q4_K, KIND_Q5_K, KIND_Q6_K])
def test_impl_matmul_prompt_rows(ctx, oracle, kind):
    """A prompt's worth of fp32 rows through the tensor-level entry (the tiled int8 GEMMs behind it): 100 rows, ragged
    tiles, bias, host tensors mirrored by the residency layer."""
    M, K, N = 200, 2048, 100
    wq = oracle.quantize(kind, gaussian(740 + kind, (M, K), 0.02))
    x = gaussian(741 + kind, (N, K))
    bias = gaussian(742 + kind, (M,))
    st, xt, wt, yt = _linear(ctx, kind, wq, M, K, x, bias=bias)
    assert st == ta.SUCCESS, ctx.last_error()
    assert_matmul_parity(yt.array, oracle.matmul(kind, wq, x, M, bias=bias), what=f"impl prompt rows kind={kind}")
    for t in (xt, wt, yt):
        ctx.host_freed(t)


def test_impl_matmul_fp16_and_errors(ctx, oracle):
    M, K, N = 64, 512, 3
    wq = oracle.quantize(KIND_Q4_K, gaussian(730, (M, K), 0.02))
    x16 = gaussian(731, (N, K)).astype(np.float16)
    st, xt, wt, yt = _linear(ctx, KIND_Q4_K, wq, M, K, x16, out_dtype=ta.DTYPE_F16)
    assert st == ta.SUCCESS, ctx.last_error()
    ref = oracle.matmul(KIND_Q4_K, wq, x16, M, out_dtype=np.float16)
    assert_matmul_parity(yt.array.astype(np.float32), ref.astype(np.float32), tol=2e-3, what="f16 out")
    # error codes of marmot_matmul_validate_quantized
    st, *_ = _linear(ctx, KIND_Q4_K, wq, M, K, gaussian(732, (N, K)), out_dtype=ta.DTYPE_F16)
    assert st == ta.UNSUPPORTED_DTYPE and "FLOAT32 input or FLOAT16" in ctx.last_error()[1]
    st, *_ = _linear(ctx, KIND_Q4_K, wq, M, K, gaussian(733, (N, K + 256)))
    assert st == ta.DIMENSION_MISMATCH and "mismatch on K" in ctx.last_error()[1]
    # a Q6_K weight handed to the Q4_K entry: not implemented -> caller falls back
    w6 = oracle.quantize(KIND_Q6_K, gaussian(734, (M, K), 0.02))
    xt = ta.HostTensor.dense(gaussian(735, (N, K)))
    wt = ta.HostTensor.quantized(w6, (M, K), KIND_Q6_K)
    yt = ta.HostTensor.empty((N, M), ta.DTYPE_F32)
    assert ctx.lib.hip_matmul_quantized_q4_k(ctx.device_ctx, xt.ptr, wt.ptr, None, yt.ptr) == ta.NOT_IMPLEMENTED
    # Q6_K with fp16 activations takes the reference's direct fp16 dot, like every other format
    st, _, _, y6 = _linear(ctx, KIND_Q6_K, w6, M, K, x16)
    assert st == ta.SUCCESS, ctx.last_error()
    assert_matmul_parity(y6.array.astype(np.float32), oracle.matmul(KIND_Q6_K, w6, x16, M).astype(np.float32),
                         tol=2e-3, what="Q6_K f16 direct")
    # generic (non block-quantized) weight
    wt.t.quant_kind = ta.KIND_GENERIC
    assert ctx.lib.hip_matmul_quantized_q6_k(ctx.device_ctx, xt.ptr, wt.ptr, None, yt.ptr) == ta.UNSUPPORTED_DTYPE
    assert "not block-quantized" in ctx.last_error()[1]
    for t in (xt, wt, yt):
        ctx.host_freed(t)


def test_residency_table(ctx, oracle):
    """Weights are uploaded once; a host update is re-uploaded on next use; views resolve inside a mirror; freed
    host ranges drop their mirrors."""
    M, K, N = 64, 256, 2
    kind = KIND_Q8_0
    wq = oracle.quantize(kind, gaussian(740, (2 * M, K), 0.02))
    stack = ta.HostTensor.quantized(wq, (2 * M, K), kind)   # two [M,K] weights in one host allocation
    x = ta.HostTensor.dense(gaussian(741, (N, K)))
    y = ta.HostTensor.empty((N, 2 * M), ta.DTYPE_F32)
    base = ctx.residency()
    fn = ctx.lib.hip_matmul_quantized_q8_0
    assert fn(ctx.device_ctx, x.ptr, stack.ptr, None, y.ptr) == ta.SUCCESS
    s1 = ctx.residency()
    assert s1.mirrors == base.mirrors + 3 and s1.uploads == base.uploads + 2  # weight + input; output not uploaded
    ref_full = oracle.matmul(kind, wq, x.array, 2 * M)
    assert_matmul_parity(ctx.to_host(y), ref_full, what="stack")
    # second call: nothing is uploaded again
    assert fn(ctx.device_ctx, x.ptr, stack.ptr, None, y.ptr) == ta.SUCCESS
    assert ctx.residency().uploads == s1.uploads
    # a view of the second half of the stack (what an expert slice or a GGUF tensor inside a mapped file is)
    half = row_bytes(kind, K) * M
    view = ta.HostTensor.quantized(wq.reshape(-1)[half:], (M, K), kind)
    view.t.data = stack.t.data + half
    yv = ta.HostTensor.empty((N, M), ta.DTYPE_F32)
    assert fn(ctx.device_ctx, x.ptr, view.ptr, None, yv.ptr) == ta.SUCCESS
    s2 = ctx.residency()
    assert s2.mirrors == s1.mirrors + 1 and s2.uploads == s1.uploads  # only the new output got a mirror
    assert np.array_equal(bits(ctx.to_host(yv)), bits(np.ascontiguousarray(ctx.to_host(y)[:, M:])))
    # host copy of the input changes: declared with memcpy_to_device(p, p), re-uploaded on next use
    x.array[:] = gaussian(742, (N, K))
    ctx.host_changed(x)
    assert fn(ctx.device_ctx, x.ptr, stack.ptr, None, y.ptr) == ta.SUCCESS
    assert ctx.residency().uploads == s2.uploads + 1
    assert_matmul_parity(ctx.to_host(y), oracle.matmul(kind, wq, x.array, 2 * M), what="after host update")
    # freeing the host ranges drops the mirrors
    for t in (stack, x, y, yv):
        ctx.host_freed(t)
    assert ctx.residency().mirrors == base.mirrors
    # raw device memory through alloc/free and plain copies (dst != src)
    d = C.c_void_p()
    assert ctx.ops.alloc(ctx.device_ctx, 4096, C.byref(d)) == ta.SUCCESS
    src = np.arange(1024, dtype=np.int32)
    dst = np.zeros_like(src)
    assert ctx.ops.memcpy_to_device(ctx.device_ctx, d, src.ctypes.data, 4096) == ta.SUCCESS
    assert ctx.ops.memcpy_from_device(ctx.device_ctx, dst.ctypes.data, d, 4096) == ta.SUCCESS
    assert np.array_equal(src, dst)
    usage = ta.AllocatorUsage()
    assert ctx.ops.allocator_usage(ctx.device_ctx, C.byref(usage)) == ta.SUCCESS and usage.current_bytes >= 4096
    ctx.ops.free(ctx.device_ctx, d)
    assert ctx.ops.graph_batch_begin(ctx.device_ctx) == ta.SUCCESS
    assert ctx.ops.graph_batch_end(ctx.device_ctx, True) == ta.SUCCESS


def test_program_quantize_dequantize_topk(ctx, oracle):
    rows, k = 7, 512
    x = gaussian(750, (rows, k))
    xt = ta.HostTensor.dense(x)
    p = ta.Program()
    outs = {}
    for kind in (KIND_Q8_0, KIND_Q8_K, KIND_Q4_K, KIND_Q5_K, KIND_Q6_K):
        qt = ta.HostTensor(np.zeros(rows * row_bytes(kind, k), np.uint8), (rows, k), ta.DTYPE_I8, kind)
        back = ta.HostTensor.empty((rows, k), ta.DTYPE_F32)
        sel = ctx.query(_sig_for(ta.OP_QUANTIZE, kind))
        p.quantize(sel.op_index, xt, qt)
        p.dequantize(ctx.query(_sig_for(ta.OP_DEQUANTIZE, kind)).op_index, qt, back)
        outs[kind] = (qt, back)
    logits = ta.HostTensor.dense(gaussian(751, (rows, 40)))
    vals = ta.HostTensor.empty((rows, 6), ta.DTYPE_F32)
    idx = ta.HostTensor.empty((rows, 6), ta.DTYPE_I32)
    p.topk(ctx.query(_sig_for(ta.OP_TOPK, 0)).op_index, logits, vals, idx, 6)
    assert ctx.execute(p) == ta.SUCCESS, ctx.last_error()
    for kind, (qt, back) in outs.items():
        if kind in (KIND_Q8_0, KIND_Q8_K):
            ref_q = np.stack([oracle.pack(kind, x[r]) for r in range(rows)])
        else:
            ref_q = oracle.quantize(kind, x)  # the K-quant weight quantizers (cpu_quantize_q4_k / _q5_k / _q6_k)
        assert np.array_equal(ctx.to_host(qt).reshape(rows, -1), ref_q)
        assert np.array_equal(bits(ctx.to_host(back)), bits(oracle.dequantize(kind, ref_q, k)))
    ov, oi = oracle.topk(logits.array, 6)
    assert np.array_equal(ctx.to_host(idx), oi) and np.array_equal(bits(ctx.to_host(vals)), bits(ov))
    # malformed program: opcode out of range
    bad = ta.Program()
    bad.code += (99).to_bytes(2, "little")
    assert ctx.execute(bad) == ta.INVALID_ARGUMENT
    for t in p.regs:
        ctx.host_freed(t)


def _sig_for(op, kind):
    s = ta.OpSignature()
    s.op_id = op
    s.input_dtype = ta.DTYPE_F32
    s.output_dtype = ta.DTYPE_F32
    s.accum_dtype = ta.DTYPE_F32
    s.qscheme_id = ta.QSCHEME_OF_KIND.get(kind, 0)
    return s


def test_program_moe_experts(ctx, oracle):
    E, F, H, k, T = 6, 256, 512, 3, 9
    kind = KIND_Q4_K
    gate, up, down = make_experts(oracle, 760, E, F, H, kind, kind)
    hidden = gaussian(761, (T, H))
    logits = gaussian(762, (T, E))
    vals, ids = oracle.topk(logits, k)
    w = oracle.softmax_rows(vals)
    ref = oracle.moe_experts(hidden, gate, up, down, ids, w, F, E, kind, kind, threads=4)
    ht = ta.HostTensor.dense(hidden)
    gt = ta.HostTensor.quantized(gate, (H, F, E), kind)
    ut = ta.HostTensor.quantized(up, (H, F, E), kind)
    dt = ta.HostTensor.quantized(down, (F, H, E), kind)
    it = ta.HostTensor.dense(ids)
    wt = ta.HostTensor.dense(w)
    ot = ta.HostTensor.empty((T, H), ta.DTYPE_F32)
    p = ta.Program()
    sel = ctx.query(_sig_for(ta.OP_MOE_EXPERTS, kind))
    assert sel.supported
    p.moe_experts(sel.op_index, ht, gt, ut, dt, it, wt, ot, ffn_type=0, weights_scale=1.0, policy=1)
    assert ctx.execute(p) == ta.SUCCESS, ctx.last_error()
    assert_moe_parity(ctx.to_host(ot), ref, what="program moe")
    # shape disagreement is reported, not executed
    bad = ta.HostTensor.quantized(down, (F, H + 256, E), kind)
    p2 = ta.Program()
    p2.moe_experts(sel.op_index, ht, gt, ut, bad, it, wt, ot)
    assert ctx.execute(p2) == ta.DIMENSION_MISMATCH
    for t in p.regs:
        ctx.host_freed(t)


def test_config4_layer_stack_as_one_program(ctx, oracle):
    """Config 4: q, k, o, gate, up as Q4_K and v, down as Q6_K at 16 tokens, fp32 activations, each linear fed its
    seeded input (q/k/v share one, gate/up share one); the dense ops between them are not part of the config.
    Bit-exact dequantization of every weight and 1e-3 matmul parity per linear."""
    print("config 4 layer stack", flush=True)
    N = 16
    specs = [  # name, kind, M, K, seed, input
        ("q", KIND_Q4_K, 4096, 4096, 40, "x"), ("k", KIND_Q4_K, 1024, 4096, 41, "x"),
        ("v", KIND_Q6_K, 1024, 4096, 42, "x"), ("o", KIND_Q4_K, 4096, 4096, 43, "a"),
        ("gate", KIND_Q4_K, 14336, 4096, 44, "h"), ("up", KIND_Q4_K, 14336, 4096, 45, "h"),
        ("down", KIND_Q6_K, 4096, 14336, 46, "f"),
    ]
    inputs = {"x": gaussian(47, (N, 4096)), "a": gaussian(470, (N, 4096)), "h": gaussian(471, (N, 4096)),
              "f": gaussian(48, (N, 14336))}
    in_t = {k: ta.HostTensor.dense(v) for k, v in inputs.items()}
    p = ta.Program()
    layers = []
    weight_bytes = 0
    for name, kind, M, K, seed, src in specs:
        wq = quantize_weights(oracle, kind, gaussian(seed, (M, K), 0.02))
        wt = ta.HostTensor.quantized(wq, (M, K), kind)
        yt = ta.HostTensor.empty((N, M), ta.DTYPE_F32)
        sel = ctx.query(ctx.matmul_signature(in_t[src], wt, yt))
        assert sel.supported, name
        p.matmul(sel.op_index, in_t[src], wt, yt)
        layers.append((name, kind, M, K, wq, wt, yt, src))
        weight_bytes += wq.size
    assert weight_bytes == 138_903_552
    before = ctx.residency()
    assert ctx.ops.graph_batch_begin(ctx.device_ctx) == ta.SUCCESS
    assert ctx.execute(p) == ta.SUCCESS, ctx.last_error()
    assert ctx.ops.graph_batch_end(ctx.device_ctx, True) == ta.SUCCESS
    after = ctx.residency()
    assert after.upload_bytes - before.upload_bytes == weight_bytes + sum(v.nbytes for v in inputs.values())
    for name, kind, M, K, wq, wt, yt, src in layers:
        ref = oracle.matmul(kind, wq, inputs[src], M, threads=16)
        m = assert_matmul_parity(ctx.to_host(yt), ref, what=f"config 4 {name}")
        print(f"  {name}: floored-rel {m[0]:.2e} sum-rel {m[1]:.2e}", flush=True)
    # second execution: weights stay resident, only nothing new is uploaded
    assert ctx.execute(p) == ta.SUCCESS
    assert ctx.residency().upload_bytes == after.upload_bytes
    # bit-exact dequantization of EVERY row of each weight through the DEQUANTIZE schema, in bands of 2048 rows (a band
    # is a view into the resident weight: 29M floats at a time instead of 58M .. 235M)
    for name, kind, M, K, wq, wt, yt, src in layers:
        rb = row_bytes(kind, K)
        for r0 in range(0, M, 2048):
            rows = min(2048, M - r0)
            sub = ta.HostTensor.quantized(wq.reshape(-1)[r0 * rb: (r0 + rows) * rb], (rows, K), kind)
            sub.t.data = wt.t.data + r0 * rb  # a view of the resident weight
            dq = ta.HostTensor.empty((rows, K), ta.DTYPE_F32)
            pd = ta.Program()
            pd.dequantize(ctx.query(_sig_for(ta.OP_DEQUANTIZE, kind)).op_index, sub, dq)
            assert ctx.execute(pd) == ta.SUCCESS, ctx.last_error()
            got = ctx.to_host(dq)
            ref = oracle.dequantize(kind, wq[r0:r0 + rows], K)
            assert np.array_equal(bits(got), bits(ref)), f"dequant {name} rows {r0}.."
            ctx.host_freed(dq)
    for t in p.regs:
        ctx.host_freed(t)


def _qkv_tensors(kind, ws, M, K, x, biases):
    xt = ta.HostTensor.dense(x)
    wts = [ta.HostTensor.quantized(w, (M, K), kind) for w in ws]
    dt = ta.DTYPE_F16 if x.dtype == np.float16 else ta.DTYPE_F32
    outs = [ta.HostTensor.empty((x.shape[0], M), dt) for _ in range(3)]
    bts = [ta.HostTensor.dense(b) if b is not None else None for b in biases]
    return xt, wts, outs, bts


@pytest.mark.parametrize("kind", [KIND_Q4_0, KIND_Q4_1, KIND_Q5_0, KIND_Q5_1, KIND_Q8_0, KIND_Q8_1, KIND_Q2_K, KIND_Q3_K,
                                  KIND_Q4_K, KIND_Q5_K, KIND_Q6_K])
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_impl_qkv_matches_oracle(ctx, oracle, kind, dtype):
    """hip_matmul_qkv_{scheme} with a marmot_matmul_qkv_desc_t (separate layout) and through a bytecode program."""
    print(f"backend impl qkv kind={kind} dtype={np.dtype(dtype).name}", flush=True)
    M, K, N = 96, 512, 6
    ws = [oracle.quantize(kind, gaussian(900 + kind + i, (M, K), 0.02)) for i in range(3)]
    x = gaussian(910 + kind, (N, K)).astype(dtype)
    biases = [gaussian(920 + kind, (M,)).astype(dtype), None, gaussian(921 + kind, (M,)).astype(dtype)]
    ref = oracle.matmul_qkv(kind, *ws, x, M, bq=biases[0], bv=biases[2])
    xt, wts, outs, bts = _qkv_tensors(kind, ws, M, K, x, biases)
    desc = ta.QkvDesc()
    desc.input = xt.ptr
    desc.layout = ta.QKV_LAYOUT_SEPARATE
    desc.separate.wq, desc.separate.wk, desc.separate.wv = (w.ptr for w in wts)
    desc.separate.bq, desc.separate.bv = bts[0].ptr, bts[2].ptr
    desc.out_q, desc.out_k, desc.out_v = (o.ptr for o in outs)
    name = {KIND_Q4_0: "q4_0", KIND_Q8_0: "q8_0", KIND_Q4_K: "q4_k", KIND_Q5_K: "q5_k", KIND_Q6_K: "q6_k",
            KIND_Q4_1: "q4_1", KIND_Q5_0: "q5_0", KIND_Q5_1: "q5_1", KIND_Q2_K: "q2_k", KIND_Q3_K: "q3_k",
            KIND_Q8_1: "q8_1"}[kind]
    st = getattr(ctx.lib, f"hip_matmul_qkv_{name}")(ctx.device_ctx, C.byref(desc))
    assert st == ta.SUCCESS, ctx.last_error()
    tol = 1e-3 if dtype == np.float32 else 2e-3
    for o, r in zip(outs, ref):
        assert o.t.memory_location == ta.MEMORY_DEVICE and o.t.needs_sync
        got = ctx.to_host(o)
        assert_matmul_parity(got.astype(np.float32), r.astype(np.float32), tol=tol, what=f"qkv impl kind={kind}")
    first = [o.array.copy() for o in outs]
    # the same call as one bytecode instruction, kernel chosen by the query
    sel = ctx.query(ctx.qkv_signature(xt, wts[0], outs[0], bias=True))
    assert sel.supported and sel.op_index == {KIND_Q4_0: 12, KIND_Q8_0: 13, KIND_Q4_K: 14, KIND_Q6_K: 15, KIND_Q5_K: 22,
                                              KIND_Q4_1: 26, KIND_Q5_0: 30, KIND_Q5_1: 34, KIND_Q2_K: 38,
                                              KIND_Q3_K: 42, KIND_Q8_1: 46}[kind]
    for o in outs:
        o.array[...] = 0
        ctx.host_changed(o)
    prog = ta.Program()
    prog.qkv(sel.op_index, xt, *wts, *outs, bq=bts[0], bv=bts[2])
    assert ctx.execute(prog) == ta.SUCCESS, ctx.last_error()
    for o, f in zip(outs, first):
        assert np.array_equal(bits(ctx.to_host(o)), bits(f))
    for t in [xt] + wts + outs + [b for b in bts if b is not None]:
        ctx.host_freed(t)


def test_impl_qkv_errors(ctx, oracle):
    """Error codes in the order of cpu_matmul_qkv_validate_desc (matmul_qkv.c:1140-1146, 1230-1300)."""
    kind, M, K, N = KIND_Q4_K, 32, 256, 2
    ws = [oracle.quantize(kind, gaussian(930 + i, (M, K), 0.02)) for i in range(3)]
    x = gaussian(933, (N, K))
    fn = ctx.lib.hip_matmul_qkv_q4_k

    def build(x_=x, M_out=M, layout=ta.QKV_LAYOUT_SEPARATE, out_dtype=None, bias=None, rope=None, wk_kind=kind):
        xt, wts, outs, bts = _qkv_tensors(kind, ws, M, K, x_, [bias, None, None])
        if M_out != M or out_dtype is not None:
            outs = [ta.HostTensor.empty((x_.shape[0], M_out), out_dtype if out_dtype is not None else ta.DTYPE_F32)
                    for _ in range(3)]
        wts[1].t.quant_kind = wk_kind
        d = ta.QkvDesc()
        d.input, d.layout = xt.ptr, layout
        d.separate.wq, d.separate.wk, d.separate.wv = (w.ptr for w in wts)
        if bts[0] is not None:
            d.separate.bq = bts[0].ptr
        d.out_q, d.out_k, d.out_v = (o.ptr for o in outs)
        if rope is not None:
            d.rope_params = C.pointer(rope)
        keep = (xt, wts, outs, bts, rope)
        made.extend([xt] + list(wts) + list(outs) + [b for b in bts if b is not None])
        return d, keep

    made = []  # every tensor a call may have mirrored: released at the end like the core does on tensor destruction
    d, keep = build()
    assert fn(ctx.device_ctx, C.byref(d)) == ta.SUCCESS
    assert fn(ctx.device_ctx, None) == ta.INVALID_ARGUMENT
    d, keep = build(layout=ta.QKV_LAYOUT_FUSED)
    assert fn(ctx.device_ctx, C.byref(d)) == ta.NOT_IMPLEMENTED
    d, keep = build(layout=0)
    assert fn(ctx.device_ctx, C.byref(d)) == ta.INVALID_ARGUMENT
    d, keep = build(out_dtype=ta.DTYPE_F16)
    assert fn(ctx.device_ctx, C.byref(d)) == ta.UNSUPPORTED_DTYPE and "share dtype" in ctx.last_error()[1]
    d, keep = build(M_out=M + 1)
    assert fn(ctx.device_ctx, C.byref(d)) == ta.DIMENSION_MISMATCH and "output shape" in ctx.last_error()[1]
    d, keep = build(x_=gaussian(934, (N, K + 256)))
    assert fn(ctx.device_ctx, C.byref(d)) == ta.DIMENSION_MISMATCH and "input dimension" in ctx.last_error()[1]
    d, keep = build(bias=gaussian(935, (M,)).astype(np.float16))
    assert fn(ctx.device_ctx, C.byref(d)) == ta.UNSUPPORTED_DTYPE and "bias dtype" in ctx.last_error()[1]
    d, keep = build(bias=gaussian(936, (M + 1,)))
    assert fn(ctx.device_ctx, C.byref(d)) == ta.DIMENSION_MISMATCH
    d, keep = build(wk_kind=KIND_Q6_K)
    assert fn(ctx.device_ctx, C.byref(d)) == ta.NOT_IMPLEMENTED
    rope = ta.RopeParams()
    rope.theta, rope.freq_scale, rope.attn_factor, rope.apply_to_q = 10000.0, 1.0, 1.0, True
    d, keep = build(rope=rope)  # no positions tensor
    assert fn(ctx.device_ctx, C.byref(d)) == ta.INVALID_ARGUMENT and "positions" in ctx.last_error()[1]
    pos = ta.HostTensor.dense(np.zeros(N, np.int8))
    rope.positions = pos.ptr
    d, keep = build(rope=rope)
    assert fn(ctx.device_ctx, C.byref(d)) == ta.UNSUPPORTED_DTYPE
    pos1 = ta.HostTensor.dense(np.zeros(N - 1, np.int32))
    rope.positions = pos1.ptr
    d, keep = build(rope=rope)
    assert fn(ctx.device_ctx, C.byref(d)) == ta.DIMENSION_MISMATCH
    pos2 = ta.HostTensor.dense(np.arange(N, dtype=np.int32))
    rope.positions = pos2.ptr
    rope.scaling_type, rope.ext_factor, rope.freq_scale, rope.orig_ctx_len = 2, 1.0, 0.5, 4096
    rope.beta_fast, rope.beta_slow = 32.0, 1.0
    d, keep = build(rope=rope)  # the YaRN ramp is computed like any other scaling
    assert fn(ctx.device_ctx, C.byref(d)) == ta.SUCCESS, ctx.last_error()
    rope.apply_to_q = False  # parameters present but applied to neither q nor k: plain projection (matmul_qkv.c:812-814)
    rope.positions = None
    d, keep = build(rope=rope)
    assert fn(ctx.device_ctx, C.byref(d)) == ta.SUCCESS
    for t in made + [pos, pos1, pos2]:
        ctx.host_freed(t)


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_program_qkv_with_rotary_epilogue(ctx, oracle, dtype):
    """QKV_SHARED_INPUT with the ROPE epilogue as the graph emits it (graph_builder.cpp:384-394): rope parameters in
    the constant pool, positions as a tensor; the frequency table is mirrored once and reused by the second run."""
    from oracle.pyoracle import RopeParams as OracleRope

    kind, M, K, N = KIND_Q4_K, 256, 1024, 7
    ws = [oracle.quantize(kind, gaussian(940 + i, (M, K), 0.02)) for i in range(3)]
    x = gaussian(943, (N, K)).astype(dtype)
    biases = [gaussian(944 + i, (M,)).astype(dtype) for i in range(3)]
    positions = np.array([0, 1, 2, 3, 4, 500, 8000], np.int32)
    xt, wts, outs, bts = _qkv_tensors(kind, ws, M, K, x, biases)
    pt = ta.HostTensor.dense(positions)
    sel = ctx.query(ctx.qkv_signature(xt, wts[0], outs[0], bias=True, rope=True))
    assert sel.supported and sel.op_index == 14
    for rope_type in (0, 1):
        rp = ta.RopeParams()
        rp.positions = pt.ptr
        rp.scaling_type, rp.rope_type, rp.theta, rp.freq_scale, rp.ext_factor, rp.attn_factor = 0, rope_type, 500000.0, 1.0, 0.0, 1.0
        rp.beta_fast, rp.beta_slow, rp.orig_ctx_len, rp.head_dim, rp.apply_to_q, rp.apply_to_k = 32.0, 1.0, 0, 64, True, True
        ref = oracle.matmul_qkv(kind, *ws, x, M, bq=biases[0], bk=biases[1], bv=biases[2], positions=positions,
                                rope=OracleRope.default(theta=500000.0, head_dim=64, rope_type=rope_type))
        before = ctx.residency().uploads
        for run in range(2):
            prog = ta.Program()
            prog.qkv(sel.op_index, xt, *wts, *outs, bq=bts[0], bk=bts[1], bv=bts[2], rope=rp)
            assert ctx.execute(prog) == ta.SUCCESS, ctx.last_error()
            for o, r in zip(outs, ref):
                got = ctx.to_host(o).astype(np.float32)
                r32 = r.astype(np.float32)
                if dtype == np.float32:
                    assert_matmul_parity(got, r32, what=f"program qkv rope type={rope_type}")
                else:
                    assert np.max(np.abs(got - r32)) <= 1e-3 * np.abs(r32).max()
            if run == 0:
                first_uploads = ctx.residency().uploads - before
        # second run: nothing is uploaded again (weights, biases, positions and the frequency table stay resident)
        assert ctx.residency().uploads - before == first_uploads
    for t in [xt, pt] + wts + outs + bts:
        ctx.host_freed(t)


# ---------------------------------------------------------------- embedding gather
@pytest.mark.parametrize("kind", [KIND_Q4_0, KIND_Q5_0, KIND_Q5_1, KIND_Q8_0, KIND_Q8_1, KIND_Q2_K, KIND_Q3_K, KIND_Q4_K, KIND_Q5_K,
                                  KIND_Q6_K])
def test_impl_and_program_embedding_gather(ctx, oracle, kind):
    """marmot_embedding_gather on a quantized table: the impl function with a descriptor and the EMBEDDING bytecode
    schema, ids of rank 2 (flattened), float32 bit-exact and float16 with scale; the table stays resident."""
    from tests.util import random_valid_blocks

    print(f"backend embedding kind={kind}", flush=True)
    rng = np.random.default_rng(960 + kind)
    vocab, dim = 300, 1024
    table = random_valid_blocks(rng, kind, vocab, dim)
    ids = rng.integers(0, vocab, (3, 5)).astype(np.int64)
    ids[0, 1] = 11
    tt = ta.HostTensor.quantized(table, (vocab, dim), kind)
    it = ta.HostTensor.dense(ids)
    ot = ta.HostTensor.empty((3, 5, dim), ta.DTYPE_F32)
    desc = ta.EmbeddingGatherDesc()
    desc.weights, desc.token_ids, desc.out = tt.ptr, it.ptr, ot.ptr
    desc.dtype_out, desc.scale, desc.padding_id, desc.bounds_check = ta.DTYPE_F32, 1.0, 11, True
    assert ctx.lib.hip_embedding_gather(ctx.device_ctx, C.byref(desc)) == ta.SUCCESS, ctx.last_error()
    assert ot.t.memory_location == ta.MEMORY_DEVICE and ot.t.needs_sync
    ref = oracle.embedding_gather(kind, table, vocab, dim, ids, padding_id=11)
    assert np.array_equal(bits(ctx.to_host(ot)), bits(ref)) and not ot.array[0, 1].any()

    o16 = ta.HostTensor.empty((15, dim), ta.DTYPE_F16)
    i32 = ta.HostTensor.dense(ids.astype(np.int32).reshape(-1))
    sel = ctx.query(ctx.embedding_signature(tt, i32, o16))
    assert sel.supported and sel.op_index == {KIND_Q4_0: 16, KIND_Q8_0: 17, KIND_Q4_K: 18, KIND_Q6_K: 19, KIND_Q5_K: 23,
                                              KIND_Q5_0: 31, KIND_Q5_1: 35, KIND_Q2_K: 39, KIND_Q3_K: 43,
                                              KIND_Q8_1: 47}[kind]
    before = ctx.residency().uploads
    prog = ta.Program()
    prog.embedding(sel.op_index, tt, i32, o16, scale=0.25, padding_id=-1, bounds_check=False)
    assert ctx.execute(prog) == ta.SUCCESS, ctx.last_error()
    ref16 = oracle.embedding_gather(kind, table, vocab, dim, ids.reshape(-1), out_dtype=np.float16, scale=0.25)
    assert np.array_equal(ctx.to_host(o16).view(np.uint16), ref16.view(np.uint16))
    # only the ids travel: the table was not uploaded again. (Counted in uploads, not bytes: a fresh host array may
    # overlap the mirror of an array an earlier test released without telling the backend, and is then uploaded
    # together with it.)
    assert ctx.residency().uploads - before == 1
    for t in (tt, it, ot, o16, i32):
        ctx.host_freed(t)


def test_embedding_gather_errors(ctx):
    from tests.util import random_valid_blocks

    vocab, dim = 8, 256
    table = random_valid_blocks(np.random.default_rng(970), KIND_Q4_K, vocab, dim)
    tt = ta.HostTensor.quantized(table, (vocab, dim), KIND_Q4_K)
    ids = ta.HostTensor.dense(np.array([1, 8, 2], np.int32))
    out = ta.HostTensor.empty((3, dim), ta.DTYPE_F32)

    def call(weights=tt, token_ids=ids, o=out, bounds=True):
        d = ta.EmbeddingGatherDesc()
        d.weights, d.token_ids, d.out = weights.ptr, token_ids.ptr, o.ptr
        d.dtype_out, d.scale, d.padding_id, d.bounds_check = o.t.dtype, 1.0, -1, bounds
        return ctx.lib.hip_embedding_gather(ctx.device_ctx, C.byref(d))

    # embedding_scalar.c:556-559: an id outside the table with the bounds check on
    assert call() == ta.INVALID_ARGUMENT and "out of range" in ctx.last_error()[1]
    assert call(bounds=False) == ta.SUCCESS and not ctx.to_host(out)[1].any()
    tmp = {
        "float_ids": ta.HostTensor.dense(np.zeros(3, np.float32)),
        "int_out": ta.HostTensor.empty((3, dim), ta.DTYPE_I32),
        "short_out": ta.HostTensor.empty((2, dim), ta.DTYPE_F32),
        "q8_k": ta.HostTensor.quantized(table, (vocab, dim), KIND_Q8_K),
        "q4_1": ta.HostTensor.quantized(table, (vocab, dim), KIND_Q4_1),
        "flat": ta.HostTensor.quantized(table, (vocab * dim,), KIND_Q4_K),
        "no_ids": ta.HostTensor(np.zeros(1, np.int32), (0,), ta.DTYPE_I32),
        "no_out": ta.HostTensor(np.zeros(1, np.float32), (0, dim), ta.DTYPE_F32),
    }
    assert call(token_ids=tmp["float_ids"]) == ta.UNSUPPORTED_DTYPE
    assert call(o=tmp["int_out"]) == ta.UNSUPPORTED_DTYPE
    assert call(o=tmp["short_out"]) == ta.DIMENSION_MISMATCH
    assert call(weights=tmp["q8_k"]) == ta.NOT_IMPLEMENTED
    # Q4_1 tables are taken (the embedding path's interleaved nibble order): the Q4_K bytes read as Q4_1 blocks are a
    # table of another width, so the shapes disagree here
    assert call(weights=tmp["q4_1"]) in (ta.DIMENSION_MISMATCH, ta.INVALID_ARGUMENT)
    assert call(weights=tmp["flat"]) == ta.DIMENSION_MISMATCH
    assert call(token_ids=tmp["no_ids"], o=tmp["no_out"]) == ta.SUCCESS
    for t in [tt, ids, out] + list(tmp.values()):
        ctx.host_freed(t)


# ---------------------------------------------------------------- ops between the linears
def test_impl_and_program_float_ops(ctx, oracle):
    """hip_rmsnorm_impl / hip_rmsnorm_gemma_impl (rank 3, residual), hip_swiglu_f32 / hip_geglu_f32 (contiguous and
    row-strided), hip_add_f32, their queries and bytecode ops, against the oracle."""
    x = gaussian(980, (2, 5, 512))
    r = gaussian(981, (2, 5, 512))
    w = gaussian(982, (512,), 0.5) + np.float32(1.0)
    xt, rt, wt = ta.HostTensor.dense(x), ta.HostTensor.dense(r), ta.HostTensor.dense(w)
    ot = ta.HostTensor.empty((2, 5, 512), ta.DTYPE_F32)
    for fn, off, op, bc in ((ctx.lib.hip_rmsnorm_impl, 0.0, ta.OP_RMS_NORM, ta.BC_OP_RMS_NORM_F32),
                            (ctx.lib.hip_rmsnorm_gemma_impl, 1.0, ta.OP_RMS_NORM_GEMMA, ta.BC_OP_RMS_NORM_GEMMA_F32)):
        desc = ta.RmsNormDesc(xt.ptr, rt.ptr, wt.ptr, ot.ptr, 1e-6)
        assert fn(ctx.device_ctx, C.byref(desc)) == ta.SUCCESS, ctx.last_error()
        ref = oracle.rms_norm(x.reshape(10, 512), w, residual=r.reshape(10, 512), eps=1e-6, weight_offset=off)
        assert np.allclose(ctx.to_host(ot).reshape(10, 512), ref, rtol=1e-5, atol=1e-8)
        sel = ctx.query(ctx.float_op_signature(op))
        assert sel.supported and sel.op_index == bc
        assert not ctx.query(ctx.float_op_signature(op, ta.DTYPE_F16)).supported
        prog = ta.Program()
        prog.rms_norm(bc, xt, wt, None, ot, 1e-5)
        assert ctx.execute(prog) == ta.SUCCESS, ctx.last_error()
        ref = oracle.rms_norm(x.reshape(10, 512), w, eps=1e-5, weight_offset=off)
        assert np.allclose(ctx.to_host(ot).reshape(10, 512), ref, rtol=1e-5, atol=1e-8)
    bad = ta.HostTensor.dense(gaussian(983, (500,)))
    desc = ta.RmsNormDesc(xt.ptr, None, bad.ptr, ot.ptr, 1e-6)
    assert ctx.lib.hip_rmsnorm_impl(ctx.device_ctx, C.byref(desc)) == ta.DIMENSION_MISMATCH

    g, u = gaussian(984, (6, 300), 2.0), gaussian(985, (6, 300))
    gt, ut, yt = ta.HostTensor.dense(g), ta.HostTensor.dense(u), ta.HostTensor.empty((6, 300), ta.DTYPE_F32)
    for fn, geglu, op, bc in ((ctx.lib.hip_swiglu_f32, False, ta.OP_SWIGLU, ta.BC_OP_SWIGLU_F32),
                              (ctx.lib.hip_geglu_f32, True, ta.OP_GEGLU, ta.BC_OP_GEGLU_F32)):
        assert fn(ctx.device_ctx, gt.ptr, ut.ptr, yt.ptr) == ta.SUCCESS, ctx.last_error()
        assert np.allclose(ctx.to_host(yt), oracle.glu(g, u, geglu=geglu), rtol=1e-5, atol=1e-7)
        sel = ctx.query(ctx.float_op_signature(op))
        assert sel.supported and sel.op_index == bc
        prog = ta.Program()
        prog.binary(bc, ut, gt, yt)  # operands swapped: act(up) * gate
        assert ctx.execute(prog) == ta.SUCCESS, ctx.last_error()
        assert np.allclose(ctx.to_host(yt), oracle.glu(u, g, geglu=geglu), rtol=1e-5, atol=1e-7)
    # row-strided: gate and up are the two halves of one [rows, 2 * cols] projection output
    both = gaussian(986, (4, 512), 2.0)
    whole = ta.HostTensor.dense(both)
    halves = []
    for h in range(2):
        view = ta.HostTensor.dense(both)  # a fresh descriptor over the same memory, then narrowed to one half
        view.array = whole.array
        view.t.data = whole.t.data + h * 256 * 4
        view.t.shape.shape[1] = 256
        view.t.shape.strides[0] = 512
        halves.append(view)
    yo = ta.HostTensor.empty((4, 256), ta.DTYPE_F32)
    assert ctx.lib.hip_swiglu_f32(ctx.device_ctx, halves[0].ptr, halves[1].ptr, yo.ptr) == ta.SUCCESS, ctx.last_error()
    assert np.allclose(ctx.to_host(yo), oracle.glu(both[:, :256], both[:, 256:]), rtol=1e-5, atol=1e-7)

    a, b_ = gaussian(987, (3, 7, 11)), gaussian(988, (3, 7, 11))
    at, bt, st_ = ta.HostTensor.dense(a), ta.HostTensor.dense(b_), ta.HostTensor.empty((3, 7, 11), ta.DTYPE_F32)
    assert ctx.lib.hip_add_f32(ctx.device_ctx, at.ptr, bt.ptr, st_.ptr) == ta.SUCCESS
    assert np.array_equal(ctx.to_host(st_), a + b_)
    sel = ctx.query(ctx.float_op_signature(ta.OP_ADD))
    assert sel.supported and sel.op_index == ta.BC_OP_ADD_F32
    for t in (xt, rt, wt, ot, bad, gt, ut, yt, whole, yo, at, bt, st_):
        ctx.host_freed(t)


def _rope_params(pos_t, **kw):
    rp = ta.RopeParams()
    rp.positions = pos_t.ptr if pos_t is not None else None
    rp.scaling_type, rp.rope_type, rp.theta, rp.freq_scale, rp.ext_factor, rp.attn_factor = 0, 0, 10000.0, 1.0, 0.0, 1.0
    rp.beta_fast, rp.beta_slow, rp.orig_ctx_len, rp.head_dim = 32.0, 1.0, 0, 0
    for k, v in kw.items():
        setattr(rp, k, v)
    return rp


def test_impl_and_program_rope(ctx, oracle):
    """hip_rope (rank 3, FLOAT32 and FLOAT16, NORM and NEOX, the three position types, in place, row-strided views),
    its query and bytecode op with and without a positions register, and cpu_rope's error order."""
    from oracle.pyoracle import RopeParams as OracleRope
    from tests.test_gpu_ops import rope_close

    x = gaussian(1300, (2, 9, 128))
    pos = (np.arange(18, dtype=np.int32).reshape(2, 9) * 113) % 4096
    for np_dt, dt in ((np.float32, ta.DTYPE_F32), (np.float16, ta.DTYPE_F16)):
        xv = x.astype(np_dt)
        xt, ot = ta.HostTensor.dense(xv), ta.HostTensor.empty((2, 9, 128), dt)
        for p in (pos, pos.astype(np.int64), pos.astype(np.float32) + np.float32(0.25)):
            pt = ta.HostTensor.dense(p)
            for rope_type in (0, 1):
                rp = _rope_params(pt, rope_type=rope_type, theta=500000.0)
                assert ctx.lib.hip_rope(ctx.device_ctx, xt.ptr, C.byref(rp), ot.ptr) == ta.SUCCESS, ctx.last_error()
                st, ref = oracle.rope(xv, p, OracleRope.default(theta=500000.0, rope_type=rope_type))
                rope_close(ctx.to_host(ot), ref, xv, f"hip_rope {np_dt.__name__} {p.dtype} type {rope_type}")
            ctx.host_freed(pt)
        sel = ctx.query(ctx.float_op_signature(ta.OP_ROPE, dt))
        assert sel.supported and sel.op_index == ta.BC_OP_ROPE
        # the program: parameters in the constant pool; a positions register replaces the tensor they name
        pt, pt2 = ta.HostTensor.dense(pos), ta.HostTensor.dense(pos + 5)
        rp = _rope_params(pt, theta=10000.0, scaling_type=1, freq_scale=0.5, attn_factor=1.25)
        oracle_rp = OracleRope.default(theta=10000.0, scaling_type=1, freq_scale=0.5, attn_factor=1.25)
        prog = ta.Program()
        prog.rope(sel.op_index, xt, ot, rp)
        assert ctx.execute(prog) == ta.SUCCESS, ctx.last_error()
        rope_close(ctx.to_host(ot), oracle.rope(xv, pos, oracle_rp)[1], xv, "program rope")
        prog = ta.Program()
        prog.rope(sel.op_index, xt, ot, rp, positions=pt2, n_past=5, n_rot=128)
        assert ctx.execute(prog) == ta.SUCCESS, ctx.last_error()
        rope_close(ctx.to_host(ot), oracle.rope(xv, pos + 5, oracle_rp)[1], xv, "program rope, positions register")
        prog = ta.Program()
        prog.rope(sel.op_index, xt, ot, None, positions=pt2)
        assert ctx.execute(prog) == ta.INVALID_ARGUMENT  # a positions register without parameters
        # in place
        it = ta.HostTensor.dense(xv.copy())
        rp = _rope_params(pt)
        assert ctx.lib.hip_rope(ctx.device_ctx, it.ptr, C.byref(rp), it.ptr) == ta.SUCCESS, ctx.last_error()
        rope_close(ctx.to_host(it), oracle.rope(xv, pos, OracleRope.default())[1], xv, "in place")
        for t in (xt, ot, pt, pt2, it):
            ctx.host_freed(t)

    # row-strided views: q is the first 128 columns of a [rows, 384] projection output, rotated into the first 128
    # columns of another; the other columns of the output keep what the host wrote there
    rows = 12
    both, dst = gaussian(1301, (rows, 384)), gaussian(1302, (rows, 384))
    whole_in, whole_out = ta.HostTensor.dense(both), ta.HostTensor.dense(dst)
    views = []
    for whole in (whole_in, whole_out):
        v = ta.HostTensor.dense(both)
        v.array = whole.array
        v.t.data = whole.t.data
        v.t.shape.shape[1] = 128
        v.t.shape.strides[0] = 384
        views.append(v)
    p = np.arange(rows, dtype=np.int32) * 7
    pt = ta.HostTensor.dense(p)
    rp = _rope_params(pt, rope_type=1)
    assert ctx.lib.hip_rope(ctx.device_ctx, views[0].ptr, C.byref(rp), views[1].ptr) == ta.SUCCESS, ctx.last_error()
    got = ctx.to_host(views[1]).reshape(rows, 384)
    rope_close(got[:, :128], oracle.rope(both[:, :128], p, OracleRope.default(rope_type=1))[1], both, "strided rope")
    assert np.array_equal(got[:, 128:], dst[:, 128:])
    # the same for a gated product written into a row-strided half
    g, u = gaussian(1303, (rows, 128)), gaussian(1304, (rows, 128))
    dst2 = gaussian(1305, (rows, 384))
    whole2 = ta.HostTensor.dense(dst2)
    v2 = ta.HostTensor.dense(dst2)
    v2.array = whole2.array
    v2.t.data = whole2.t.data
    v2.t.shape.shape[1] = 128
    v2.t.shape.strides[0] = 384
    gt, ut = ta.HostTensor.dense(g), ta.HostTensor.dense(u)
    # the gated products want all three operands row-strided or all contiguous: narrow views of wider buffers
    gv, uv = [], []
    for src, keep in ((g, gv), (u, uv)):
        wide = ta.HostTensor.dense(np.concatenate([src, np.zeros((rows, 64), np.float32)], axis=1))
        wide.t.shape.shape[1] = 128
        keep.append(wide)
    assert ctx.lib.hip_swiglu_f32(ctx.device_ctx, gv[0].ptr, uv[0].ptr, v2.ptr) == ta.SUCCESS, ctx.last_error()
    got2 = ctx.to_host(v2).reshape(rows, 384)
    assert np.allclose(got2[:, :128], oracle.glu(g, u), rtol=1e-5, atol=1e-7)
    assert np.array_equal(got2[:, 128:], dst2[:, 128:])

    # errors, in cpu_rope's order (rope_dispatch.c:18-88, 145-188)
    xt, ot = ta.HostTensor.dense(x), ta.HostTensor.empty((2, 9, 128), ta.DTYPE_F32)
    good = _rope_params(pt)
    full = ta.HostTensor.dense(pos)
    rp = _rope_params(full)
    lib, dc = ctx.lib, ctx.device_ctx
    assert lib.hip_rope(dc, xt.ptr, None, ot.ptr) == ta.INVALID_ARGUMENT
    assert lib.hip_rope(dc, xt.ptr, C.byref(_rope_params(None)), ot.ptr) == ta.INVALID_ARGUMENT
    assert lib.hip_rope(dc, None, C.byref(rp), ot.ptr) == ta.INVALID_ARGUMENT
    o16 = ta.HostTensor.empty((2, 9, 128), ta.DTYPE_F16)
    assert lib.hip_rope(dc, xt.ptr, C.byref(rp), o16.ptr) == ta.UNSUPPORTED_DTYPE       # types differ
    i32 = ta.HostTensor.dense(np.zeros((2, 9, 128), np.int32))
    assert lib.hip_rope(dc, i32.ptr, C.byref(rp), i32.ptr) == ta.UNSUPPORTED_DTYPE
    v1 = ta.HostTensor.dense(np.zeros(128, np.float32))
    assert lib.hip_rope(dc, v1.ptr, C.byref(rp), v1.ptr) == ta.DIMENSION_MISMATCH       # rank 1
    odd = ta.HostTensor.dense(np.zeros((18, 7), np.float32))
    assert lib.hip_rope(dc, odd.ptr, C.byref(rp), odd.ptr) == ta.DIMENSION_MISMATCH     # odd dimension
    empty = ta.HostTensor.dense(np.zeros((0, 8), np.float32))
    assert lib.hip_rope(dc, empty.ptr, C.byref(rp), empty.ptr) == ta.INVALID_ARGUMENT
    assert lib.hip_rope(dc, xt.ptr, C.byref(good), ot.ptr) == ta.DIMENSION_MISMATCH     # 12 positions for 18 rows
    o2 = ta.HostTensor.empty((2, 9, 64), ta.DTYPE_F32)
    assert lib.hip_rope(dc, xt.ptr, C.byref(rp), o2.ptr) == ta.DIMENSION_MISMATCH       # output shape
    p16 = ta.HostTensor.dense(pos.astype(np.float16))
    assert lib.hip_rope(dc, xt.ptr, C.byref(_rope_params(p16)), ot.ptr) == ta.UNSUPPORTED_DTYPE
    tr = ta.HostTensor.dense(x)
    tr.t.shape.strides[2], tr.t.shape.strides[1] = 2, 256
    assert lib.hip_rope(dc, tr.ptr, C.byref(rp), ot.ptr) == ta.NOT_IMPLEMENTED          # inner stride
    short = ta.HostTensor.dense(x)
    short.t.shape.strides[1] = 64
    assert lib.hip_rope(dc, short.ptr, C.byref(rp), ot.ptr) == ta.DIMENSION_MISMATCH    # row stride < dim
    f64 = ta.HostTensor.dense(np.zeros((2, 9, 128), np.float32))
    f64.t.dtype = 10  # MARMOT_DTYPE_FLOAT64: the reference rotates it, this backend declines
    assert lib.hip_rope(dc, f64.ptr, C.byref(rp), f64.ptr) == ta.NOT_IMPLEMENTED
    assert not ctx.query(ctx.float_op_signature(ta.OP_ROPE, 10)).supported
    assert lib.hip_rope(dc, xt.ptr, C.byref(rp), ot.ptr) == ta.SUCCESS
    for t in (whole_in, whole_out, pt, whole2, gt, ut, gv[0], uv[0], xt, ot, full, o16, i32, v1, odd, empty, o2, p16,
              f64):
        ctx.host_freed(t)


def test_program_norm_feeds_linears_without_quantization_launches(ctx, oracle):
    """A decoder layer's feed-forward half at 16 tokens as one bytecode program: rms_norm -> gate, up (Q4_K) -> swiglu
    -> down (Q6_K) -> residual add. The normalization leaves its rows packed, gate and up both find them (no packing
    launch of their own); the gated product is packed once by the down projection. Results against the oracle's
    chain (bound against the output scale, as for every re-quantizing chain)."""
    from tests.util import assert_moe_parity

    T, H, F = 16, 1024, 2816
    x = gaussian(990, (T, H))
    w_norm = gaussian(991, (H,), 0.3) + np.float32(1.0)
    gate = oracle.quantize(KIND_Q4_K, gaussian(992, (F, H), 0.03))
    up = oracle.quantize(KIND_Q4_K, gaussian(993, (F, H), 0.03))
    down = oracle.quantize(KIND_Q6_K, gaussian(994, (H, F), 0.03))
    xt, wn = ta.HostTensor.dense(x), ta.HostTensor.dense(w_norm)
    gw, uw = ta.HostTensor.quantized(gate, (F, H), KIND_Q4_K), ta.HostTensor.quantized(up, (F, H), KIND_Q4_K)
    dw = ta.HostTensor.quantized(down, (H, F), KIND_Q6_K)
    h, g, u, a = (ta.HostTensor.empty(s, ta.DTYPE_F32) for s in ((T, H), (T, F), (T, F), (T, F)))
    d, y = ta.HostTensor.empty((T, H), ta.DTYPE_F32), ta.HostTensor.empty((T, H), ta.DTYPE_F32)
    mm = {KIND_Q4_K: 3, KIND_Q6_K: 4}
    prog = ta.Program()
    prog.rms_norm(ta.BC_OP_RMS_NORM_F32, xt, wn, None, h, 1e-5)
    prog.matmul(mm[KIND_Q4_K], h, gw, g)
    prog.matmul(mm[KIND_Q4_K], h, uw, u)
    prog.binary(ta.BC_OP_SWIGLU_F32, g, u, a)
    prog.matmul(mm[KIND_Q6_K], a, dw, d)
    prog.binary(ta.BC_OP_ADD_F32, xt, d, y)
    ref_h = oracle.rms_norm(x, w_norm, eps=1e-5)
    ref_a = oracle.glu(oracle.matmul(KIND_Q4_K, gate, ref_h, F, threads=8), oracle.matmul(KIND_Q4_K, up, ref_h, F, threads=8))
    ref_d = oracle.matmul(KIND_Q6_K, down, ref_a, H, threads=8)
    for run in range(2):
        before = ctx.residency()
        packs0, hits0 = before.activation_packs, before.activation_pack_hits
        assert ctx.execute(prog) == ta.SUCCESS, ctx.last_error()
        after = ctx.residency()
        # two packed copies per run (the normalization's output, the gated product), three linears that found one
        assert after.activation_packs - packs0 == 2, run
        assert after.activation_pack_hits - hits0 == 2, run   # gate and up; down packed its own input
        assert_moe_parity(ctx.to_host(d), ref_d, what=f"ffn chain run {run}")
        assert np.allclose(ctx.to_host(y), x + ctx.to_host(d), rtol=0, atol=0)
        assert np.allclose(ctx.to_host(h), ref_h, rtol=1e-5, atol=1e-8)
    # writing the normalized tensor from the host ends its packed copy: the next linear packs the new contents
    h.array[:] = gaussian(995, (T, H))
    ctx.ops.memcpy_to_device(ctx.device_ctx, h.t.data, h.t.data, h.array.nbytes)
    one = ta.Program()
    one.matmul(mm[KIND_Q4_K], h, gw, g)
    packs0 = ctx.residency().activation_packs
    assert ctx.execute(one) == ta.SUCCESS, ctx.last_error()
    assert ctx.residency().activation_packs - packs0 == 1
    from tests.util import assert_matmul_parity
    assert_matmul_parity(ctx.to_host(g), oracle.matmul(KIND_Q4_K, gate, h.array, F, threads=8), what="after host write")
    for t in (xt, wn, gw, uw, dw, h, g, u, a, d, y):
        ctx.host_freed(t)


# ---------------------------------------------------------------- paged attention
def _attention_tensors(ctx, case):
    """Host tensors of a paged-attention case: q / k_new / v_new as views of one buffer (a fused projection's output),
    bfloat16 as uint16 bits with the type said explicitly. Like memory fresh from marmot's allocator, no mirror of a
    previous owner of these addresses survives (the core notifies the backend when it frees host memory)."""
    from tests.attention_cases import to_storage

    act_dt = {"f32": None, "f16": None, "bf16": ta.DTYPE_BF16}[case["act"]]
    kv_dt = {"f32": None, "f16": None, "bf16": ta.DTYPE_BF16, "fp8": ta.DTYPE_F8_E4M3}[case["kv"]]
    T, hq, d = case["q"].shape
    hkv = case["k_new"].shape[1]
    fused = np.zeros((T, hq + 2 * hkv, d), dtype=case["q"].dtype)
    fused[:, :hq], fused[:, hq:hq + hkv], fused[:, hq + hkv:] = case["q"], case["k_new"], case["v_new"]
    t = {
        "fused": fused,
        "token_meta": ta.HostTensor.dense(case["token_meta"]),
        "q": ta.HostTensor.strided(fused[:, :hq], act_dt),
        "k_new": ta.HostTensor.strided(fused[:, hq:hq + hkv], act_dt),
        "v_new": ta.HostTensor.strided(fused[:, hq + hkv:], act_dt),
        "kv_k": ta.HostTensor.strided(case["kv_k"].copy(), kv_dt),
        "kv_v": ta.HostTensor.strided(case["kv_v"].copy(), kv_dt),
        "block_table": ta.HostTensor.dense(case["block_table"]),
        "out": ta.HostTensor.strided(np.zeros((T, hq, d), dtype=case["q"].dtype), act_dt),
    }
    if case["kv"] == "fp8":  # FLOAT32 scales [blocks, layers, kv heads], handed over through the descriptor's pnext
        t["k_scale"] = ta.HostTensor.dense(case["k_scale"].copy())
        t["v_scale"] = ta.HostTensor.dense(case["v_scale"].copy())
    for name, x in t.items():
        if name != "fused":
            ctx.host_range_freed(x)
    desc = ta.PagedAttentionDesc.default()
    desc.token_count, desc.layer_idx, desc.scale = T, case["layer_idx"], case["scale"]
    desc.num_q_heads, desc.num_kv_heads, desc.head_dim, desc.block_size = hq, hkv, d, case["block_size"]
    for name in ("token_meta", "q", "k_new", "v_new", "kv_k", "kv_v", "block_table", "out"):
        setattr(desc, name, t[name].ptr)
    return t, desc


@pytest.mark.parametrize("act,kv", [("f32", "f16"), ("f16", "f16"), ("bf16", "bf16"), ("f32", "f32")])
def test_impl_and_program_paged_attention(ctx, oracle, act, kv):
    """hip_paged_attention_impl, its kernel query and its bytecode op against the oracle: caches bit for bit, output
    within fp32 summation noise and one rounding of the output type; a second call (decode step) on the caches the
    first one left on the device."""
    from tests.attention_cases import TOLERANCE, make_case, to_f32

    case = make_case(70, [(45, 1), (0, 12), (90, 3)], num_q_heads=8, num_kv_heads=2, head_dim=128, block_size=16,
                     act=act, kv=kv)
    ref_k, ref_v = case["kv_k"].copy(), case["kv_v"].copy()
    st, ref = oracle.paged_attention(case["token_meta"], case["q"], case["k_new"], case["v_new"], ref_k, ref_v,
                                     case["block_table"], case["layer_idx"], case["scale"], act_bf16=act == "bf16",
                                     kv_bf16=kv == "bf16")
    assert st == 0
    tol = TOLERANCE[act] * np.abs(to_f32(ref_v, kv)).max()

    def close(got):
        return np.max(np.abs(to_f32(got, act).astype(np.float64) - to_f32(ref, act).astype(np.float64))) <= tol

    t, desc = _attention_tensors(ctx, case)
    assert ctx.lib.hip_paged_attention_impl(ctx.device_ctx, C.byref(desc)) == ta.SUCCESS, ctx.last_error()
    assert close(ctx.to_host(t["out"]))
    assert np.array_equal(ctx.to_host(t["kv_k"]).view(np.uint8), ref_k.view(np.uint8))
    assert np.array_equal(ctx.to_host(t["kv_v"]).view(np.uint8), ref_v.view(np.uint8))
    # the same call as a bytecode op on fresh tensors
    sig = ta.OpSignature()
    sig.op_id, sig.accum_dtype = ta.OP_PAGED_ATTENTION, ta.DTYPE_F32
    sig.input_dtype = sig.output_dtype = t["q"].t.dtype
    sig.weight_dtype = t["kv_k"].t.dtype
    sel = ctx.query(sig)
    assert sel.supported and sel.op_index == ta.BC_OP_PAGED_ATTENTION
    t2, d2 = _attention_tensors(ctx, case)
    p = ta.Program()
    p.paged_attention(sel.op_index, t2["token_meta"], t2["q"], t2["k_new"], t2["v_new"], t2["kv_k"], t2["kv_v"],
                      t2["block_table"], t2["out"], d2.token_count, d2.layer_idx, d2.num_q_heads, d2.num_kv_heads,
                      d2.head_dim, d2.block_size, d2.scale)
    assert ctx.execute(p) == ta.SUCCESS, ctx.last_error()
    assert np.array_equal(ctx.to_host(t2["out"]).view(np.uint8), ctx.to_host(t["out"]).view(np.uint8))
    assert np.array_equal(ctx.to_host(t2["kv_k"]).view(np.uint8), ref_k.view(np.uint8))
    # a decode step on top: one more token per sequence, the caches stay on the device between the calls
    step = make_case(71, [(46, 1), (12, 1), (93, 1)], num_q_heads=8, num_kv_heads=2, head_dim=128, block_size=16,
                     act=act, kv=kv)
    # same block table and cache as after the first call; only the new tokens' metadata and rows differ
    bs = case["block_size"]
    slots = sorted(set(int(s) for s in case["token_meta"][:, 0]))
    last = {s: int(case["token_meta"][case["token_meta"][:, 0] == s, 1].max()) for s in slots}
    meta = np.array([[s, last[s] + 1, int(case["block_table"][s, (last[s] + 1) // bs]) * bs + (last[s] + 1) % bs, 0]
                     for s in slots], dtype=np.uint32)
    nxt = dict(case, token_meta=meta, q=step["q"][:3], k_new=step["k_new"][:3], v_new=step["v_new"][:3], kv_k=ref_k,
               kv_v=ref_v)
    st, ref2 = oracle.paged_attention(meta, nxt["q"], nxt["k_new"], nxt["v_new"], ref_k, ref_v, case["block_table"],
                                      case["layer_idx"], case["scale"], act_bf16=act == "bf16", kv_bf16=kv == "bf16")
    assert st == 0
    t3, d3 = _attention_tensors(ctx, nxt)
    d3.kv_k, d3.kv_v = t["kv_k"].ptr, t["kv_v"].ptr  # the tensors the first call updated
    assert ctx.lib.hip_paged_attention_impl(ctx.device_ctx, C.byref(d3)) == ta.SUCCESS, ctx.last_error()
    got2 = ctx.to_host(t3["out"])
    assert np.max(np.abs(to_f32(got2, act).astype(np.float64) - to_f32(ref2, act).astype(np.float64))) <= tol
    assert np.array_equal(ctx.to_host(t["kv_k"]).view(np.uint8), ref_k.view(np.uint8))
    for group in (t, t2, t3):
        for name, x in group.items():
            if name != "fused":
                ctx.host_freed(x)


def test_impl_and_program_paged_attention_fp8_cache(ctx, oracle):
    """The FLOAT8_E4M3 cache through hip_paged_attention_impl (scale tensors in the descriptor's extension) and through
    the bytecode op (scale tensors as registers): a prompt call that fills an empty cache, then a louder decode step on
    the cache and scales the first call left on the device. Cache bytes and scales bit for bit against the oracle."""
    from tests.attention_cases import TOLERANCE
    from tests.test_gpu_attention import _fp8_case, _next_step

    case = _fp8_case(90, [(0, 21), (0, 9), (0, 40)], room=1, num_q_heads=8, num_kv_heads=2, head_dim=64, block_size=16)
    case["kv"] = "fp8"

    def reference(c):
        state = {n: c[n].copy() for n in ("kv_k", "kv_v", "k_scale", "v_scale")}
        st, ref = oracle.paged_attention(c["token_meta"], c["q"], c["k_new"], c["v_new"], state["kv_k"], state["kv_v"],
                                         c["block_table"], c["layer_idx"], c["scale"], kv_k_scale=state["k_scale"],
                                         kv_v_scale=state["v_scale"])
        assert st == 0
        return ref, state

    def same_state(t, state):
        return all(np.array_equal(ctx.to_host(t[n]).view(np.uint8), state[n].view(np.uint8))
                   for n in ("kv_k", "kv_v", "k_scale", "v_scale"))

    ref, state = reference(case)
    tol = TOLERANCE["f32"] * 240.0 * max(state["v_scale"].max(), 1e-30)
    t, desc = _attention_tensors(ctx, case)
    ext = ta.PagedAttentionKvScaleExt(C.sizeof(ta.PagedAttentionKvScaleExt), 1, t["k_scale"].ptr, t["v_scale"].ptr)
    desc.pnext = C.addressof(ext)
    assert ctx.lib.hip_paged_attention_impl(ctx.device_ctx, C.byref(desc)) == ta.SUCCESS, ctx.last_error()
    assert np.max(np.abs(ctx.to_host(t["out"]).astype(np.float64) - ref)) <= tol
    assert same_state(t, state)
    # the same call as a bytecode op on fresh tensors
    sig = ta.OpSignature()
    sig.op_id, sig.accum_dtype = ta.OP_PAGED_ATTENTION, ta.DTYPE_F32
    sig.input_dtype = sig.output_dtype = ta.DTYPE_F32
    sig.weight_dtype = ta.DTYPE_F8_E4M3
    sel = ctx.query(sig)
    assert sel.supported and sel.op_index == ta.BC_OP_PAGED_ATTENTION
    t2, d2 = _attention_tensors(ctx, case)
    p = ta.Program()
    p.paged_attention(sel.op_index, t2["token_meta"], t2["q"], t2["k_new"], t2["v_new"], t2["kv_k"], t2["kv_v"],
                      t2["block_table"], t2["out"], d2.token_count, d2.layer_idx, d2.num_q_heads, d2.num_kv_heads,
                      d2.head_dim, d2.block_size, d2.scale, kv_k_scale=t2["k_scale"], kv_v_scale=t2["v_scale"])
    assert ctx.execute(p) == ta.SUCCESS, ctx.last_error()
    assert np.array_equal(ctx.to_host(t2["out"]).view(np.uint8), ctx.to_host(t["out"]).view(np.uint8))
    assert same_state(t2, state)
    # a decode step, sequence 0 four times louder: its block's scale grows and its rows are re-encoded on the device
    step = _next_step(dict(case, **state), state, 91, [4.0, 0.25, 1.0])
    ref2, state2 = reference(step)
    assert not np.array_equal(state2["k_scale"], state["k_scale"])
    t3, d3 = _attention_tensors(ctx, step)
    d3.kv_k, d3.kv_v = t["kv_k"].ptr, t["kv_v"].ptr  # the tensors the first call updated
    d3.pnext = C.addressof(ext)
    assert ctx.lib.hip_paged_attention_impl(ctx.device_ctx, C.byref(d3)) == ta.SUCCESS, ctx.last_error()
    tol2 = TOLERANCE["f32"] * 240.0 * state2["v_scale"].max()
    assert np.max(np.abs(ctx.to_host(t3["out"]).astype(np.float64) - ref2)) <= tol2
    assert same_state(t, state2)
    for group in (t, t2, t3):
        for name, x in group.items():
            if name != "fused":
                ctx.host_freed(x)


def test_impl_paged_attention_errors(ctx):
    """The checks of cpu_paged_attention_impl in its order (paged_attention_ref.c:573-823), then what this backend
    leaves to the fallback."""
    from tests.attention_cases import make_case

    case = make_case(72, [(5, 2)], num_q_heads=4, num_kv_heads=2, head_dim=64, block_size=8)
    t, desc = _attention_tensors(ctx, case)

    def call(**kw):
        d = ta.PagedAttentionDesc.default()
        C.memmove(C.byref(d), C.byref(desc), C.sizeof(d))
        for k, v in kw.items():
            setattr(d, k, v.ptr if isinstance(v, ta.HostTensor) else v)
        return ctx.lib.hip_paged_attention_impl(ctx.device_ctx, C.byref(d))

    assert call() == ta.SUCCESS
    assert call(struct_version=2) == ta.INVALID_ARGUMENT and "descriptor invalid" in ctx.last_error()[1]
    assert call(token_count=0) == ta.SUCCESS
    assert call(block_size=6) == ta.INVALID_ARGUMENT and "power of two" in ctx.last_error()[1]
    assert call(num_kv_heads=3) == ta.INVALID_ARGUMENT
    f32_meta = ta.HostTensor.dense(np.zeros((2, 4), np.float32))
    assert call(token_meta=f32_meta) == ta.UNSUPPORTED_DTYPE and "uint32 metadata" in ctx.last_error()[1]
    ints = ta.HostTensor.dense(np.zeros((2, 4, 64), np.int32))
    assert call(q=ints) == ta.UNSUPPORTED_DTYPE
    half_out = ta.HostTensor.dense(np.zeros((2, 4, 64), np.float16))
    assert call(out=half_out) == ta.UNSUPPORTED_DTYPE and "matching" in ctx.last_error()[1]
    assert call(token_count=1) == ta.DIMENSION_MISMATCH and "token_meta shape" in ctx.last_error()[1]
    assert call(num_q_heads=8, num_kv_heads=2) == ta.DIMENSION_MISMATCH and "num_q_heads" in ctx.last_error()[1]
    assert call(head_dim=32) == ta.DIMENSION_MISMATCH and "head_dim" in ctx.last_error()[1]
    assert call(layer_idx=2) == ta.DIMENSION_MISMATCH and "layer_idx" in ctx.last_error()[1]
    assert call(block_size=16) == ta.DIMENSION_MISMATCH and "block_size" in ctx.last_error()[1]
    half_cache = ta.HostTensor.dense(case["kv_v"].astype(np.float16))
    assert call(kv_v=half_cache) == ta.DIMENSION_MISMATCH and "kv dtype" in ctx.last_error()[1]
    bad = case["token_meta"].copy()
    bad[1, 0] = case["block_table"].shape[0]
    assert call(token_meta=ta.HostTensor.dense(bad)) == ta.DIMENSION_MISMATCH and "seq_slot" in ctx.last_error()[1]
    bad[1, 0], bad[1, 2] = 0, case["kv_k"].shape[0] * 8
    assert call(token_meta=ta.HostTensor.dense(bad)) == ta.DIMENSION_MISMATCH and "kv_slot" in ctx.last_error()[1]
    fp8 = [ta.HostTensor.strided(np.zeros(case["kv_k"].shape, np.uint8), ta.DTYPE_F8_E4M3) for _ in range(2)]
    assert call(kv_k=fp8[0], kv_v=fp8[1]) == ta.INVALID_ARGUMENT and "requires scale tensors" in ctx.last_error()[1]
    ext = ta.PagedAttentionKvScaleExt(C.sizeof(ta.PagedAttentionKvScaleExt), 1, t["kv_k"].ptr, t["kv_v"].ptr)
    assert call(pnext=C.addressof(ext)) == ta.INVALID_ARGUMENT and "require FP8" in ctx.last_error()[1]
    # the scale tensors of an FP8 cache: FLOAT32, [blocks, layers, kv heads] (paged_attention_ref.c:694-722)
    shape3 = case["kv_k"].shape[:3]
    for arr, code, text in ((np.zeros(shape3, np.float16), ta.UNSUPPORTED_DTYPE, "must be float32"),
                            (np.zeros(shape3[:2], np.float32), ta.DIMENSION_MISMATCH, "must be 3D"),
                            (np.zeros((shape3[0], shape3[1], shape3[2] + 1), np.float32), ta.DIMENSION_MISMATCH,
                             "shape mismatch")):
        sc = [ta.HostTensor.dense(arr.copy()) for _ in range(2)]
        bad_ext = ta.PagedAttentionKvScaleExt(C.sizeof(ta.PagedAttentionKvScaleExt), 1, sc[0].ptr, sc[1].ptr)
        assert call(kv_k=fp8[0], kv_v=fp8[1], pnext=C.addressof(bad_ext)) == code and text in ctx.last_error()[1]
    wide = make_case(73, [(2, 1)], num_q_heads=1, num_kv_heads=1, head_dim=320, block_size=4)
    tw, dw = _attention_tensors(ctx, wide)
    assert ctx.lib.hip_paged_attention_impl(ctx.device_ctx, C.byref(dw)) == ta.NOT_IMPLEMENTED
    for group in (t, tw):
        for name, x in group.items():
            if name != "fused":
                ctx.host_freed(x)


def test_program_whole_decoder_layer(ctx, oracle):
    """One decoder layer of a Llama-shaped model as ONE bytecode program on this backend, every node of the decode
    graph between the embedding and the logits: rms_norm -> q, k, v projections (Q4_K, Q4_K, Q6_K) -> rotary embedding
    of q and k -> paged attention (cache write + attention through the block table, fp16 cache) -> output projection
    -> residual add -> rms_norm -> gate, up -> swiglu -> down -> residual add. 12 tokens: three sequences with history,
    one of them a prompt chunk. Against the oracle's chain of the same operations."""
    from oracle.pyoracle import RopeParams as OracleRope
    from tests.attention_cases import make_case
    from tests.util import assert_moe_parity

    hq, hkv, hd, H, F, bs = 8, 2, 64, 512, 1024, 16
    case = make_case(80, [(21, 1), (40, 1), (7, 10)], num_q_heads=hq, num_kv_heads=hkv, head_dim=hd, block_size=bs,
                     act="f32", kv="f16", layers=1, layer_idx=0)
    meta = case["token_meta"]
    T = meta.shape[0]
    x = gaussian(1400, (T, H))
    w1 = gaussian(1401, (H,), 0.2) + np.float32(1.0)
    w2 = gaussian(1402, (H,), 0.2) + np.float32(1.0)
    wq = oracle.quantize(KIND_Q4_K, gaussian(1403, (hq * hd, H), 0.05))
    wk = oracle.quantize(KIND_Q4_K, gaussian(1404, (hkv * hd, H), 0.05))
    wv = oracle.quantize(KIND_Q6_K, gaussian(1405, (hkv * hd, H), 0.05))
    wo = oracle.quantize(KIND_Q4_K, gaussian(1406, (H, hq * hd), 0.05))
    wg = oracle.quantize(KIND_Q4_K, gaussian(1407, (F, H), 0.05))
    wu = oracle.quantize(KIND_Q4_K, gaussian(1408, (F, H), 0.05))
    wd = oracle.quantize(KIND_Q6_K, gaussian(1409, (H, F), 0.05))
    pos = meta[:, 1].astype(np.int32)
    pos_q, pos_k = np.repeat(pos, hq), np.repeat(pos, hkv)  # one position per (token, head) row
    scale = float(1.0 / np.sqrt(hd))

    # ---- the oracle's chain
    r_h = oracle.rms_norm(x, w1, eps=1e-5)
    r_q = oracle.matmul(KIND_Q4_K, wq, r_h, hq * hd, threads=8)
    r_k = oracle.matmul(KIND_Q4_K, wk, r_h, hkv * hd, threads=8)
    r_v = oracle.matmul(KIND_Q6_K, wv, r_h, hkv * hd, threads=8)
    rp = OracleRope.default(rope_type=0)
    st, r_qr = oracle.rope(r_q.reshape(T * hq, hd), pos_q, rp)
    assert st == 0
    st, r_kr = oracle.rope(r_k.reshape(T * hkv, hd), pos_k, rp)
    assert st == 0
    ref_k, ref_v = case["kv_k"].copy(), case["kv_v"].copy()
    st, r_att = oracle.paged_attention(meta, r_qr.reshape(T, hq, hd), r_kr.reshape(T, hkv, hd), r_v.reshape(T, hkv, hd),
                                       ref_k, ref_v, case["block_table"], 0, scale)
    assert st == 0
    r_o = oracle.matmul(KIND_Q4_K, wo, r_att.reshape(T, hq * hd), H, threads=8)
    r_x1 = x + r_o
    r_h2 = oracle.rms_norm(r_x1, w2, eps=1e-5)
    r_a = oracle.glu(oracle.matmul(KIND_Q4_K, wg, r_h2, F, threads=8), oracle.matmul(KIND_Q4_K, wu, r_h2, F, threads=8))
    r_y = r_x1 + oracle.matmul(KIND_Q6_K, wd, r_a, H, threads=8)

    # ---- the same as one program; 2-D projection outputs are viewed as [tokens, heads, head_dim] / [rows, head_dim]
    dense, empty, view = ta.HostTensor.dense, ta.HostTensor.empty, ta.HostTensor.strided
    xt, w1t, w2t = dense(x), dense(w1), dense(w2)
    wts = {n: ta.HostTensor.quantized(b, s, k) for n, (b, s, k) in {
        "q": (wq, (hq * hd, H), KIND_Q4_K), "k": (wk, (hkv * hd, H), KIND_Q4_K), "v": (wv, (hkv * hd, H), KIND_Q6_K),
        "o": (wo, (H, hq * hd), KIND_Q4_K), "g": (wg, (F, H), KIND_Q4_K), "u": (wu, (F, H), KIND_Q4_K),
        "d": (wd, (H, F), KIND_Q6_K)}.items()}
    h, q2, k2, v2 = empty((T, H), ta.DTYPE_F32), empty((T, hq * hd), ta.DTYPE_F32), empty((T, hkv * hd), ta.DTYPE_F32), \
        empty((T, hkv * hd), ta.DTYPE_F32)
    q_rows, k_rows = view(q2.array.reshape(T * hq, hd)), view(k2.array.reshape(T * hkv, hd))
    q3, k3, v3 = view(q2.array.reshape(T, hq, hd)), view(k2.array.reshape(T, hkv, hd)), view(v2.array.reshape(T, hkv, hd))
    att = empty((T, hq * hd), ta.DTYPE_F32)
    att3 = view(att.array.reshape(T, hq, hd))
    o, x1, h2, g, u, a, d, y = (empty(s, ta.DTYPE_F32) for s in
                                ((T, H), (T, H), (T, H), (T, F), (T, F), (T, F), (T, H), (T, H)))
    mt, tbl = dense(meta), dense(case["block_table"])
    kvk, kvv = view(case["kv_k"].copy()), view(case["kv_v"].copy())
    pq, pk = dense(pos_q), dense(pos_k)
    rq, rk = _rope_params(pq, rope_type=0), _rope_params(pk, rope_type=0)
    every = [xt, w1t, w2t, h, q2, k2, v2, att, o, x1, h2, g, u, a, d, y, mt, tbl, kvk, kvv, pq, pk] + list(wts.values())
    for t in every:
        ctx.host_range_freed(t)  # fresh memory: no mirror of a previous owner of these addresses
    mm = {KIND_Q4_K: 3, KIND_Q6_K: 4}
    p = ta.Program()
    p.rms_norm(ta.BC_OP_RMS_NORM_F32, xt, w1t, None, h, 1e-5)
    p.matmul(mm[KIND_Q4_K], h, wts["q"], q2)
    p.matmul(mm[KIND_Q4_K], h, wts["k"], k2)
    p.matmul(mm[KIND_Q6_K], h, wts["v"], v2)
    p.rope(ta.BC_OP_ROPE, q_rows, q_rows, rq)
    p.rope(ta.BC_OP_ROPE, k_rows, k_rows, rk)
    p.paged_attention(ta.BC_OP_PAGED_ATTENTION, mt, q3, k3, v3, kvk, kvv, tbl, att3, T, 0, hq, hkv, hd, bs, scale)
    p.matmul(mm[KIND_Q4_K], att, wts["o"], o)
    p.binary(ta.BC_OP_ADD_F32, xt, o, x1)
    p.rms_norm(ta.BC_OP_RMS_NORM_F32, x1, w2t, None, h2, 1e-5)
    p.matmul(mm[KIND_Q4_K], h2, wts["g"], g)
    p.matmul(mm[KIND_Q4_K], h2, wts["u"], u)
    p.binary(ta.BC_OP_SWIGLU_F32, g, u, a)
    p.matmul(mm[KIND_Q6_K], a, wts["d"], d)
    p.binary(ta.BC_OP_ADD_F32, x1, d, y)
    uploads0 = ctx.residency().uploads
    assert ctx.execute(p) == ta.SUCCESS, ctx.last_error()
    # intermediate tensors never travel: only the inputs (x, two norm weights), the seven weights, metadata and block
    # table, the two caches, the two position tensors and the rotary frequency table were uploaded
    assert ctx.residency().uploads - uploads0 == 3 + 7 + 2 + 2 + 2 + 1
    # Stage by stage, every operation against the oracle ON THE DEVICE'S OWN INPUTS of that stage (each linear
    # re-quantizes its input, so end-to-end differences grow with the chain; a stage's own error does not). Views are
    # read through the tensor object that was written (the "device copy is newer" flag belongs to it).
    from tests.attention_cases import TOLERANCE
    from tests.util import assert_matmul_parity

    g_h = ctx.to_host(h).copy()
    assert np.allclose(g_h, r_h, rtol=1e-5, atol=1e-8)
    g_q, g_k = ctx.to_host(q_rows).copy(), ctx.to_host(k_rows).copy()
    g_v = ctx.to_host(v2).copy()
    for got, w_, kind_, M_, pos_, heads in ((g_q, wq, KIND_Q4_K, hq * hd, pos_q, hq), (g_k, wk, KIND_Q4_K, hkv * hd, pos_k, hkv)):
        st, want = oracle.rope(oracle.matmul(kind_, w_, g_h, M_, threads=8).reshape(T * heads, hd), pos_, rp)
        assert st == 0
        assert_matmul_parity(got, want, what="projection + rotary embedding")
    assert_matmul_parity(g_v, oracle.matmul(KIND_Q6_K, wv, g_h, hkv * hd, threads=8), what="v projection")
    s_k, s_v = case["kv_k"].copy(), case["kv_v"].copy()
    st, want = oracle.paged_attention(meta, g_q.reshape(T, hq, hd), g_k.reshape(T, hkv, hd), g_v.reshape(T, hkv, hd),
                                      s_k, s_v, case["block_table"], 0, scale)
    assert st == 0
    g_att = ctx.to_host(att3).reshape(T, hq * hd).copy()
    assert np.max(np.abs(g_att - want.reshape(T, hq * hd))) <= TOLERANCE["f32"] * np.abs(s_v.astype(np.float32)).max()
    assert np.array_equal(ctx.to_host(kvk).view(np.uint8), s_k.view(np.uint8))  # the cache after the device's own rows
    assert np.array_equal(ctx.to_host(kvv).view(np.uint8), s_v.view(np.uint8))
    g_o = ctx.to_host(o).copy()
    assert_matmul_parity(g_o, oracle.matmul(KIND_Q4_K, wo, g_att, H, threads=8), what="output projection")
    g_x1 = ctx.to_host(x1).copy()
    assert np.array_equal(bits(g_x1), bits(x + g_o))
    g_h2 = ctx.to_host(h2).copy()
    assert np.allclose(g_h2, oracle.rms_norm(g_x1, w2, eps=1e-5), rtol=1e-5, atol=1e-8)
    g_a = ctx.to_host(a).copy()
    want_a = oracle.glu(oracle.matmul(KIND_Q4_K, wg, g_h2, F, threads=8), oracle.matmul(KIND_Q4_K, wu, g_h2, F, threads=8))
    assert_moe_parity(g_a, want_a, what="gate, up and the gated product")
    g_d = ctx.to_host(d).copy()
    assert_matmul_parity(g_d, oracle.matmul(KIND_Q6_K, wd, g_a, H, threads=8), what="down projection")
    assert np.array_equal(bits(ctx.to_host(y)), bits(g_x1 + g_d))
    # end to end against the oracle's own chain: five re-quantization points in a row
    assert_moe_parity(g_att, r_att.reshape(T, hq * hd), what="attention output inside the layer")
    assert_moe_parity(ctx.to_host(y), r_y, tol=1e-2, what="decoder layer output, end to end")
    # the cache rows the layer wrote: fp16 roundings of keys / values that differ from the oracle's by the linears'
    # summation order, so the comparison is numerical, not bitwise
    got_k = ctx.to_host(kvk).astype(np.float32)
    assert np.max(np.abs(got_k - ref_k.astype(np.float32))) <= 2e-3 * np.abs(ref_k.astype(np.float32)).max()
    for t in every:
        ctx.host_freed(t)
