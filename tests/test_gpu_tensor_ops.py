"""GPU parity of the tensor operations a GGUF model graph places around the quantized linears (activations, softmax,
conversions, row gather, slice, and the metadata-only reshape / view), through the raw C ABI, through the tensor-level
impl functions and as bytecode programs, against the CPU oracle and the reference's golden vectors."""
import ctypes as C

import numpy as np
import pytest

from marmot_amd import capi
from marmot_amd import tensor_abi as ta
from oracle.pyoracle import DT_BF16, DT_F16, DT_F32
from tests.util import gaussian

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def hip():
    from marmot_amd import HipBackend

    b = HipBackend(0)
    yield b
    b.close()


@pytest.fixture(scope="module")
def ctx():
    with ta.HipContext() as c:
        yield c


def bits16(a):
    return np.ascontiguousarray(a).view(np.uint16)


# The device's erff / tanhf / expf are accurate to a few units in the last place of their results; 1 + erf(.) and
# 1 + tanh(.) cancel for x << 0, which turns that into an absolute error of |x| * 2^-22.
def close_activation(got, ref, x, what):
    err = np.abs(got.astype(np.float64) - ref.astype(np.float64))
    bound = 4e-6 * np.abs(ref.astype(np.float64)) + 3e-7 * np.abs(x.astype(np.float64)) + 1e-30
    assert np.all(np.isfinite(got)) and np.all(err <= bound), f"{what}: {float((err - bound).max()):.3e}"


def close_activation_f16(got, ref, x, what):
    """One FLOAT16 rounding of fp32 results that may differ by the bound above: the same code, or a neighbouring one
    (at most a spacing of FLOAT16 at the value, plus the fp32 bound where that is larger: results that cancel to
    about -1e-7 on one side and to -0 on the other)."""
    g, r = got.astype(np.float64), ref.astype(np.float64)
    bound = np.spacing(np.abs(ref)).astype(np.float64) + 3e-7 * np.abs(x.astype(np.float64))
    err = np.abs(g - r)
    assert np.all(np.isfinite(g)) and np.all(err <= bound), f"{what}: {float((err - bound).max()):.3e}"
    assert np.count_nonzero(err) <= max(8, got.size // 200), f"{what}: {np.count_nonzero(err)} values differ"


# ------------------------------------------------------------------ raw C ABI
def test_unary_matches_oracle_and_reference_goldens(hip, oracle, ref_goldens):
    print("unary: goldens", flush=True)
    x = ref_goldens["g_activation_input"]
    for op, key in ((hip.UNARY_GELU, "gelu"), (hip.UNARY_GELU_TANH, "gelu_tanh"), (hip.UNARY_SILU, "silu")):
        assert np.allclose(hip.unary(op, x), ref_goldens["g_activation_" + key], rtol=2e-6, atol=1e-8), key
    for n in (1, 63, 4096, 100003):
        x = np.concatenate([gaussian(1200 + n, (n,), 3.0), np.array([0.0, -0.0, 11.5, -11.5, 40.0, -40.0], np.float32)])
        for op in (hip.UNARY_GELU, hip.UNARY_GELU_TANH, hip.UNARY_SILU):
            print(f"unary: op {op} n {n}", flush=True)
            got = hip.unary(op, x)
            close_activation(got, oracle.unary(op, x), x, f"unary {op} n={n}")
            assert np.array_equal(hip.unary(op, x, in_place=True), got)
    h = gaussian(1210, (5000,), 2.0).astype(np.float16)
    for op in (hip.UNARY_GELU, hip.UNARY_GELU_TANH, hip.UNARY_SILU):
        close_activation_f16(hip.unary(op, h), oracle.unary(op, h), h, f"unary {op} FLOAT16")
    assert hip.unary(hip.UNARY_GELU, np.zeros((0, 4), np.float32)).shape == (0, 4)
    assert hip.lib.marmot_hip_unary(hip.dev, 9, C.c_void_p(8), 0, 1, C.c_void_p(8)) == -1
    assert hip.lib.marmot_hip_unary(hip.dev, 0, C.c_void_p(8), capi.DT_BF16, 1, C.c_void_p(8)) == -6


def test_softmax_matches_oracle_and_reference_goldens(hip, oracle, ref_goldens):
    shape = tuple(int(v) for v in ref_goldens["g_softmax_shape"])
    x = ref_goldens["g_softmax_input"].reshape(shape)
    assert np.allclose(hip.softmax(x, -1).ravel(), ref_goldens["g_softmax_expected_axis_last"], rtol=2e-6)
    assert np.allclose(hip.softmax(x, 0).ravel(), ref_goldens["g_softmax_expected_axis0"], rtol=2e-6)
    for shape, axis in (((5, 8), -1), ((300, 128), 1), ((4, 1000), -1), ((2, 6, 5), 1), ((3, 4, 7), 0), ((2, 32000), 1),
                        ((7,), 0), ((1, 129), 1), ((64, 60), -1), ((3, 151936), -1)):
        print(f"softmax {shape} axis {axis}", flush=True)
        x = gaussian(1300 + len(shape) + shape[-1], shape, 4.0)
        got, ref = hip.softmax(x, axis), oracle.softmax(x, axis)
        n = shape[axis]
        # rows of up to 128 contiguous values are summed in index order like the CPU loop: only expf differs; longer
        # rows are summed as a tree, which moves 1 / sum by up to the error of the sequential fp32 sum itself
        rtol = 3e-6 if n <= 128 and axis in (-1, len(shape) - 1) else max(3e-6, n * 2e-9)
        assert np.allclose(got, ref, rtol=rtol, atol=1e-30), (shape, np.abs(got - ref).max())
        assert np.allclose(got.sum(axis=axis, dtype=np.float64), 1.0, atol=max(1e-5, 2 * rtol))
        assert np.array_equal(hip.softmax(x, axis, in_place=True), got)
    x = np.array([[0.0, -87.5, -88.0, -89.0, -1000.0]], np.float32)
    for pad in (0, 200):  # the one-thread and the 256-thread kernel
        row = np.concatenate([x, np.full((1, pad), -2000.0, np.float32)], axis=1)
        got = hip.softmax(row)
        assert got[0, 1] > 0 and np.all(got[0, 2:] == 0) and abs(got[0, 0] - 1.0) < 1e-6
    assert hip.lib.marmot_hip_softmax(hip.dev, C.c_void_p(8), 1, 0, 1, C.c_void_p(8)) == -1


def ulps16(a_bits: np.ndarray, b_bits: np.ndarray) -> np.ndarray:
    """Distance in units of the last place between two arrays of non-negative 16-bit float patterns."""
    return np.abs(a_bits.astype(np.int32) - b_bits.astype(np.int32))


@pytest.mark.parametrize("dtype_name", ["f16", "bf16"])
def test_softmax_16_bit_types_match_oracle_and_reference_goldens(hip, oracle, ref_goldens, dtype_name):
    """FLOAT16 / BFLOAT16 softmax: the reference's check for these types (g_softmax at 5e-3 / 1.2e-2, twice that along
    axis 0, tests/backend/test_backend_softmax.c:6-45, 53-54), then the oracle's two roundings: the device's expf and
    the tree sum of long rows move a value across a rounding boundary now and then, by one unit of the last place at
    most."""
    dtype = capi.DT_F16 if dtype_name == "f16" else capi.DT_BF16
    tol = 5e-3 if dtype_name == "f16" else 1.2e-2
    shape = tuple(int(v) for v in ref_goldens["g_softmax_shape"])
    xb = oracle.convert(ref_goldens["g_softmax_input"].reshape(shape).astype(np.float32), capi.DT_F32, dtype)
    for axis, key, factor in ((-1, "g_softmax_expected_axis_last", 1.0), (0, "g_softmax_expected_axis0", 2.0)):
        got = oracle.convert(hip.softmax(xb, axis, dtype=dtype), dtype, capi.DT_F32)
        assert np.max(np.abs(got.ravel().astype(np.float64) - ref_goldens[key].astype(np.float64))) <= tol * factor
    for shape, axis in (((5, 8), -1), ((300, 128), 1), ((4, 1000), -1), ((2, 6, 5), 1), ((3, 4, 7), 0), ((2, 32000), 1),
                        ((7,), 0), ((1, 129), 1), ((64, 60), -1)):
        print(f"softmax {dtype_name} {shape} axis {axis}", flush=True)
        xb = oracle.convert(gaussian(1400 + len(shape) + shape[-1], shape, 3.0), capi.DT_F32, dtype)
        got, ref = hip.softmax(xb, axis, dtype=dtype), oracle.softmax_typed(xb, dtype, axis)
        d = ulps16(got, ref)
        assert d.max() <= 1 and np.mean(d == 0) >= 0.99, (shape, int(d.max()), float(np.mean(d == 0)))
        assert np.array_equal(hip.softmax(xb, axis, in_place=True, dtype=dtype), got)
    assert hip.lib.marmot_hip_softmax_typed(hip.dev, capi.DT_I32, C.c_void_p(8), 1, 4, 1, C.c_void_p(8)) == -6
    assert hip.lib.marmot_hip_softmax_typed(hip.dev, dtype, C.c_void_p(8), 1, 0, 1, C.c_void_p(8)) == -1


def test_convert_is_bit_exact(hip, oracle, ref_goldens):
    g = ref_goldens
    assert np.array_equal(hip.convert(g["g_conv_f16_src"], DT_F32, DT_F16), g["g_conv_f16_f16_bits"])
    assert np.array_equal(hip.convert(g["g_conv_bf16_src"], DT_F32, DT_BF16), g["g_conv_bf16_bf16_bits"])
    assert np.array_equal(hip.convert(g["g_conv_bf16_bf16_bits"], DT_BF16, DT_F32), g["g_conv_bf16_roundtrip"])
    assert np.array_equal(hip.convert(g["g_conv_f16_bf16_bridge_f16_bits"], DT_F16, DT_BF16),
                          g["g_conv_f16_bf16_bridge_bf16_from_f16_bits"])
    assert np.array_equal(hip.convert(g["g_conv_f16_bf16_bridge_bf16_bits"], DT_BF16, DT_F16),
                          g["g_conv_f16_bf16_bridge_f16_from_bf16_bits"])
    all16 = np.arange(1 << 16, dtype=np.uint16)
    finite_h = all16[(all16 & 0x7c00) != 0x7c00]
    finite_b = all16[(all16 & 0x7f80) != 0x7f80]
    h = finite_h.view(np.float16).astype(np.float64)
    with np.errstate(over="ignore"):
        nxt = np.nextafter(finite_h.view(np.float16), np.float16(np.inf)).astype(np.float64)
    ties = ((h + nxt) / 2).astype(np.float32)
    x = np.concatenate([gaussian(1400 + i, (30000,), s) for i, s in enumerate((1e-7, 1e-4, 1.0, 300.0, 7e4))] +
                       [ties, np.nextafter(ties, np.float32(np.inf)), np.nextafter(ties, np.float32(-np.inf)),
                        np.array([65504.0, 65519.99, 65520.0, 65536.0, -65520.0, 2.0 ** -25, 2.0 ** -24,
                                  1.5 * 2.0 ** -25, np.inf, -np.inf, 0.0, -0.0], np.float32)])
    for src, sdt in ((x, DT_F32), (finite_h, DT_F16), (finite_b, DT_BF16)):
        for ddt in (DT_F32, DT_F16, DT_BF16):
            print(f"convert {sdt} -> {ddt} n {src.size}", flush=True)
            got, ref = hip.convert(src, sdt, ddt), oracle.convert(src, sdt, ddt)
            assert np.array_equal(got.view(np.uint8), ref.view(np.uint8)), (sdt, ddt)
    # NaN inputs: equal types copy every bit pattern; widening keeps a NaN a NaN (the payload is not part of the
    # contract: the hardware conversion quiets a signaling NaN). Narrowing a NaN to BFLOAT16 is left open: the
    # reference's rounding bias can carry a NaN payload into the sign bit (src/utils/dtype_ref.c:86-96).
    for dt in (DT_F16, DT_BF16):
        assert np.array_equal(hip.convert(all16, dt, dt), all16)
        wide, ref = hip.convert(all16, dt, DT_F32), oracle.convert(all16, dt, DT_F32)
        nan = np.isnan(ref)
        assert np.array_equal(np.isnan(wide), nan) and np.array_equal(wide[~nan].view(np.uint32), ref[~nan].view(np.uint32))
    assert hip.lib.marmot_hip_convert(hip.dev, C.c_void_p(8), capi.DT_I32, C.c_void_p(8), 0, 4) == -6


def test_gather_rows_is_bit_exact(hip, oracle):
    rng = np.random.Generator(np.random.PCG64(1500))
    for rows, cols, dtype in ((7, 5, np.float32), (100, 64, np.float16), (3, 1, np.int32), (16, 4096, np.float32),
                              (9, 3, np.uint8), (50, 4100, np.float16), (4, 20000, np.float32)):
        x = rng.integers(0, 250, size=(rows, cols)).astype(dtype)
        for idt in (np.int32, np.uint32):
            idx = rng.integers(0, rows, size=11).astype(idt)
            print(f"gather {rows}x{cols} {np.dtype(dtype).name} idx {np.dtype(idt).name}", flush=True)
            assert np.array_equal(hip.gather_rows(x, idx), oracle.gather_rows(x, idx))
        wide = rng.integers(0, 250, size=(rows, cols + 3)).astype(dtype)
        idx = rng.integers(0, rows, size=5).astype(np.int32)
        got = hip.gather_rows(wide[:, :cols], idx, out_stride=cols + 2)  # strided rows in and out
        assert np.array_equal(got[:, :cols], wide[idx, :cols])
        assert np.all(got[:, cols:].view(np.uint8) == 0xFF)  # the gaps between output rows are not written
        assert hip.gather_rows(x, np.zeros(0, np.int32)).shape == (0, cols)
    x = np.arange(12, dtype=np.float32).reshape(4, 3)
    for bad in (np.array([0, 4], np.int32), np.array([-1, 0], np.int32), np.array([1, 2, 0xFFFFFFFF], np.uint32)):
        with pytest.raises(capi.MarmotHipError) as e:
            hip.gather_rows(x, bad)
        assert e.value.code == -1 and "out of range" in str(e.value)
    assert np.array_equal(hip.gather_rows(x, np.array([3, 0], np.int32)), x[[3, 0]])  # the error leaves no residue


def test_slice_is_bit_exact(hip, oracle, ref_goldens):
    g = ref_goldens
    shape = tuple(int(v) for v in g["g_tensor_slice3d_shape_src"])
    got = hip.slice(g["g_tensor_slice3d_src"].reshape(shape), g["g_tensor_slice3d_starts"],
                    [int(v) for v in g["g_tensor_slice3d_sizes"]])
    assert np.array_equal(got.ravel(), g["g_tensor_slice3d_expected"])
    rng = np.random.Generator(np.random.PCG64(1600))
    for shape, dtype in (((9,), np.float32), ((5, 7), np.float16), ((3, 4, 5), np.int32), ((2, 3, 4, 5), np.uint8),
                         ((2, 2, 3, 2, 3), np.float64), ((2, 1, 2, 2, 1, 3, 2, 2), np.int16), ((64, 4096), np.float32),
                         ((3, 700, 129), np.float16)):
        x = rng.integers(0, 250, size=shape).astype(dtype)
        for _ in range(4):
            starts = [int(rng.integers(0, n)) for n in shape]
            sizes = [int(rng.integers(1, n - s + 1)) for n, s in zip(shape, starts)]
            print(f"slice {shape} {starts} {sizes}", flush=True)
            assert np.array_equal(hip.slice(x, starts, sizes), oracle.slice(x, starts, sizes))
        assert np.array_equal(hip.slice(x, [0] * len(shape), list(shape)), x)
        assert hip.slice(x, [0] * len(shape), [0] + list(shape[1:])).size == 0
    with pytest.raises(capi.MarmotHipError) as e:
        hip.slice(np.zeros((4, 4), np.float32), [2, 0], [3, 4])
    assert e.value.code == -1


# ------------------------------------------------------------------ tensor-level impl functions and programs
def _sig(ctx, op_id, in_dtype=ta.DTYPE_F32, out_dtype=None):
    sig = ctx.float_op_signature(op_id, in_dtype)
    if out_dtype is not None:
        sig.output_dtype = out_dtype
    return sig


def test_queries_for_the_graph_nodes(ctx):
    for op, bc in ((ta.OP_GELU, ta.BC_OP_GELU), (ta.OP_GELU_TANH, ta.BC_OP_GELU_TANH), (ta.OP_SILU, ta.BC_OP_SILU)):
        for dt in (ta.DTYPE_F32, ta.DTYPE_F16):
            sel = ctx.query(_sig(ctx, op, dt))
            assert sel.supported and sel.op_index == bc
        assert not ctx.query(_sig(ctx, op, ta.DTYPE_BF16)).supported
    for dt in (ta.DTYPE_F32, ta.DTYPE_F16, ta.DTYPE_BF16):  # one executor, the type is read from the tensors
        sel = ctx.query(_sig(ctx, ta.OP_SOFTMAX, dt))
        assert sel.supported and sel.op_index == ta.BC_OP_SOFTMAX_F32
    assert not ctx.query(_sig(ctx, ta.OP_SOFTMAX, ta.DTYPE_F16, ta.DTYPE_F32)).supported
    assert not ctx.query(_sig(ctx, ta.OP_SOFTMAX, ta.DTYPE_I32)).supported
    for op, bc in ((ta.OP_RESHAPE, ta.BC_OP_RESHAPE), (ta.OP_VIEW, ta.BC_OP_VIEW), (ta.OP_SLICE, ta.BC_OP_SLICE),
                   (ta.OP_GATHER_ROWS, ta.BC_OP_GATHER_ROWS)):
        sel = ctx.query(_sig(ctx, op, ta.DTYPE_F16))
        assert sel.supported and sel.op_index == bc
    assert ctx.query(_sig(ctx, ta.OP_CONVERT, ta.DTYPE_F32, ta.DTYPE_BF16)).op_index == ta.BC_OP_CONVERT
    assert not ctx.query(_sig(ctx, ta.OP_CONVERT, ta.DTYPE_F32, ta.DTYPE_I32)).supported
    assert ctx.tables.op_count == 64
    for bc, n, schema in ((ta.BC_OP_GELU, 8, 1), (ta.BC_OP_SOFTMAX_F32, 8, 5), (ta.BC_OP_RESHAPE, 16, 14),
                          (ta.BC_OP_VIEW, 12, 15), (ta.BC_OP_SLICE, 12, 19), (ta.BC_OP_GATHER_ROWS, 6, 20),
                          (ta.BC_OP_CONVERT, 24, 25)):
        assert ctx.tables.imm_size[bc] == n and ctx.tables.schema_id[bc] == schema


def test_impl_unary_and_softmax(ctx, oracle):
    x = gaussian(1700, (3, 5, 64), 2.0)
    xt, ot = ta.HostTensor.dense(x), ta.HostTensor.empty(x.shape, ta.DTYPE_F32)
    for fn, op, bc in ((ctx.lib.hip_gelu, oracle.UNARY_GELU, ta.BC_OP_GELU),
                       (ctx.lib.hip_gelu_tanh, oracle.UNARY_GELU_TANH, ta.BC_OP_GELU_TANH),
                       (ctx.lib.hip_silu, oracle.UNARY_SILU, ta.BC_OP_SILU)):
        assert fn(ctx.device_ctx, xt.ptr, None, ot.ptr) == ta.SUCCESS, ctx.last_error()
        assert ot.t.memory_location == ta.MEMORY_DEVICE and ot.t.needs_sync
        close_activation(ctx.to_host(ot), oracle.unary(op, x), x, f"impl unary {op}")
        ot.array[...] = 0
        ctx.host_changed(ot)
        prog = ta.Program()
        prog.unary(bc, xt, ot, ta.ActivationParams())  # parameters without tensors are accepted and unused
        assert ctx.execute(prog) == ta.SUCCESS, ctx.last_error()
        close_activation(ctx.to_host(ot), oracle.unary(op, x), x, f"program unary {op}")
    h = gaussian(1701, (6, 40)).astype(np.float16)
    ht, hot = ta.HostTensor.dense(h), ta.HostTensor.empty(h.shape, ta.DTYPE_F16)
    assert ctx.lib.hip_gelu(ctx.device_ctx, ht.ptr, None, hot.ptr) == ta.SUCCESS, ctx.last_error()
    close_activation_f16(ctx.to_host(hot), oracle.unary(oracle.UNARY_GELU, h), h, "impl gelu FLOAT16")
    # errors: dtype mismatch, shape mismatch, unsupported type, a bias tensor
    assert ctx.lib.hip_gelu(ctx.device_ctx, xt.ptr, None, hot.ptr) == ta.UNSUPPORTED_DTYPE
    small = ta.HostTensor.empty((3, 5, 63), ta.DTYPE_F32)
    assert ctx.lib.hip_silu(ctx.device_ctx, xt.ptr, None, small.ptr) == ta.DIMENSION_MISMATCH
    it, iot = ta.HostTensor.dense(np.zeros((2, 2), np.int32)), ta.HostTensor.empty((2, 2), ta.DTYPE_I32)
    assert ctx.lib.hip_gelu(ctx.device_ctx, it.ptr, None, iot.ptr) == ta.NOT_IMPLEMENTED
    params = ta.ActivationParams()
    params.bias = xt.ptr
    assert ctx.lib.hip_gelu(ctx.device_ctx, xt.ptr, C.byref(params), ot.ptr) == ta.NOT_IMPLEMENTED
    assert ctx.lib.hip_gelu(ctx.device_ctx, None, None, ot.ptr) == ta.INVALID_ARGUMENT

    for shape, axis in (((4, 8), -1), ((2, 6, 5), 1), ((3, 4, 7), 0), ((5, 300), 1)):
        x = gaussian(1710 + shape[-1], shape, 3.0)
        st, so = ta.HostTensor.dense(x.copy()), ta.HostTensor.empty(shape, ta.DTYPE_F32)
        desc = ta.SoftmaxDesc(st.ptr, so.ptr, axis)
        assert ctx.lib.hip_softmax_impl(ctx.device_ctx, C.byref(desc)) == ta.SUCCESS, ctx.last_error()
        assert np.allclose(ctx.to_host(so), oracle.softmax(x, axis), rtol=3e-6, atol=1e-30)
        prog = ta.Program()
        prog.softmax(ta.BC_OP_SOFTMAX_F32, st, st, axis)  # in place
        assert ctx.execute(prog) == ta.SUCCESS, ctx.last_error()
        assert np.allclose(ctx.to_host(st), oracle.softmax(x, axis), rtol=3e-6, atol=1e-30)
        for t in (st, so):
            ctx.host_freed(t)
    # FLOAT16 and BFLOAT16 tensors (bfloat16 bits travel in uint16 arrays): the implementation and the program
    for dtype, ta_dtype in ((capi.DT_F16, ta.DTYPE_F16), (capi.DT_BF16, ta.DTYPE_BF16)):
        for shape, axis in (((4, 8), -1), ((2, 6, 5), 1), ((5, 300), 1)):
            xb = oracle.convert(gaussian(1730 + shape[-1], shape, 3.0), capi.DT_F32, dtype)
            want = oracle.softmax_typed(xb, dtype, axis)
            view = xb.view(np.float16) if dtype == capi.DT_F16 else xb
            st = ta.HostTensor.strided(view.copy(), ta_dtype)
            so = ta.HostTensor.strided(np.zeros_like(view), ta_dtype)
            desc = ta.SoftmaxDesc(st.ptr, so.ptr, axis)
            assert ctx.lib.hip_softmax_impl(ctx.device_ctx, C.byref(desc)) == ta.SUCCESS, ctx.last_error()
            d = np.abs(ctx.to_host(so).view(np.uint16).astype(np.int32) - want.astype(np.int32))
            assert d.max() <= 1 and np.mean(d == 0) >= 0.98, (dtype, shape, int(d.max()))
            prog = ta.Program()
            prog.softmax(ta.BC_OP_SOFTMAX_F32, st, st, axis)  # in place
            assert ctx.execute(prog) == ta.SUCCESS, ctx.last_error()
            d = np.abs(ctx.to_host(st).view(np.uint16).astype(np.int32) - want.astype(np.int32))
            assert d.max() <= 1, (dtype, shape, int(d.max()))
            for t in (st, so):
                ctx.host_freed(t)
    st, so = ta.HostTensor.dense(gaussian(1720, (4, 8))), ta.HostTensor.empty((4, 8), ta.DTYPE_F32)
    for axis, code in ((2, ta.INVALID_ARGUMENT), (-3, ta.INVALID_ARGUMENT)):
        desc = ta.SoftmaxDesc(st.ptr, so.ptr, axis)
        assert ctx.lib.hip_softmax_impl(ctx.device_ctx, C.byref(desc)) == code
        assert "axis out of range" in ctx.last_error()[1]
    desc = ta.SoftmaxDesc(st.ptr, ta.HostTensor.empty((4, 9), ta.DTYPE_F32).ptr, 1)
    assert ctx.lib.hip_softmax_impl(ctx.device_ctx, C.byref(desc)) == ta.DIMENSION_MISMATCH
    desc = ta.SoftmaxDesc(st.ptr, ta.HostTensor.empty((4, 8), ta.DTYPE_F16).ptr, 1)
    assert ctx.lib.hip_softmax_impl(ctx.device_ctx, C.byref(desc)) == ta.UNSUPPORTED_DTYPE
    assert ctx.lib.hip_softmax_impl(ctx.device_ctx, None) == ta.INVALID_ARGUMENT
    for t in (xt, ot, ht, hot, small, it, iot, st, so):
        ctx.host_freed(t)


def test_reshape_and_view_move_no_bytes(ctx, oracle):
    """The outputs alias the input's host bytes, the residency table resolves them into the input's mirror: no upload,
    no download and no new mirror between an operation that wrote the input on the device and one that reads the view."""
    a, b_ = gaussian(1800, (6, 64)), gaussian(1801, (6, 64))
    at, bt, st_ = ta.HostTensor.dense(a), ta.HostTensor.dense(b_), ta.HostTensor.empty((6, 64), ta.DTYPE_F32)
    assert ctx.lib.hip_add_f32(ctx.device_ctx, at.ptr, bt.ptr, st_.ptr) == ta.SUCCESS  # the sum lives on the device
    before = ctx.residency()
    rt = ta.HostTensor.header((2, 3, 64), ta.DTYPE_F32)
    shape = (C.c_size_t * 3)(2, 3, 64)
    assert ctx.lib.hip_reshape(ctx.device_ctx, st_.ptr, rt.ptr, shape, 3) == ta.SUCCESS, ctx.last_error()
    assert rt.t.data == st_.t.data and not rt.t.owns_data and rt.t.capacity_bytes == st_.t.capacity_bytes
    assert [rt.t.shape.strides[i] for i in range(3)] == [192, 64, 1]
    assert rt.t.memory_location == ta.MEMORY_DEVICE and rt.t.needs_sync  # inherited from the input
    vt = ta.HostTensor.header((2, 64), ta.DTYPE_F32)
    vt.t.shape.strides[0], vt.t.shape.strides[1] = 64, 1
    assert ctx.lib.hip_view(ctx.device_ctx, st_.ptr, vt.ptr, 3 * 64 * 4) == ta.SUCCESS, ctx.last_error()
    assert vt.t.data == st_.t.data + 3 * 64 * 4 and vt.t.capacity_bytes == 3 * 64 * 4
    # softmax of the view (rows 3 and 4 of the sum), in a program that also holds the two metadata nodes
    ot = ta.HostTensor.empty((2, 64), ta.DTYPE_F32)
    rt2, vt2 = ta.HostTensor.header((12, 32), ta.DTYPE_F32), ta.HostTensor.header((2, 64), ta.DTYPE_F32)
    vt2.t.shape.strides[0], vt2.t.shape.strides[1] = 64, 1
    prog = ta.Program()
    prog.reshape(ta.BC_OP_RESHAPE, st_, rt2, (12, 32))
    prog.view(ta.BC_OP_VIEW, st_, vt2, 3 * 64 * 4)
    prog.softmax(ta.BC_OP_SOFTMAX_F32, vt2, ot, -1)
    assert ctx.execute(prog) == ta.SUCCESS, ctx.last_error()
    assert rt2.t.shape.ndim == 2 and rt2.t.data == st_.t.data and vt2.t.data == vt.t.data
    after = ctx.residency()
    assert after.uploads == before.uploads and after.downloads == before.downloads
    assert after.mirrors == before.mirrors + 1  # the softmax output only
    assert np.allclose(ctx.to_host(ot), oracle.softmax((a + b_)[3:5]), rtol=3e-6)
    # the view is also what the host sees once the parent is brought home
    assert np.array_equal(ctx.to_host(st_), a + b_)
    # errors of the reference, in its order
    assert ctx.lib.hip_reshape(ctx.device_ctx, st_.ptr, rt.ptr, (C.c_size_t * 2)(5, 64), 2) == ta.DIMENSION_MISMATCH
    assert ctx.lib.hip_reshape(ctx.device_ctx, st_.ptr, rt.ptr, shape, 0) == ta.INVALID_ARGUMENT
    ht = ta.HostTensor.header((2, 64), ta.DTYPE_F16)
    assert ctx.lib.hip_view(ctx.device_ctx, st_.ptr, ht.ptr, 0) == ta.INVALID_ARGUMENT
    assert "matching dtypes" in ctx.last_error()[1]
    assert ctx.lib.hip_view(ctx.device_ctx, st_.ptr, vt.ptr, 2) == ta.INVALID_ARGUMENT
    assert "align" in ctx.last_error()[1]
    assert ctx.lib.hip_view(ctx.device_ctx, st_.ptr, vt.ptr, 6 * 64 * 4 + 4) == ta.INVALID_ARGUMENT
    assert ctx.lib.hip_view(ctx.device_ctx, st_.ptr, vt.ptr, 5 * 64 * 4) == ta.DIMENSION_MISMATCH
    for t in (at, bt, st_, ot):
        ctx.host_freed(t)


def test_impl_and_program_slice_gather_convert(ctx, oracle):
    rng = np.random.Generator(np.random.PCG64(1900))
    x = gaussian(1901, (4, 6, 40))
    xt, ot = ta.HostTensor.dense(x), ta.HostTensor.empty((2, 3, 16), ta.DTYPE_F32)
    starts, sizes = (C.c_size_t * 3)(1, 2, 8), (C.c_size_t * 3)(2, 3, 16)
    assert ctx.lib.hip_slice(ctx.device_ctx, xt.ptr, ot.ptr, starts, sizes) == ta.SUCCESS, ctx.last_error()
    assert np.array_equal(ctx.to_host(ot), x[1:3, 2:5, 8:24])
    prog = ta.Program()
    prog.slice(ta.BC_OP_SLICE, xt, ot, (0, 0, 24), (2, 3, 16))
    assert ctx.execute(prog) == ta.SUCCESS, ctx.last_error()
    assert np.array_equal(ctx.to_host(ot), x[0:2, 0:3, 24:40])
    assert ctx.lib.hip_slice(ctx.device_ctx, xt.ptr, ot.ptr, (C.c_size_t * 3)(3, 0, 0), sizes) == ta.INVALID_ARGUMENT
    assert ctx.lib.hip_slice(ctx.device_ctx, xt.ptr, ot.ptr, starts, (C.c_size_t * 3)(2, 3, 8)) == ta.DIMENSION_MISMATCH

    # gather_rows: the last-token rows of a hidden-state matrix, indices from the host, rows of a strided parent
    hidden = gaussian(1902, (37, 96))
    idx = np.array([36, 0, 17, 17], np.int32)
    ht, it, gt = ta.HostTensor.dense(hidden), ta.HostTensor.dense(idx), ta.HostTensor.empty((4, 96), ta.DTYPE_F32)
    assert ctx.lib.hip_gather_rows(ctx.device_ctx, ht.ptr, it.ptr, gt.ptr) == ta.SUCCESS, ctx.last_error()
    assert np.array_equal(ctx.to_host(gt), hidden[idx])
    left = ta.HostTensor.strided(hidden[:, :50])
    gl = ta.HostTensor.empty((4, 50), ta.DTYPE_F32)
    ut = ta.HostTensor.dense(idx.astype(np.uint32))
    prog = ta.Program()
    prog.gather_rows(ta.BC_OP_GATHER_ROWS, left, ut, gl)
    assert ctx.execute(prog) == ta.SUCCESS, ctx.last_error()
    assert np.array_equal(ctx.to_host(gl), hidden[idx, :50])
    bad = ta.HostTensor.dense(np.array([0, 37, 1, 2], np.int32))
    assert ctx.lib.hip_gather_rows(ctx.device_ctx, ht.ptr, bad.ptr, gt.ptr) == ta.INVALID_ARGUMENT
    assert "out of range" in ctx.last_error()[1]
    i64 = ta.HostTensor.dense(idx.astype(np.int64))
    assert ctx.lib.hip_gather_rows(ctx.device_ctx, ht.ptr, i64.ptr, gt.ptr) == ta.UNSUPPORTED_DTYPE
    assert ctx.lib.hip_gather_rows(ctx.device_ctx, ht.ptr, it.ptr, gl.ptr) == ta.DIMENSION_MISMATCH
    h16 = ta.HostTensor.empty((4, 96), ta.DTYPE_F16)
    assert ctx.lib.hip_gather_rows(ctx.device_ctx, ht.ptr, it.ptr, h16.ptr) == ta.UNSUPPORTED_DTYPE

    # convert: host addresses; outside a batch the destination's host bytes are current when the call returns
    src = gaussian(1903, (1000,), 30.0)
    s_t, d_t = ta.HostTensor.dense(src), ta.HostTensor.empty((1000,), ta.DTYPE_F16)
    assert ctx.lib.hip_convert(ctx.device_ctx, ta.DTYPE_F16, d_t.t.data, ta.DTYPE_F32, s_t.t.data, 1000) == ta.SUCCESS
    assert np.array_equal(bits16(d_t.array), oracle.convert(src, DT_F32, DT_F16))
    b_t = ta.HostTensor(np.zeros(1000, np.uint16), (1000,), ta.DTYPE_BF16)
    prog = ta.Program()
    prog.convert(ta.BC_OP_CONVERT, b_t, d_t, 1000)  # FLOAT16 -> BFLOAT16 through the const-pool addresses
    assert ctx.execute(prog) == ta.SUCCESS, ctx.last_error()
    assert np.array_equal(b_t.array, oracle.convert(bits16(d_t.array), DT_F16, DT_BF16))
    # inside a batch the result stays on the device and feeds the next node without a download
    ops = ctx.ops
    f_t = ta.HostTensor.empty((1000,), ta.DTYPE_F32)
    act = ta.HostTensor.empty((1000,), ta.DTYPE_F32)
    assert ops.graph_batch_begin(ctx.device_ctx) == ta.SUCCESS
    before = ctx.residency()
    assert ctx.lib.hip_convert(ctx.device_ctx, ta.DTYPE_F32, f_t.t.data, ta.DTYPE_BF16, b_t.t.data, 1000) == ta.SUCCESS
    assert ctx.lib.hip_silu(ctx.device_ctx, f_t.ptr, None, act.ptr) == ta.SUCCESS
    assert ops.graph_batch_end(ctx.device_ctx, True) == ta.SUCCESS
    assert ctx.residency().downloads == before.downloads
    widened = oracle.convert(b_t.array, DT_BF16, DT_F32)
    close_activation(ctx.to_host(act), oracle.unary(oracle.UNARY_SILU, widened), widened, "convert -> silu in a batch")
    assert ctx.lib.hip_convert(ctx.device_ctx, ta.DTYPE_I32, f_t.t.data, ta.DTYPE_F32, s_t.t.data, 4) == ta.NOT_IMPLEMENTED
    for t in (xt, ot, ht, it, gt, gl, ut, bad, i64, h16, s_t, d_t, b_t, f_t, act):
        ctx.host_freed(t)
