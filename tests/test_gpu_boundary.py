"""GPU tests of the C-ABI boundary itself: state that must not leak from one
call into the next, and stores that must stay inside the tensors they were
given."""
import ctypes

import numpy as np
import pytest

import oracle_lib

pytestmark = pytest.mark.gpu


def _rand_q(rng, dt, shape):
    info = np.iinfo(dt)
    return rng.integers(info.min, info.max + 1, shape, dtype=dt)


def bits(a):
    return np.ascontiguousarray(a).view(np.uint32)


def test_quant_mode_belongs_to_one_op(rt, oracle):
    """om_mi355x_SetQuantMode applies to the next quantize / dequantize /
    dynamic-quantize / fused-layer call of the thread and to nothing after it:
    a model compiled with --enable-fast-math --disable-quantization-zero-point
    (mode 3 in front of each of its ops) followed on the same thread by a model
    compiled with default options (which calls nothing) gets the default
    lowering's bits (src/Compiler/CompilerPasses.cpp:298-301: the form is a
    property of the compiled model).  Straight through the C entry points, as
    generated code calls them, without touching the mode in between."""
    lib = rt.load()
    assert rt.quant_mode() == 0 and rt.pending_quant_mode() == 0
    rng = np.random.default_rng(31)
    sep = np.arange(1, 1601, dtype=np.float32) * np.float32(0.15)   # x / 0.3 and x * (1 / 0.3) differ here
    x = np.concatenate([sep, rng.normal(0, 40, 70000).astype(np.float32)])
    scale, zp = np.float32(0.3), np.array(7, np.uint8)
    want3 = oracle.quantize_linear_mode(x, scale, zp, 3)
    want0 = oracle.quantize_linear(x, scale, zp)
    assert (want3 != want0).any()
    dX, dS, dZ = (rt.DeviceArray.from_numpy(np.asarray(a)) for a in (x, scale, zp))
    dQ = rt.DeviceArray(x.shape, np.uint8)
    dD = rt.DeviceArray(x.shape, np.float32)
    dys, dyz = rt.DeviceArray((), np.float32), rt.DeviceArray((), np.uint8)
    quantize = rt.PreparedCall("om_mi355x_QuantizeLinear", dQ, dX, dS, dZ, 1, 1)
    dequantize = rt.PreparedCall("om_mi355x_DequantizeLinear", dD, dQ, dS, dZ, 1)
    dynamic = rt.PreparedCall("om_mi355x_DynamicQuantizeLinear", dQ, dys, dyz, dX)
    W = _rand_q(rng, np.int8, (64, 48))
    xs = rng.uniform(-3, 5, (40, 64)).astype(np.float32)
    dXs, dW = rt.DeviceArray.from_numpy(xs), rt.DeviceArray.from_numpy(W)
    dbs = rt.DeviceArray.from_numpy(np.array(0.01, np.float32))
    dY = rt.DeviceArray((40, 48), np.float32)
    fused = rt.PreparedCall("om_mi355x_DynQuantMatMulDequant", dY, dXs, dW, None, dbs, None, 0)

    def set_mode(m):
        lib.om_mi355x_SetQuantMode(None, ctypes.c_int64(m))

    # the first model: mode 3 in front of the op
    set_mode(3)
    assert rt.pending_quant_mode() == 3
    quantize()
    assert rt.pending_quant_mode() == 0
    rt.synchronize()
    assert np.array_equal(dQ.numpy(), want3)
    # the second model: the same op with nothing in front of it
    quantize()
    rt.synchronize()
    assert np.array_equal(dQ.numpy(), want0)
    # the same for the other consumers; an op of another kind in between (a
    # matmul) neither takes the mode nor clears it
    q = want0
    set_mode(2)
    rt.MatMulInteger(_rand_q(rng, np.uint8, (4, 16)), _rand_q(rng, np.int8, (16, 8)))
    assert rt.pending_quant_mode() == 2
    dequantize()
    dequantize_default = oracle.dequantize_linear(q, scale, zp)
    rt.synchronize()
    assert np.array_equal(bits(dD.numpy()), bits(oracle.dequantize_linear(q, scale, None)))
    dequantize()
    rt.synchronize()
    assert np.array_equal(bits(dD.numpy()), bits(dequantize_default))
    for mode in (1, 2, 3):
        wy, ws, wz = oracle.dynamic_quantize_linear_mode(x, mode)
        set_mode(mode)
        dynamic()
        rt.synchronize()
        assert np.array_equal(dQ.numpy(), wy) and dys.numpy() == ws and dyz.numpy() == wz, mode
        wy, ws, wz = oracle.dynamic_quantize_linear(x)
        dynamic()
        rt.synchronize()
        assert np.array_equal(dQ.numpy(), wy) and dys.numpy() == ws and dyz.numpy() == wz, mode
        aq, a_s, a_z = oracle.dynamic_quantize_linear_mode(xs, mode)
        set_mode(mode)
        fused()
        rt.synchronize()
        want = oracle.dequant_epilogue(oracle.matmul_integer(aq, W, a_z, None), a_s, np.float32(0.01))
        assert np.array_equal(bits(dY.numpy()), bits(want)), mode
        aq, a_s, a_z = oracle.dynamic_quantize_linear(xs)
        fused()
        rt.synchronize()
        want = oracle.dequant_epilogue(oracle.matmul_integer(aq, W, a_z, None), a_s, np.float32(0.01))
        assert np.array_equal(bits(dY.numpy()), bits(want)), mode
    # an op that fails its checks still takes the mode with it
    set_mode(1)
    bad = rt.PreparedCall("om_mi355x_QuantizeLinear", dD, dX, dS, dZ, 1, 1)      # f32 output: refused
    bad()
    with pytest.raises(rt.RuntimeError_):
        bad.check()
    assert rt.pending_quant_mode() == 0
    # a value outside 0..3 is refused and changes nothing
    set_mode(2)
    set_mode(4)
    with pytest.raises(rt.RuntimeError_, match="SetQuantMode"):
        quantize.check()
    assert rt.pending_quant_mode() == 2
    set_mode(0)
    for f in (quantize, dequantize, dynamic, fused, bad):
        f.close()
    for d in (dX, dS, dZ, dQ, dD, dys, dyz, dXs, dW, dbs, dY):
        d.free()


@pytest.mark.parametrize("forced", [True, False])
def test_weights_in_registers_kernel_stays_inside_a_ragged_output(rt, oracle, forced, monkeypatch):
    """k_gemm_i8_wreg drops the rows of its last 32-row tiles that lie past M
    through the range check of its buffer stores.  The output is placed inside
    a larger GPU buffer filled with a sentinel: 40 rows' worth of it before and
    after must come back untouched, for the int32 and the f32 epilogue, whatever
    the remainder M % 32 is."""
    if forced:
        monkeypatch.setenv("OM_MI355X_GEMM_TILE", "4")
        shapes = [(17, 32), (30, 64), (129, 416), (131, 384), (300, 800), (1000, 416), (333, 896)]
    else:
        shapes = [(4001, 2304), (4065, 3072), (4095, 3072)]
    rng = np.random.default_rng(4242 + forced)
    K = 768
    for M, N in shapes:
        A, B = _rand_q(rng, np.uint8, (M, K)), _rand_q(rng, np.int8, (K, N))
        az = _rand_q(rng, np.uint8, ())
        acc = oracle.matmul_integer(A, B, az, None)
        guard = 40 * N
        for epi in ("i32", "f32"):
            fill = np.full(guard + M * N + guard, 0x5A5A5A5A, np.uint32)
            buf = rt.DeviceArray.from_numpy(fill.view(np.int32 if epi == "i32" else np.float32))
            y = rt.DeviceArray.view_of(buf, guard, (M, N))
            if epi == "i32":
                rt.MatMulInteger(A, B, az, None, out=y)
                want = acc.view(np.uint32)
            else:
                bs = rng.uniform(1e-3, 1e-2, N).astype(np.float32)
                rt.MatMulIntegerDequant(A, B, az, None, np.float32(0.0173), bs, None, out=y)
                want = bits(oracle.dequant_epilogue(acc, np.float32(0.0173), bs))
            assert "wreg" in rt.last_gemm_kernel(), (M, N, rt.last_gemm_kernel())
            rt.synchronize()
            whole = buf.numpy().view(np.uint32)
            assert (whole[:guard] == 0x5A5A5A5A).all(), (M, N, epi, "before")
            assert (whole[guard + M * N:] == 0x5A5A5A5A).all(), (M, N, epi, "after")
            assert np.array_equal(whole[guard:guard + M * N].reshape(M, N), want), (M, N, epi)
            buf.free()
        if N % 128:
            continue
        # 8-bit results, gathered in LDS and stored 16 bytes a lane
        bz0 = np.zeros((), np.int8)
        a_s, b_s, y_s, yz = np.float32(0.0173), np.float32(0.004), np.float32(0.08), np.uint8(131)
        want = oracle.qlinear_matmul(A, a_s, az, B, b_s, bz0, y_s, yz, oracle_lib.SATURATE)
        buf = rt.DeviceArray.from_numpy(np.full(guard + M * N + guard, 0x5A, np.uint8))
        y = rt.DeviceArray.view_of(buf, guard, (M, N))
        rt.QLinearMatMul(A, a_s, az, B, b_s, bz0, y_s, yz, rt.SATURATE, out=y)
        assert "wreg" in rt.last_gemm_kernel(), (M, N, rt.last_gemm_kernel())
        rt.synchronize()
        whole = buf.numpy()
        assert (whole[:guard] == 0x5A).all(), (M, N, "q8", "before")
        assert (whole[guard + M * N:] == 0x5A).all(), (M, N, "q8", "after")
        assert np.array_equal(whole[guard:guard + M * N].reshape(M, N), want), (M, N, "q8")
        buf.free()


def test_dispatch_keeps_bs_to_whole_trips(rt, oracle):
    """k_gemm_i8_bs runs four K steps per trip of its loop; the dispatch gives it
    only products whose K is a multiple of 256 (the step counts it is validated
    at).  4096 x 1088 x 4096 -- 17 steps, the launch that once ended a benchmark
    loop with an illegal memory access (tests/test_bs_address_model.py) -- takes
    the 128 x 128 tiles of k_gemm_i8_dma instead and matches the oracle; the
    same product over K = 1024 still takes k_gemm_i8_bs."""
    rng = np.random.default_rng(1088)
    A = rng.integers(0, 256, (4096, 1088), dtype=np.uint8)
    B = rng.integers(-128, 128, (1088, 4096), dtype=np.int8)
    az = np.uint8(129)
    print("dispatch test: 4096x1088x4096", flush=True)
    got = rt.MatMulInteger(A, B, az, None)
    assert rt.last_gemm_kernel() == "k_gemm_i8_dma (128x128 tiles)", rt.last_gemm_kernel()
    assert np.array_equal(got, oracle.matmul_integer(A, B, az, None, passes=True))
    got = rt.MatMulInteger(A[:, :1024], B[:1024], az, None)
    assert rt.last_gemm_kernel() == "k_gemm_i8_bs (128x256 tiles)", rt.last_gemm_kernel()
    assert np.array_equal(got, oracle.matmul_integer(np.ascontiguousarray(A[:, :1024]), np.ascontiguousarray(B[:1024]), az, None, passes=True))
