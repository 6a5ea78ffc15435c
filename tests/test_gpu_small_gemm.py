"""Parity of k_gemm_i8_flight -- the kernel for products that one round of
blocks covers (K = 512, 768 or 1024), and the dynamically quantized layer in
one launch -- with the CPU oracle, through the C-ABI.  Bit-exact, fp32
included (same sequence of correctly rounded operations)."""
import numpy as np
import pytest

import oracle_lib
from om_mi355x import workloads as wl

pytestmark = pytest.mark.gpu


def _rand_q(rng, dt, shape):
    info = np.iinfo(dt)
    return rng.integers(info.min, info.max + 1, shape, dtype=dt)


def bits(a):
    return np.ascontiguousarray(a).view(np.uint32)


def same_f32(a, b):
    a, b = np.asarray(a, np.float32), np.asarray(b, np.float32)
    return a.shape == b.shape and bool(np.all((bits(a) == bits(b)) | (np.isnan(a) & np.isnan(b))))


def mm(oracle, A, B, a_zp, b_zp):
    """The oracle's MatMulInteger; large products through its OpenMP restatement
    of the reference's passes (pinned to the triple loop in test_oracle.py)."""
    big = A.shape[0] * A.shape[1] * B.shape[1] > 1 << 27
    return oracle.matmul_integer(A, B, a_zp, b_zp, passes=big)


SHAPES = [(65, 512, 100), (128, 768, 768), (200, 1024, 1000), (512, 1024, 4096), (1000, 768, 416),
          (2048, 768, 256), (97, 768, 33), (1000, 512, 1024), (256, 1024, 2048)]


@pytest.mark.parametrize("M,K,N", SHAPES)
def test_one_round_kernel_all_operand_types_and_epilogues(rt, oracle, M, K, N):
    """Every pair of operand types, zero points absent / scalar / per row and per
    column, and the three epilogues (int32; f32 with per-column scale, bias and
    Relu; 8-bit requantize, wrapping and saturating) on shapes with ragged edges
    in both directions that the dispatch gives to k_gemm_i8_flight."""
    rng = np.random.default_rng(M * 7 + K + N)
    for adt, bdt in ((np.uint8, np.int8), (np.int8, np.uint8), (np.uint8, np.uint8), (np.int8, np.int8)):
        A, B = _rand_q(rng, adt, (M, K)), _rand_q(rng, bdt, (K, N))
        az, bz = _rand_q(rng, adt, (M,)), _rand_q(rng, bdt, (N,))
        for a_zp, b_zp in ((None, None), (az[:1], None), (az[:1], bz[:1]), (az, bz)):
            want = mm(oracle, A, B, a_zp, b_zp)
            got = rt.MatMulInteger(A, B, a_zp, b_zp)
            # (one zero point per row of A is left to the other kernels)
            assert ("flight" in rt.last_gemm_kernel()) == (a_zp is None or a_zp.size == 1), rt.last_gemm_kernel()
            assert np.array_equal(got, want), (adt, bdt, a_zp is not None, b_zp is not None)
        acc = mm(oracle, A, B, az[:1], bz[:1])
        a_s = np.float32(0.0173)
        bs = rng.uniform(1e-3, 1e-2, N).astype(np.float32)
        bias = rng.normal(0, 2, N).astype(np.float32)
        want = oracle.dequant_epilogue(acc, a_s, bs) + bias
        assert same_f32(rt.MatMulIntegerDequant(A, B, az[:1], bz[:1], a_s, bs, bias), want)
        assert same_f32(rt.MatMulIntegerDequant(A, B, az[:1], bz[:1], a_s, bs, bias, activation=1),
                        np.fmax(want, np.float32(0)))
        assert "flight" in rt.last_gemm_kernel()
        if adt == bdt:
            ys = np.float32(0.37)
            yz = _rand_q(rng, adt, ())
            for mode, omode in ((rt.WRAP, oracle_lib.WRAP), (rt.SATURATE, oracle_lib.SATURATE)):
                want = oracle.qlinear_matmul(A, a_s, az[:1], B, np.float32(0.005), bz[:1], ys, yz, omode)
                got = rt.QLinearMatMul(A, a_s, az[:1], B, np.float32(0.005), bz[:1], ys, yz, mode)
                assert "flight" in rt.last_gemm_kernel()
                assert np.array_equal(got, want), (adt, mode)


def test_one_round_kernel_is_forced_and_falls_through(rt, oracle, monkeypatch):
    """OM_MI355X_GEMM_TILE=5 names the kernel; a shape it does not take (K no
    multiple of 256, more blocks than one round) still computes, with another
    kernel."""
    monkeypatch.setenv("OM_MI355X_GEMM_TILE", "5")
    rng = np.random.default_rng(55)
    for (M, K, N), mine in (((300, 768, 500), True), ((300, 704, 500), False), ((8192, 768, 3072), False)):
        A, B = _rand_q(rng, np.uint8, (M, K)), _rand_q(rng, np.int8, (K, N))
        az = _rand_q(rng, np.uint8, ())
        assert np.array_equal(rt.MatMulInteger(A, B, az, None), mm(oracle, A, B, az, None)), (M, K, N)
        assert ("flight" in rt.last_gemm_kernel()) == mine, (M, K, N, rt.last_gemm_kernel())


@pytest.mark.parametrize("M,K,N", [(33, 768, 768), (128, 768, 768), (100, 512, 200), (512, 1024, 1024), (65, 1024, 97),
                                   (1024, 768, 768), (2048, 512, 100), (40, 768, 3072)])
def test_dynamically_quantized_layer_in_one_launch(rt, oracle, M, K, N):
    """DynamicQuantizeLinear -> MatMulInteger -> Cast -> Mul (-> Add -> Relu) as
    one launch of k_gemm_i8_flight: the blocks agree on minimum and maximum
    through the exchange slots, every block quantizes its own 32 rows.  Against
    the oracle's chain of the separate ops, bit for bit; host and GPU-resident
    operands; signed and unsigned weights, weight zero points; inputs whose
    minimum or maximum sits in the last (ragged) row block, NaN and infinities
    among the activations."""
    rng = np.random.default_rng(M + K * 3 + N)
    x = rng.normal(0, 1, (M, K)).astype(np.float32)
    x[M - 1, K - 1] = 7.5            # the maximum in the last row
    x[0, 0] = -6.25
    for bdt in (np.int8, np.uint8):
        W = _rand_q(rng, bdt, (K, N))
        ws = rng.uniform(1e-3, 1e-2, N).astype(np.float32)
        bias = rng.normal(0, 1, N).astype(np.float32)
        bz = _rand_q(rng, bdt, (N,))
        aq, a_s, a_zp = oracle.dynamic_quantize_linear(x)
        for b_zp in (None, bz[:1], bz):
            acc = mm(oracle, aq, W, a_zp, b_zp)
            want = oracle.dequant_epilogue(acc, a_s, ws)
            got = rt.DynQuantMatMulDequant(x, W, b_zp, ws)
            assert "flight (rows quantized" in rt.last_gemm_kernel(), rt.last_gemm_kernel()
            assert same_f32(got, want), (bdt, b_zp is not None)
        wantb = np.fmax(oracle.dequant_epilogue(mm(oracle, aq, W, a_zp, None), a_s, ws[:1]) + bias,
                        np.float32(0))
        assert same_f32(rt.DynQuantMatMulDequant(x, W, None, ws[:1], bias, activation=1), wantb)
    # GPU-resident operands, called repeatedly (the launch number in the slots moves on)
    dX, dW, dS = rt.DeviceArray.from_numpy(x), rt.DeviceArray.from_numpy(W), rt.DeviceArray.from_numpy(ws)
    dY = rt.DeviceArray((M, N), np.float32)
    rt.mark_constant(dW)
    acc = mm(oracle, aq, W, a_zp, None)
    want = oracle.dequant_epilogue(acc, a_s, ws)
    for _ in range(5):
        rt.DynQuantMatMulDequant(dX, dW, None, dS, out=dY)
    rt.synchronize()
    assert same_f32(dY.numpy(), want)
    rt.unmark_constant(dW)
    for d in (dX, dW, dS, dY):
        d.free()
    # special values: NaN is ignored by the minimum / maximum and quantizes to
    # the lower bound, infinities saturate (and make the scale infinite)
    x2 = x.copy()
    x2[3, 5] = np.nan
    aq, a_s, a_zp = oracle.dynamic_quantize_linear(x2)
    W = _rand_q(rng, np.int8, (K, N))
    want = oracle.dequant_epilogue(mm(oracle, aq, W, a_zp, None), a_s, ws)
    assert same_f32(rt.DynQuantMatMulDequant(x2, W, None, ws), want)
    x2[M // 2, 7] = np.inf
    aq, a_s, a_zp = oracle.dynamic_quantize_linear(x2)
    want = oracle.dequant_epilogue(mm(oracle, aq, W, a_zp, None), a_s, ws)
    assert same_f32(rt.DynQuantMatMulDequant(x2, W, None, ws), want)


def test_config1_is_one_launch(rt, oracle):
    c = wl.config1()
    aq, a_s, a_zp = oracle.dynamic_quantize_linear(c["A"])
    want = oracle.dequant_epilogue(oracle.matmul_integer(aq, c["B"], a_zp, c["b_zp"]), a_s, c["b_scale"])
    assert same_f32(rt.DynQuantMatMulDequant(c["A"], c["B"], c["b_zp"], c["b_scale"]), want)
    assert rt.last_gemm_kernel() == "k_gemm_i8_flight (rows quantized in the kernel)"


@pytest.mark.parametrize("mode", [0, 1])
def test_fused_layer_takes_an_activation_that_is_not_16_byte_aligned(rt, oracle, mode):
    """A GPU-resident activation that starts 4 bytes into its buffer (a view):
    the one-launch kernels want 16-byte rows, so the layer runs as
    DynamicQuantizeLinear + GEMM, whose quantize pass then stores the rows minus
    128 with a kernel that takes any alignment -- also when the quotient is
    computed as x * (1 / scale) (mode 1), where this used to be refused."""
    M, K, N = 72, 768, 256
    rng = np.random.default_rng(72 + mode)
    x = rng.normal(0, 1, (M, K)).astype(np.float32)
    W = _rand_q(rng, np.int8, (K, N))
    ws = rng.uniform(1e-3, 1e-2, N).astype(np.float32)
    buf = rt.DeviceArray.from_numpy(np.concatenate([np.zeros(1, np.float32), x.ravel()]))
    dx = rt.DeviceArray.__new__(rt.DeviceArray)
    dx.shape, dx.dtype, dx.ptr, dx.owner = (M, K), np.dtype(np.float32), buf.ptr + 4, buf
    aq, a_s, a_zp = oracle.dynamic_quantize_linear_mode(x, mode)
    want = oracle.dequant_epilogue(mm(oracle, aq, W, a_zp, None), a_s, ws)
    rt.set_quant_mode(mode)  # (what a model compiled with that option emits in front of each op)
    try:
        got = rt.DynQuantMatMulDequant(dx, W, None, ws)
    finally:
        rt.set_quant_mode(0)
    got = got.numpy() if hasattr(got, "numpy") else got
    assert "flight (rows quantized" not in rt.last_gemm_kernel()
    assert same_f32(got, want)
    buf.free()


def test_qlinear_matmul_with_a_scale_per_column(rt, oracle):
    """b_scale as one value per column of B (what a QDQ model with per-channel
    weights recomposes to).  PARITY UNPINNED against the reference, whose
    lowering refuses this form (QLinearMatMul.cpp:53-68): the expected values
    are its expression (:127-138) with column j's scale -- f32(acc) * ((a_scale
    * b_scale[j]) / y_scale), roundEven, + y_zp, narrowed -- over the oracle's
    exact int32 product, restated here in numpy; with all columns' scales equal
    that restatement is checked against the oracle's own QLinearMatMul first."""
    rng = np.random.default_rng(4242)

    def expect(A, a_s, az, B, bs, bz, y_s, yz, saturate):
        acc = mm(oracle, A, B, az, bz)
        s = (np.float32(a_s) * bs.astype(np.float32)) / np.float32(y_s)
        q = np.rint(acc.astype(np.float32) * s[None, :]).astype(np.int64) + int(yz)
        info = np.iinfo(yz.dtype)
        if saturate:
            return np.clip(q, info.min, info.max).astype(yz.dtype)
        return (q & 0xFF).astype(np.uint8).view(yz.dtype) if yz.dtype == np.int8 else (q & 0xFF).astype(np.uint8)

    for (M, K, N), adt in (((200, 1024, 1000), np.uint8), ((300, 768, 384), np.int8), ((48, 200, 130), np.uint8),
                            ((1024, 768, 3072), np.uint8)):
        A, B = _rand_q(rng, adt, (M, K)), _rand_q(rng, np.int8, (K, N))
        az, yz = _rand_q(rng, adt, ()), _rand_q(rng, adt, ())
        bz = _rand_q(rng, np.int8, (N,)) if M != 1024 else np.zeros(N, np.int8)
        a_s, y_s = np.float32(0.0173), np.float32(0.11)
        same = np.full(N, 0.004, np.float32)
        for sat, omode, mode in ((False, oracle_lib.WRAP, rt.WRAP), (True, oracle_lib.SATURATE, rt.SATURATE)):
            assert np.array_equal(expect(A, a_s, az, B, same, bz, y_s, yz, sat),
                                  oracle.qlinear_matmul(A, a_s, az, B, same[0], bz, y_s, yz, omode))
            bs = rng.uniform(1e-3, 8e-3, N).astype(np.float32)
            got = rt.QLinearMatMul(A, a_s, az, B, bs, bz, y_s, yz, mode)
            assert np.array_equal(got, expect(A, a_s, az, B, bs, bz, y_s, yz, sat)), (M, K, N, sat, rt.last_gemm_kernel())


def _limits(a):
    a = np.asarray(a, np.float32)
    return np.array([np.fmin.reduce(a, axis=None), np.fmax.reduce(a, axis=None)], np.float32)


@pytest.mark.parametrize("M,K,N,N2", [(128, 768, 3072, 768), (4096, 768, 3072, 768), (16, 4096, 1024, 512),
                                      # ragged rows and a last column tile past N in the weights-in-registers kernel
                                      (2945, 768, 3040, 416),
                                      (33, 200, 130, 70), (300, 768, 1000, 416), (2, 64, 8, 5),
                                      # second layer quantized inside its kernel: one round of blocks; every block for itself
                                      (128, 768, 1024, 768), (200, 512, 768, 1000), (8, 1024, 2048, 512), (16, 512, 2048, 11008)])
def test_chain_of_layers_hands_the_limits_on(rt, oracle, M, K, N, N2):
    """om_mi355x_DynQuantMatMulDequantLimits: y_limits of a layer is minimum and
    maximum of its result (NaN ignored), bit for bit what numpy finds in it,
    whatever kernel produced y (in its epilogue, or a pass over y behind it) and
    with bias, Relu or Gelu applied; a second layer given them as x_limits
    returns exactly what it returns without them, and what the oracle's chain of
    the separate ops gives.  Host and GPU-resident tensors."""
    rng = np.random.default_rng(M + N)
    x = rng.normal(0, 1, (M, K)).astype(np.float32)
    W1, W2 = _rand_q(rng, np.int8, (K, N)), _rand_q(rng, np.int8, (N, N2))
    s1 = rng.uniform(1e-3, 1e-2, N).astype(np.float32)
    s2 = rng.uniform(1e-3, 1e-2, N2).astype(np.float32)
    bias = rng.normal(0, 1, N).astype(np.float32)
    for act in (0, 1, 2):
        h_plain = rt.DynQuantMatMulDequant(x, W1, None, s1, bias, activation=act)
        h, hl = rt.DynQuantMatMulDequantLimits(x, W1, None, s1, bias, activation=act)
        assert same_f32(h, h_plain), (act, rt.last_gemm_kernel())
        assert same_f32(hl, _limits(h)), (act, hl, _limits(h), rt.last_gemm_kernel())
        y_plain = rt.DynQuantMatMulDequant(h, W2, None, s2)
        kernel = rt.last_gemm_kernel()
        y, yl = rt.DynQuantMatMulDequantLimits(h, W2, None, s2, x_limits=hl)
        assert rt.last_gemm_kernel() == kernel  # (known limits do not change the kernel)
        assert same_f32(y, y_plain), (act, kernel)
        assert same_f32(yl, _limits(y))
        if act != 2:  # (the oracle's Gelu differs from the kernel's in the last bits)
            aq, a_s, a_zp = oracle.dynamic_quantize_linear(h)
            assert same_f32(y, oracle.dequant_epilogue(mm(oracle, aq, W2, a_zp, None), a_s, s2))
    # GPU-resident, the limits never leave the GPU
    dx, dW1, dW2, ds1, ds2 = (rt.DeviceArray.from_numpy(v) for v in (x, W1, W2, s1, s2))
    dh, dhl = rt.DeviceArray((M, N), np.float32), rt.DeviceArray((2,), np.float32)
    dy = rt.DeviceArray((M, N2), np.float32)
    for _ in range(3):
        rt.DynQuantMatMulDequantLimits(dx, dW1, None, ds1, None, out=dh, activation=1, y_limits=dhl)
        rt.DynQuantMatMulDequantLimits(dh, dW2, None, ds2, None, out=dy, x_limits=dhl, want_limits=False)
    rt.synchronize()
    h = rt.DynQuantMatMulDequant(x, W1, None, s1, None, activation=1)
    assert same_f32(dh.numpy(), h) and same_f32(dhl.numpy(), _limits(h))
    assert same_f32(dy.numpy(), rt.DynQuantMatMulDequant(h, W2, None, s2))
    for d in (dx, dW1, dW2, ds1, ds2, dh, dhl, dy):
        d.free()


def test_limits_with_nan_infinities_and_the_other_quotient(rt, oracle):
    """NaN in the result is ignored by the limits (as the reductions of
    DynamicQuantizeLinear ignore it), infinities are not; limits handed to a
    layer under SetQuantMode(1) and (2) give what that mode gives without them;
    limits of the wrong size are refused."""
    rng = np.random.default_rng(99)
    M, K, N = 70, 320, 96
    x = rng.normal(0, 1, (M, K)).astype(np.float32)
    W = _rand_q(rng, np.int8, (K, N))
    s = rng.uniform(1e-3, 1e-2, N).astype(np.float32)
    bias = rng.normal(0, 1, N).astype(np.float32)
    bias[5], bias[9] = np.nan, np.inf
    h, hl = rt.DynQuantMatMulDequantLimits(x, W, None, s, bias)
    assert np.isnan(h[:, 5]).all() and same_f32(hl, _limits(h)) and hl[1] == np.inf
    bias[9] = 1.0
    h, hl = rt.DynQuantMatMulDequantLimits(x, W, None, s, bias)
    assert np.isfinite(hl).all() and same_f32(hl, _limits(h))
    W2 = _rand_q(rng, np.int8, (N, 40))
    s2 = rng.uniform(1e-3, 1e-2, 40).astype(np.float32)
    h = np.nan_to_num(h, nan=0.25)
    hl = _limits(h)
    try:
        for mode in (1, 2, 3):
            rt.set_quant_mode(mode)
            want = rt.DynQuantMatMulDequant(h, W2, None, s2)
            got, _ = rt.DynQuantMatMulDequantLimits(h, W2, None, s2, x_limits=hl, want_limits=False)
            assert same_f32(got, want), mode
            aq, a_s, a_zp = oracle.dynamic_quantize_linear_mode(h, mode)
            assert same_f32(got, oracle.dequant_epilogue(mm(oracle, aq, W2, a_zp, None), a_s, s2)), mode
    finally:
        rt.set_quant_mode(0)
    with pytest.raises(rt.RuntimeError_, match="limits"):
        rt.DynQuantMatMulDequantLimits(h, W2, None, s2, x_limits=np.zeros(3, np.float32))
